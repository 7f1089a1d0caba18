"""A plain, slow forward pass of the Kegozen design: whole sequences, no cache, no paging, one function per
mechanism, float64 torch on the CPU.  It shares no code with the engine: it reads a model folder with ``json`` and
the ``safetensors`` package and writes every sum as a loop or a dense matrix expression.

The design in short (x_t is the residual stream of token t, positions p count from 0):

* x_t = embed[tok_t]; a layer: x <- x + n1b(mixer(n1(x))); x <- x + n2b(ff(n2(x))); every n is
  x / sqrt(mean x^2 + eps) * (1 + g).
* mixer "mamba2": (z | u | B | C | dt) = W_in h; u, B, C pass a causal convolution over time (per channel, with a
  bias) and silu; dt <- softplus(dt + dt_bias); per head S_t = exp(-exp(A_log) dt_t) S_{t-1} + dt_t B_t u_t^T,
  y_t = S_t^T C_t + D u_t; the heads side by side are multiplied by silu(z), RMS-normed in equal parts (a gain per
  channel) and projected.
* mixer "attention": grouped-query softmax attention; q and k are RMS-normed per head (one gain vector for all
  heads), the first rot.dims dims of each head turn as neighbouring pairs (2i, 2i+1) with frequencies that may be
  stretched for long wavelengths (and a magnitude on cos and sin); values turn by their own position over all their
  dims, and a head's output turns back by the query's position; a query sees the last ``size`` positions and, of the
  positions before those, one mean key and mean value for every whole block of ``pool`` positions.
* mixer "latent_attention": q = W_uq rms(W_dq h); (c | kr) = W_dkv h, c RMS-normed; per head the key is
  (W_uk c | kr turned), the value W_uv c; the turned part pairs dim i with i + rot_dim/2; causal over all positions.
* ff: down(silu(gate h) * up h); or a mixture: sigmoid scores of a router, the ``top`` largest choose experts, each
  runs on (score * h), plus a shared expert times sigmoid(w_sg . h); or none.
* logits = head n_final(x).
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import torch

F = torch.float64


# --------------------------------------------------------------------------
# mechanisms
# --------------------------------------------------------------------------
def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def one_plus_norm(x: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    return rms(x, eps) * (1.0 + g)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def causal_convolution(u: torch.Tensor, taps: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """u [T, C]; taps [C, K], the last column weighs the present token; zeros before the start."""
    T, C = u.shape
    K = taps.shape[1]
    out = torch.zeros((T, C), dtype=F)
    for t in range(T):
        acc = bias.clone()
        for j in range(K):
            s = t - (K - 1 - j)
            if s >= 0:
                acc = acc + taps[:, j] * u[s]
        out[t] = acc
    return out


def state_space_head(u, B, C, dt, a_log: float, d_skip: float) -> torch.Tensor:
    """One head.  u [T, vdim], B, C [T, N], dt [T].  S_t = exp(-exp(a_log) dt_t) S_{t-1} + dt_t B_t u_t^T;
    y_t = S_t^T C_t + d_skip u_t."""
    T, N = B.shape
    S = torch.zeros((N, u.shape[1]), dtype=F)
    y = torch.zeros_like(u)
    for t in range(T):
        S = math.exp(-math.exp(a_log) * float(dt[t])) * S + float(dt[t]) * torch.outer(B[t], u[t])
        y[t] = S.T @ C[t] + d_skip * u[t]
    return y


def mamba2(h: torch.Tensor, w: Dict[str, torch.Tensor], m, eps: float) -> torch.Tensor:
    heads, vdim, N, G, parts = (int(m[k]) for k in ("heads", "vdim", "state", "groups", "norm_groups"))
    inner, T = heads * vdim, h.shape[0]
    p = h @ w["in"].T
    z, rest, dt = p[:, :inner], p[:, inner:2 * inner + 2 * G * N], p[:, 2 * inner + 2 * G * N:]
    rest = silu(causal_convolution(rest, w["conv"], w["conv.b"]))
    u = rest[:, :inner].reshape(T, heads, vdim)
    B = rest[:, inner:inner + G * N].reshape(T, G, N)
    C = rest[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + w["dt_bias"])
    y = torch.zeros((T, heads, vdim), dtype=F)
    for a in range(heads):
        g = a // (heads // G)
        y[:, a] = state_space_head(u[:, a], B[:, g], C[:, g], dt[:, a], float(w["A_log"][a]), float(w["D"][a]))
    y = y.reshape(T, inner) * silu(z)
    y = rms(y.reshape(T, parts, inner // parts), eps).reshape(T, inner) * w["norm"]
    return y @ w["o"].T


def pair_frequencies(dims: int, base: float, scaling=None):
    """(frequency of pair i, magnitude of cos and sin)."""
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def dim_of(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(scaling["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def turn(x: torch.Tensor, positions: Sequence[float], freqs: Sequence[float], layout: str, mag: float = 1.0) -> torch.Tensor:
    """x [T, heads, d]: the first 2 * len(freqs) dims of every head turn; pair i is (2i, 2i+1) ("interleaved") or
    (i, i + len(freqs)) ("halves")."""
    out = x.clone()
    n = len(freqs)
    for t, p in enumerate(positions):
        for i, fr in enumerate(freqs):
            a, b = (2 * i, 2 * i + 1) if layout == "interleaved" else (i, i + n)
            c, s = math.cos(p * fr) * mag, math.sin(p * fr) * mag
            out[t, :, a] = x[t, :, a] * c - x[t, :, b] * s
            out[t, :, b] = x[t, :, b] * c + x[t, :, a] * s
    return out


def pooled_window_softmax(q, k, v, scale: float, size: int, pool: int) -> torch.Tensor:
    """One head.  q, k [T, d], v [T, vd].  Query i sees j with 0 <= i - j < size and the mean key / mean value of
    every block [bP, bP + P) with bP + P - 1 <= i - size."""
    T = q.shape[0]
    out = torch.zeros((T, v.shape[1]), dtype=F)
    for i in range(T):
        keys, vals = [], []
        if pool > 0 and size > 0:
            b = 0
            while b * pool + pool - 1 <= i - size:
                keys.append(k[b * pool:(b + 1) * pool].mean(dim=0))
                vals.append(v[b * pool:(b + 1) * pool].mean(dim=0))
                b += 1
        for j in range(i + 1):
            if size <= 0 or i - j < size:
                keys.append(k[j])
                vals.append(v[j])
        s = torch.stack(keys) @ q[i] * scale
        pr = torch.softmax(s, dim=0)
        out[i] = pr @ torch.stack(vals)
    return out


def attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m, eps: float, round_cache=None) -> torch.Tensor:
    H, G, d, vd = (int(m[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
    T = h.shape[0]
    q = (h @ w["q"].T).reshape(T, H, d)
    k = (h @ w["k"].T).reshape(T, G, d)
    v = (h @ w["v"].T).reshape(T, G, vd)
    if "q.norm" in w:
        q = rms(q, eps) * w["q.norm"]
        k = rms(k, eps) * w["k.norm"]
    rot = m.get("rot")
    pos = list(range(T))
    if rot:
        freqs, mag = pair_frequencies(int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
        q = turn(q, pos, freqs, "interleaved", mag)
        k = turn(k, pos, freqs, "interleaved", mag)
        vf, _ = pair_frequencies(vd, float(rot["base"]))
        v = turn(v, pos, vf, "interleaved")
    if round_cache is not None:
        k, v = round_cache(k), round_cache(v)
    mask = m.get("mask") or {}
    size, pool = int(mask.get("size", 0) or 0), int(mask.get("pool", 0) or 0)
    o = torch.zeros((T, H, vd), dtype=F)
    for a in range(H):
        g = a // (H // G)
        o[:, a] = pooled_window_softmax(q[:, a], k[:, g], v[:, g], float(m["scale"]), size, pool)
    if rot:
        o = turn(o, [-p for p in pos], vf, "interleaved")
    return o.reshape(T, H * vd) @ w["o"].T


def latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m, eps: float) -> torch.Tensor:
    H, d, r, vd, rank = (int(m[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
    T = h.shape[0]
    if "dq" in w:
        cq = rms(h @ w["dq"].T, eps) * w["dq.norm"]
        q = (cq @ w["uq"].T).reshape(T, H, d + r)
    else:
        q = (h @ w["q"].T).reshape(T, H, d + r)
    dkv = h @ w["dkv"].T
    c = rms(dkv[:, :rank], eps) * w["dkv.norm"]
    kr = dkv[:, rank:].reshape(T, 1, r)
    freqs, _ = pair_frequencies(int(m["rot"]["dims"]), float(m["rot"]["base"]))
    pos = list(range(T))
    q_rot = turn(q[:, :, d:].contiguous(), pos, freqs, "halves")
    kr = turn(kr, pos, freqs, "halves")[:, 0]
    kp = (c @ w["uk"].T).reshape(T, H, d)
    v = (c @ w["uv"].T).reshape(T, H, vd)
    o = torch.zeros((T, H, vd), dtype=F)
    for a in range(H):
        s = (q[:, a, :d] @ kp[:, a].T + q_rot[:, a] @ kr.T) * float(m["scale"])
        s = s.masked_fill(torch.triu(torch.ones((T, T), dtype=torch.bool), diagonal=1), float("-inf"))
        o[:, a] = torch.softmax(s, dim=1) @ v[:, a]
    return o.reshape(T, H * vd) @ w["o"].T


def gated_expert(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str) -> torch.Tensor:
    return (silu(h @ w[prefix + "gate"].T) * (h @ w[prefix + "up"].T)) @ w[prefix + "down"].T


def feed_forward(h: torch.Tensor, w: Dict[str, torch.Tensor], mlp) -> torch.Tensor:
    if mlp["kind"] == "dense":
        return gated_expert(h, w, "")
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    scores = torch.sigmoid(h @ w["router"].T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: (-float(scores[t, e]), e))[:top]
        for e in order:
            out[t] += gated_expert((scores[t, e] * h[t])[None], w, f"e{e}.")[0]
    if mlp.get("shared"):
        out = out + torch.sigmoid(h @ w["shared.sg"].T) * gated_expert(h, w, "shared.")
    return out


MIXERS = {"mamba2": mamba2, "attention": attention, "latent_attention": latent_attention}


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------
class PlainKegozen:
    def __init__(self, config: dict, tensors: Dict[str, torch.Tensor]):
        self.cfg = config
        self.w = {k: v.to(F) for k, v in tensors.items()}
        self.eps = float(config["norm"]["eps"])

    @classmethod
    def from_folder(cls, folder: str) -> "PlainKegozen":
        from safetensors import safe_open
        with open(os.path.join(folder, "config.json")) as f:
            cfg = json.load(f)
        tensors = {}
        with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
            for name in f.keys():
                tensors[name] = f.get_tensor(name)
        return cls(cfg, tensors)

    def sub(self, prefix: str) -> Dict[str, torch.Tensor]:
        return {k[len(prefix):]: v for k, v in self.w.items() if k.startswith(prefix)}

    def layers_forward(self, tokens: Sequence[int]) -> List[torch.Tensor]:
        """The residual stream after every layer."""
        x = self.w["embed"][list(tokens)].clone()
        out = []
        for i, layer in enumerate(self.cfg["layers"]):
            p = f"l{i}."
            h = one_plus_norm(x, self.w[p + "norm1"], self.eps)
            a = MIXERS[layer["type"]](h, self.sub(p + "mix."), layer["mixer"], self.eps)
            x = x + one_plus_norm(a, self.w[p + "norm1b"], self.eps)
            if layer.get("mlp") is not None:
                h = one_plus_norm(x, self.w[p + "norm2"], self.eps)
                f = feed_forward(h, self.sub(p + "mlp."), layer["mlp"])
                x = x + one_plus_norm(f, self.w[p + "norm2b"], self.eps)
            out.append(x)
        return out

    def logits(self, tokens: Sequence[int]) -> torch.Tensor:
        x = self.layers_forward(tokens)[-1]
        return one_plus_norm(x, self.w["final.norm"], self.eps) @ self.w["head"].T

    forward = logits

    def greedy_generate(self, tokens: Sequence[int], count: int) -> List[int]:
        """``count`` tokens, each the argmax (lowest index among equals) of the logits after all tokens before it."""
        seq, out = list(tokens), []
        for _ in range(count):
            nxt = int(torch.argmax(self.logits(seq)[-1]))
            out.append(nxt)
            seq.append(nxt)
        return out
