"""A plain, slow forward pass of the Tilivik design: whole sequences, no cache, no paging, one function per
mechanism, float64 torch on the CPU.  It shares no code with the engine: it reads a model folder with ``json`` and
the ``safetensors`` package and writes every sum as a loop or a dense matrix expression.

The design in short (x_t is the residual stream of token t, positions p count from 0):

* x_t = embed[tok_t] + bigram[(tok_{t-1} * mul_prev + tok_t * mul_cur) mod buckets] (row ``buckets`` for t = 0)
  + pe(t), pe(p)[2i] = sin(p w_i), pe(p)[2i+1] = cos(p w_i), w_i = 10000^(-2i/width).
* a layer: x <- x + mixer(shift(n1(x))); x <- x + ff(n2(x)); n(x) = x / sqrt(mean x^2 + eps) * g with ONE number g;
  shift(h)_t = h_t + (h_{t-1} - h_t) * s (s per channel, h_{-1} = 0).
* layers [start, stop) run ``times`` times in a row; before pass t > 0 the embedding output is added again, and
  before every pass the row t of ``loop.step``.
* mixer "lightning": per head S_t = c S_{t-1} + k_t v_t^T, o_t = S_t^T q_t with q, k, v = silu(projections) and a
  fixed decay c per head; the concatenated heads are RMS-normed together (gain), gated by sigmoid(W_g h), projected.
* mixer "parallel": a_l * left + a_r * right, both reading the same input.  left: grouped-query softmax attention
  without rotation; values are divided by their root mean square per head; scores are scaled, capped smoothly
  (c tanh(s / c)), and a learned bias by the (log-bucketed) distance is added; a key is visible inside a sliding
  window or among the first few positions; the heads are gated by sigmoid(W_g h).  right: gated linear attention,
  S_t = diag(alpha_t) S_{t-1} + k_t v_t^T, alpha = sigmoid(W_a2 W_a1 h + b)^(1/tau) per key channel, o_t = S_t^T q_t
  with q scaled by dim^-1/2, an RMS norm per head (gain shared by the heads), a silu gate.
* ff: every token id names its ``top`` experts in a table; the result is the mean of those experts' outputs
  down(silu(gate h) * up h).
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


def scalar_norm(x: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose gain is one number for all coordinates."""
    return rms(x, eps) * g.reshape(())


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def position_vectors(T: int, width: int) -> torch.Tensor:
    out = torch.zeros((T, width), dtype=F)
    for p in range(T):
        for c in range(width):
            i = c // 2
            a = p * 10000.0 ** (-2.0 * i / width)
            out[p, c] = math.sin(a) if c % 2 == 0 else math.cos(a)
    return out


def embedding(tokens: Sequence[int], embed: torch.Tensor, bigram: Optional[torch.Tensor], hash_cfg) -> torch.Tensor:
    T, width = len(tokens), embed.shape[1]
    x = embed[list(tokens)].clone()
    if bigram is not None:
        buckets, mp, mc = int(hash_cfg["buckets"]), int(hash_cfg["mul_prev"]), int(hash_cfg["mul_cur"])
        for t in range(T):
            row = buckets if t == 0 else (int(tokens[t - 1]) * mp + int(tokens[t]) * mc) % buckets
            x[t] += bigram[row]
    return x + position_vectors(T, width)


def token_shift(h: torch.Tensor, s: torch.Tensor) -> torch.Tensor:
    prev = torch.zeros_like(h)
    prev[1:] = h[:-1]
    return h + (prev - h) * s


def decayed_linear_attention(q, k, v, decay) -> torch.Tensor:
    """One head.  q, k [T, dim], v [T, vdim]; decay [T, dim] (a factor for every row of the state, every token).
    S_t = diag(decay_t) S_{t-1} + k_t v_t^T; o_t = S_t^T q_t."""
    T, dim = q.shape
    S = torch.zeros((dim, v.shape[1]), dtype=F)
    out = torch.zeros((T, v.shape[1]), dtype=F)
    for t in range(T):
        S = decay[t][:, None] * S + torch.outer(k[t], v[t])
        out[t] = S.T @ q[t]
    return out


def lightning(h: torch.Tensor, w: Dict[str, torch.Tensor], m, eps: float) -> torch.Tensor:
    heads, dim, vdim = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    q = silu(h @ w["q"].T).view(T, heads, dim)
    k = silu(h @ w["k"].T).view(T, heads, dim)
    v = silu(h @ w["v"].T).view(T, heads, vdim)
    o = torch.zeros((T, heads, vdim), dtype=F)
    for a in range(heads):
        decay = torch.full((T, dim), float(m["decay"][a]), dtype=F)
        o[:, a] = decayed_linear_attention(q[:, a], k[:, a], v[:, a], decay)
    y = rms(o.reshape(T, heads * vdim), eps) * w["norm"]
    y = y * torch.sigmoid(h @ w["g"].T)
    return y @ w["o"].T


def distance_bucket(n: int, rows: int, far: float) -> int:
    half = rows // 2
    if n < half:
        return n
    if half < 1 or far <= half:
        return rows - 1
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def visible(i: int, j: int, size: int, keep_first: int) -> bool:
    return j <= i and (i - j < size or j < keep_first)


def biased_window_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m, eps: float) -> torch.Tensor:
    """Dense over the whole sequence: a [T, T] matrix of scores per head, the bias and the visibility written out
    pair by pair.  ``softcap``, ``bias_max`` (with the tensor ``rel``) and ``mask`` may each be absent."""
    H, G, dim, vdim = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    q = (h @ w["q"].T).view(T, H, dim)
    k = (h @ w["k"].T).view(T, G, dim)
    v = rms((h @ w["v"].T).view(T, G, vdim), eps)
    cap, scale = m.get("softcap"), float(m["scale"])
    mask = m.get("mask")
    size, keep = (int(mask["size"]), int(mask.get("keep_first", 0))) if mask else (T + 1, 0)
    seen = torch.tensor([[visible(i, j, size, keep) for j in range(T)] for i in range(T)])
    bucket = None
    if m.get("bias_max") is not None:
        rows = w["rel"].shape[0]
        bucket = torch.tensor([[distance_bucket(i - j, rows, float(m["bias_max"])) if j <= i else 0 for j in range(T)]
                               for i in range(T)])
    out = torch.zeros((T, H, vdim), dtype=F)
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * scale
        if cap:
            s = float(cap) * torch.tanh(s / float(cap))
        if bucket is not None:
            s = s + w["rel"][:, a][bucket]
        s = s.masked_fill(~seen, float("-inf"))
        out[:, a] = torch.softmax(s, dim=1) @ v[:, g]
    y = out.reshape(T, H * vdim) * torch.sigmoid(h @ w["g"].T)
    return y @ w["o"].T


def gated_linear_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m, eps: float) -> torch.Tensor:
    heads, dim, vdim = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    q = (h @ w["q"].T).view(T, heads, dim) * dim ** -0.5
    k = (h @ w["k"].T).view(T, heads, dim)
    v = (h @ w["v"].T).view(T, heads, vdim)
    z = (h @ w["a1"].T) @ w["a2"].T + w["a2.b"]
    alpha = (torch.sigmoid(z) ** (1.0 / float(m["tau"]))).view(T, heads, dim)
    o = torch.zeros((T, heads, vdim), dtype=F)
    for a in range(heads):
        o[:, a] = rms(decayed_linear_attention(q[:, a], k[:, a], v[:, a], alpha[:, a]), eps) * w["norm"]
    y = o.reshape(T, heads * vdim) * silu(h @ w["g"].T)
    return y @ w["o"].T


def parallel_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m, eps: float) -> torch.Tensor:
    left = biased_window_attention(h, {k[5:]: t for k, t in w.items() if k.startswith("left.")}, m["left"], eps)
    right = gated_linear_attention(h, {k[6:]: t for k, t in w.items() if k.startswith("right.")}, m["right"], eps)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


def table_experts(h: torch.Tensor, tokens: Sequence[int], w: Dict[str, torch.Tensor], mlp) -> torch.Tensor:
    top = int(mlp["router"]["top"])
    out = torch.zeros_like(h)
    for t, tok in enumerate(tokens):
        for e in w["table"][int(tok)].tolist():
            z = silu(w[f"e{e}.gate"] @ h[t]) * (w[f"e{e}.up"] @ h[t])
            out[t] += (w[f"e{e}.down"] @ z) / top
    return out


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------
class PlainTilivik:
    def __init__(self, config: dict, tensors: Dict[str, torch.Tensor]):
        self.cfg = config
        self.t = {k: (v.to(F) if v.dtype.is_floating_point else v.long()) for k, v in tensors.items()}
        self.eps = float(config["norm"]["eps"])

    @classmethod
    def from_folder(cls, folder: str) -> "PlainTilivik":
        from safetensors.torch import load_file
        with open(os.path.join(folder, "config.json")) as f:
            cfg = json.load(f)
        return cls(cfg, load_file(os.path.join(folder, "model.safetensors")))

    def sub(self, prefix: str) -> Dict[str, torch.Tensor]:
        return {k[len(prefix):]: v for k, v in self.t.items() if k.startswith(prefix)}

    def run_order(self) -> List[tuple]:
        """(layer, pass or None) in the order the layers run."""
        L = len(self.cfg["layers"])
        loop = self.cfg.get("loop")
        if not loop:
            return [(i, None) for i in range(L)]
        a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
        order = [(i, None) for i in range(a)]
        for t in range(times):
            order += [(i, t) for i in range(a, b)]
        return order + [(i, None) for i in range(b, L)]

    def layer(self, i: int, x: torch.Tensor, tokens: Sequence[int]) -> torch.Tensor:
        spec, p = self.cfg["layers"][i], f"l{i}."
        h = token_shift(scalar_norm(x, self.t[p + "norm1"], self.eps), self.t[p + "shift"])
        w = self.sub(p + "mix.")
        if spec["type"] == "lightning":
            x = x + lightning(h, w, spec["mixer"], self.eps)
        elif spec["type"] == "parallel":
            x = x + parallel_mixer(h, w, spec["mixer"], self.eps)
        else:
            raise ValueError(spec["type"])
        if spec.get("mlp") is not None:
            x = x + table_experts(scalar_norm(x, self.t[p + "norm2"], self.eps), tokens, self.sub(p + "mlp."), spec["mlp"])
        return x

    def forward(self, tokens: Sequence[int], streams: Optional[list] = None) -> torch.Tensor:
        """Logits [T, vocab]; ``streams`` collects the residual stream after every layer run."""
        bi = (self.cfg.get("embedding") or {}).get("bigram")
        x0 = embedding(tokens, self.t["embed"], self.t["bigram"] if bi else None, bi)
        x = x0
        loop = self.cfg.get("loop")
        for i, t in self.run_order():
            if t is not None and i == int(loop["start"]):
                if t > 0:
                    x = x + x0
                x = x + self.t["loop.step"][t]
            x = self.layer(i, x, tokens)
            if streams is not None:
                streams.append(x.clone())
        return scalar_norm(x, self.t["final.norm"], self.eps) @ self.t["head"].T

    def greedy_generate(self, prompt: Sequence[int], new_tokens: int) -> List[int]:
        """The tokens greedy decoding appends (the lowest index among equal logits), each from a full forward pass."""
        toks, out = list(prompt), []
        for _ in range(new_tokens):
            nxt = int(torch.argmax(self.forward(toks)[-1]))
            out.append(nxt)
            toks.append(nxt)
        return out
