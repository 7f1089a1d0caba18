"""Mixers between two stacked products: x -> W_in x (float32 results) -> a mechanism in float32 -> W_out y.

``ProjectedMixer`` is the common form: a mixer names the rows of its input matrix and the columns of its output
matrix, and computes ``mix`` between them.  It runs alone (two products of its own), or as one of several mixers
side by side (``side_by_side``), which read the same input through ONE product of their stacked input matrices and
whose gated results leave through ONE product over their concatenated columns; a scale of each mixer's share is
applied where its result is rounded to the activation type.  A token shift in front of the input product is an
option of whoever owns the products.

The mechanisms here: linear attention with a decayed matrix state per head, with a fixed decay per head
(``lightning_attention``) or a decay per token and key channel from a low-rank gate (``gated_linear_attention``),
and softmax attention without rotation over a window and a sequence's first positions, with capped scores, a
learned bias by distance and normed values (``biased_window_attention``).
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from .. import ops
from ..config.forward_config import PartSpec
from ..weights.loader import WeightSpec
from .base import MIXERS, KVCacheRequest, LayerMemory, Mixer, Runtime, StateRequest, register_mixer
from .mixers import LONG_TILE, attention_cache_request, attention_planner
from .rows import ProductRows


def _pad_rows(mats: List[torch.Tensor], multiple: int = 8) -> torch.Tensor:
    """The matrices stacked along rows (one storage type), zero rows added up to a multiple."""
    dt = mats[0].dtype
    rows = sum(int(m.shape[0]) for m in mats)
    out = torch.zeros((-(-rows // multiple) * multiple, mats[0].shape[1]), dtype=dt, device=mats[0].device)
    at = 0
    for m in mats:
        out[at:at + m.shape[0]] = m.to(dt)
        at += m.shape[0]
    return out


class ProjectedMixer(Mixer):
    """A mixer of the form W_out mix(W_in shift(x)).

    A subclass sets ``w_in`` [rows (a multiple of 8), hidden], ``w_out`` [hidden, width_out], ``state_floats`` (float32
    values of state a request keeps for the mechanism) and implements ``mix(proj, batch, memory, state, y, scale)``:
    ``proj`` float32 [n, rows] (a column slice of a wider product is fine), ``state`` float32 [slots, state_floats]
    (a column slice of the slot's row) or None, ``y`` [n, width_out] in the activation type (a column slice is fine)
    receives the mechanism's gated result times ``scale``.

    ``shift`` in the params (with the weight ``shift`` [hidden]): the input is first replaced, channel by channel, by
    x_t + (x_{t-1} - x_t) * shift, x_{-1} = 0; the last input row of a request is state too.  The state slot's row is
    [shift row | mechanism]."""

    graph_safe = True
    tape_safe = True
    padding_safe = False      # a padding token would move the state
    writes_into = True

    hidden: int
    w_in: torch.Tensor
    w_out: torch.Tensor
    state_floats: int = 0
    shift: Optional[torch.Tensor] = None

    @staticmethod
    def shift_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        return {"shift": WeightSpec((int(spec.params["hidden_size"]),), init="zeros")} if spec.params.get("shift") else {}

    def init_shift(self, spec: PartSpec, weights: Dict[str, torch.Tensor]) -> None:
        self.shift = weights["shift"].float().contiguous() if spec.params.get("shift") else None

    # ---- what the cache manager provides -----------------------------------------------
    def state_request(self) -> Optional[StateRequest]:
        n = (self.hidden if self.shift is not None else 0) + int(self.state_floats)
        return StateRequest((n,), torch.float32) if n else None

    def step_rows(self, rows: int, kind: str) -> int:
        return ProductRows.step_rows(rows, kind)

    standalone = True      # False for a mixer that runs inside ``side_by_side``: its products are that part's

    def tune(self, num_tokens: int) -> None:
        if not self.standalone:
            return
        n = int(num_tokens)
        self.rt.tune_linear(self.rt.buffer("mix_in", (n, self.hidden)), self.w_in, out_dtype=torch.float32)
        self.rt.tune_linear(self.rt.buffer("mix_y", (n, self.w_out.shape[1])), self.w_out, out_dtype=torch.float32)

    # ---- the mechanism --------------------------------------------------------------------
    def mix(self, proj, batch, memory: LayerMemory, state, y, scale: float) -> None:
        raise NotImplementedError

    def shifted(self, x: torch.Tensor, batch, memory: LayerMemory) -> torch.Tensor:
        """The rows the input product reads: x itself in the activation type, or its token shift."""
        n = x.shape[0]
        if self.shift is None:
            if x.dtype == self.rt.dtype:
                return x
            return ops.convert(x, self.rt.buffer("mix_in", (n, self.hidden)))
        h = self.rt.buffer("mix_in", (n, self.hidden))
        return ops.token_shift(x, self.shift, memory.state[:, :self.hidden], batch.tok_seq, batch.positions,
                               batch.entry_start, batch.entry_len, batch.entry_slot, out=h)

    def forward(self, x: torch.Tensor, batch, memory: LayerMemory, out=None) -> torch.Tensor:
        n, rt = x.shape[0], self.rt
        h = self.shifted(x, batch, memory)
        proj = ops.linear(h, self.w_in, out=rt.buffer("mix_proj", (n, self.w_in.shape[0]), torch.float32))
        y = rt.buffer("mix_y", (n, self.w_out.shape[1]))
        at = self.hidden if self.shift is not None else 0
        state = memory.state[:, at:at + self.state_floats] if self.state_floats else None
        self.mix(proj, batch, memory, state, y, 1.0)
        if out is None:
            if ops.linear_sums_supported(y, self.w_out):
                # few rows: the product's partial sums go on as they are; the norm (or the step between layers) that
                # takes the mixer's result adds them, so no kernel is launched for that alone
                S = ops.linear_splits(n, self.hidden, self.w_out.shape[1])
                return ops.linear_sums(y, self.w_out, out=rt.buffer("mix_out_sums", (S, n, self.hidden), torch.float32))
            out = rt.buffer("mix_out", (n, self.hidden), torch.float32)
        return ops.linear(y, self.w_out, out=out)


@register_mixer("lightning_attention")
class LightningAttention(ProjectedMixer):
    """Linear attention with a fixed decay per head: q, k = silu(W x) [heads, dim], v = silu(W_v x) [heads, vdim];
    per head S_t = c_h S_{t-1} + k_t v_t^T, o_t = S_t^T q_t, no other scale; the concatenated heads are RMS-normed
    together (gain ``norm`` [heads * vdim]), times sigmoid(W_g x), then W_o.  S is float32 state of the request.
    params: hidden_size, heads, dim, vdim, decay (one factor a head), eps, shift (False)."""

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        p = spec.params
        H, nh, dim, vdim = (int(p[k]) for k in ("hidden_size", "heads", "dim", "vdim"))
        w = {"q": WeightSpec((nh * dim, H)), "k": WeightSpec((nh * dim, H)), "v": WeightSpec((nh * vdim, H)),
             "g": WeightSpec((nh * vdim, H)), "norm": WeightSpec((nh * vdim,), init="ones"), "o": WeightSpec((H, nh * vdim))}
        w.update(ProjectedMixer.shift_specs(spec))
        return w

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden, self.nh, self.dim, self.vdim = (int(p[k]) for k in ("hidden_size", "heads", "dim", "vdim"))
        self.eps = float(p.get("eps", 1e-6))
        decay = [float(c) for c in p["decay"]]
        if len(decay) != self.nh:
            raise ValueError(f"lightning_attention: {len(decay)} decays for {self.nh} heads")
        self.decay = torch.tensor(decay, dtype=torch.float32, device=weights["q"].device)
        self.w_in = _pad_rows([weights[k] for k in ("q", "k", "v", "g")])
        self.w_out = weights["o"]
        self.norm = weights["norm"].float().contiguous()
        self.state_floats = ops.linear_attention_state_floats(self.nh, self.dim, self.vdim)
        self.init_shift(spec, weights)

    def mix(self, proj, batch, memory, state, y, scale):
        n, qk, vd = proj.shape[0], self.nh * self.dim, self.nh * self.vdim
        o = self.rt.buffer("linear_attention_read", (n, vd), torch.float32)
        ops.linear_attention(proj[:, :qk], proj[:, qk:2 * qk], proj[:, 2 * qk:2 * qk + vd], state, batch.entry_start,
                             batch.entry_len, batch.entry_past, batch.entry_slot, self.nh, self.dim, self.vdim, out=o,
                             head_decay=self.decay, silu=True)
        ops.gated_rms_norm_act(o, self.norm, proj[:, 2 * qk + vd:2 * qk + 2 * vd], 1, vd, self.eps, "sigmoid", out=y,
                               scale=scale)


@register_mixer("gated_linear_attention")
class GatedLinearAttention(ProjectedMixer):
    """Linear attention with a decay per token and key channel: q = W_q x * dim^-1/2, k = W_k x [heads, dim],
    v = W_v x [heads, vdim]; alpha = sigmoid(W_a2 (W_a1 x) + b)^(1/tau) [heads, dim]; per head
    S_t = diag(alpha_t) S_{t-1} + k_t v_t^T, o_t = S_t^T q_t; every head's o is RMS-normed over vdim (gain ``norm``
    [vdim], shared by the heads), the heads times silu(W_g x), then W_o.  S is float32 state of the request; the
    gate's logarithm, power and the recurrence are float32.
    params: hidden_size, heads, dim, vdim, tau, rank (of the gate; -1: the checkpoint's), eps, shift (False)."""

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        p = spec.params
        H, nh, dim, vdim, rank = (int(p[k]) for k in ("hidden_size", "heads", "dim", "vdim", "rank"))
        w = {"q": WeightSpec((nh * dim, H)), "k": WeightSpec((nh * dim, H)), "v": WeightSpec((nh * vdim, H)),
             "g": WeightSpec((nh * vdim, H)), "a1": WeightSpec((rank, H)), "a2": WeightSpec((nh * dim, rank)),
             "a2_bias": WeightSpec((nh * dim,), init="zeros"), "norm": WeightSpec((vdim,), init="ones"),
             "o": WeightSpec((H, nh * vdim))}
        w.update(ProjectedMixer.shift_specs(spec))
        return w

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden, self.nh, self.dim, self.vdim = (int(p[k]) for k in ("hidden_size", "heads", "dim", "vdim"))
        self.rank = int(weights["a1"].shape[0])      # the checkpoint's own when the params leave it open (-1)
        self.eps, self.tau = float(p.get("eps", 1e-6)), float(p["tau"])
        if not self.tau > 0:
            raise ValueError("gated_linear_attention: tau must be positive")
        self.w_in = _pad_rows([weights[k] for k in ("q", "k", "v", "g", "a1")])
        self.w_out = weights["o"]
        self.a2 = weights["a2"].contiguous()
        self.a2_bias = weights["a2_bias"].to(self.a2.dtype).contiguous()
        self.norm = weights["norm"].float().contiguous()
        self.state_floats = ops.linear_attention_state_floats(self.nh, self.dim, self.vdim)
        self.init_shift(spec, weights)

    def mix(self, proj, batch, memory, state, y, scale):
        n, qk, vd = proj.shape[0], self.nh * self.dim, self.nh * self.vdim
        rt = self.rt
        a_at = 2 * qk + 2 * vd
        alpha = ops.lowrank_decay(proj[:, a_at:a_at + self.rank], self.a2, self.a2_bias, self.tau,
                                  out=rt.buffer("linear_attention_decay", (n, qk), torch.float32))
        o = rt.buffer("linear_attention_read", (n, vd), torch.float32)
        ops.linear_attention(proj[:, :qk], proj[:, qk:2 * qk], proj[:, 2 * qk:2 * qk + vd], state, batch.entry_start,
                             batch.entry_len, batch.entry_past, batch.entry_slot, self.nh, self.dim, self.vdim, out=o,
                             decay=alpha, qscale=self.dim ** -0.5)
        ops.gated_rms_norm_act(o, self.norm, proj[:, 2 * qk + vd:a_at], self.nh, self.vdim, self.eps, "silu", out=y,
                               scale=scale)


def distance_bias_table(rel: torch.Tensor, far: float) -> torch.Tensor:
    """The bias by distance as a table [heads, L] (float32; distances beyond L - 1 take the last entry) from the
    learned rows ``rel`` [B, heads]: distance n < B/2 reads row n; beyond, rows are spaced evenly in log(n) up to
    ``far``, row min(B - 1, B/2 + floor(log(n / (B/2)) / log(far / (B/2)) * (B - B/2)))."""
    B = int(rel.shape[0])
    half = B // 2
    if half < 1 or not far > half:      # no logarithmic part: the near rows, then the last row for all the rest
        rows = list(range(half)) + [B - 1]
    else:
        rows, n = [], 0
        while True:
            r = n if n < half else min(B - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (B - half))))
            rows.append(r)
            if r >= B - 1 or n > (1 << 22):
                break
            n += 1
    idx = torch.tensor(rows, dtype=torch.long, device=rel.device)
    return rel.float()[idx].t().contiguous()


@register_mixer("biased_window_attention")
class BiasedWindowAttention(ProjectedMixer):
    """Grouped-query softmax attention without rotation: q = W_q x [heads, dim], k = W_k x [kv_heads, dim],
    v = W_v x [kv_heads, vdim], each value head divided by its root mean square (no gain) before it is cached;
    score = (q . k) * scale, then cap * tanh(score / cap), then plus a learned bias by the distance i - j (see
    ``distance_bias_table``; the scale does not multiply it); position i sees j <= i with i - j < window or
    j < keep_first (kept positions keep their true distances); the heads times sigmoid(W_g x), then W_o.

    The cache holds heads of one size, the larger of dim and vdim (in bfloat16 rounded up to a multiple of 16), the
    rest zero.  Scores, cap, bias and softmax are float32.
    params: hidden_size, heads, kv_heads, dim, vdim, scale, softcap (0: none), bias_max (None: no bias), bias_rows
    (rows of the bias tensor; 0: whatever the checkpoint holds), window (0: all keys), keep_first, eps, value_norm
    (True), shift (False)."""

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        p = spec.params
        H, nh, nkv, dim, vdim = (int(p[k]) for k in ("hidden_size", "heads", "kv_heads", "dim", "vdim"))
        w = {"q": WeightSpec((nh * dim, H)), "k": WeightSpec((nkv * dim, H)), "v": WeightSpec((nkv * vdim, H)),
             "g": WeightSpec((nh * vdim, H)), "o": WeightSpec((H, nh * vdim))}
        if p.get("bias_max") is not None:
            # the number of rows is the tensor's own (any number when the params give none)
            w["rel"] = WeightSpec((int(p.get("bias_rows", 0) or 0) or -1, nh))
        w.update(ProjectedMixer.shift_specs(spec))
        return w

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden, self.nh, self.nkv, self.dim, self.vdim = (int(p[k]) for k in ("hidden_size", "heads", "kv_heads", "dim", "vdim"))
        if self.nh % self.nkv:
            raise ValueError(f"biased_window_attention: {self.nh} heads are not a multiple of {self.nkv} key/value heads")
        self.scale, self.softcap = float(p["scale"]), float(p.get("softcap", 0.0) or 0.0)
        self.window, self.keep_first = int(p.get("window", 0) or 0), int(p.get("keep_first", 0) or 0)
        self.eps, self.value_norm = float(p.get("eps", 1e-6)), bool(p.get("value_norm", True))
        big = max(self.dim, self.vdim)
        self.d = -(-big // 16) * 16 if (rt.dtype == torch.bfloat16 and big <= 128) else big
        self.w_in = _pad_rows([weights[k] for k in ("q", "k", "v", "g")])
        self.w_out = weights["o"]
        self.bias = distance_bias_table(weights["rel"], float(p["bias_max"])) if "rel" in weights else None
        self.state_floats = 0
        self.init_shift(spec, weights)
        # the step's tokens are dealt out as for any softmax attention: single tokens, tiles of prompt portions
        self.plan_key = attention_planner(LONG_TILE, self.nh).key

    def planner(self):
        return attention_planner(LONG_TILE, self.nh)

    def attend(self, q, att, batch, view, kc, vc) -> None:
        """Tokens of short entries go to the kernel that splits one query's keys over many wavefronts, longer
        portions to the matrix-core prompt kernel, both with the cap, the bias and the kept positions; every shape
        those kernels do not take (float32, heads beyond 128) goes to the plain kernel."""
        extras = dict(softcap=self.softcap, bias=self.bias, keep_first=self.keep_first)
        plan = batch.plans[self.plan_key]
        n_short, n_long, N = plan.sizes["num_short"], plan.sizes["num_long"], batch.num_tokens
        cores = (ops.attention_decode_supported(q.dtype, self.nh, self.nkv, self.d, kc.shape[2])
                 and ops.attention_prefill_supported(q.dtype, self.nh, self.nkv, self.d, kc.shape[2]))
        if not cores:
            ops.attention_biased(q, kc, vc, batch.tok_seq, batch.positions, view.block_tables, self.nh, self.nkv, self.d,
                                 self.scale, self.window, out=att, **extras)
            return
        if n_short:
            ws = self.rt.buffer("attn_split", (ops.attention_decode_workspace(n_short, self.nh, self.d),), torch.float32)
            ops.attention_decode(q, kc, vc, batch.tok_seq, batch.positions, view.block_tables, self.nh, self.nkv, self.d,
                                 self.scale, plan.sizes["max_short_keys"], self.window, out=att,
                                 tok_index=plan.dev["short_idx"] if n_short < N else None, workspace=ws, **extras)
        if n_long:
            max_keys = plan.sizes["max_long_keys"]
            need = ops.attention_prefill_workspace(q.shape[0], self.nh, self.d, max_keys, self.window, plan.sizes["num_tiles"])
            ws = self.rt.buffer("attn_prompt_split", (need,), torch.float32) if need else None
            ops.attention_prefill(q, kc, vc, plan.dev["tile_entry"], plan.dev["tile_off"], batch.entry_start,
                                  batch.entry_len, batch.entry_past, view.block_tables, self.nh, self.nkv, self.d,
                                  self.scale, self.window, out=att, max_keys=max_keys, workspace=ws,
                                  tile=plan.sizes["tile"], **extras)

    def cache_request(self) -> Optional[KVCacheRequest]:
        if self.window > 0:
            rq = attention_cache_request("window", self.nkv, self.d, self.window)
            return KVCacheRequest(rq.kind, rq.window, rq.tensors, keep_first=self.keep_first)
        return attention_cache_request("full", self.nkv, self.d)

    def mix(self, proj, batch, memory, state, y, scale):
        n, rt = proj.shape[0], self.rt
        view = batch.groups[memory.group]
        qd, kd = self.nh * self.dim, self.nkv * self.dim
        kc, vc = memory.tensors["k"], memory.tensors["v"]
        q = rt.buffer("attn_q", (n, self.nh * self.d))
        ops.normed_kv_store(proj, 0, qd, qd + kd, q, view.slots if memory.writes else None, kc if memory.writes else None,
                            vc if memory.writes else None, self.nh, self.nkv, self.dim, self.vdim, self.d, self.eps,
                            norm_values=self.value_norm)
        att = rt.buffer("attn_out", (n, self.nh * self.d))
        self.attend(q, att, batch, view, kc, vc)
        g_at = qd + kd + self.nkv * self.vdim
        ops.gate_heads(att, proj[:, g_at:g_at + self.nh * self.vdim], self.vdim, self.d, "sigmoid", out=y, scale=scale)


@register_mixer("side_by_side")
class SideBySide(ProjectedMixer):
    """Several ``ProjectedMixer``s that read the same input: the result is sum_i scale_i * mixer_i(x).  Their input
    matrices are stacked into one product and their output matrices joined along the columns into one, so the sum
    over the mixers is made inside the output product (in float32); each mixer's share is scaled where its gated
    result is rounded to the activation type.  At most one of them keeps pages in the cache; each keeps its own
    state, one after the other in the request's slot.
    params: hidden_size, mixers (PartSpecs, whose parameter names stand in this part's weights as "<i>.<name>"),
    scales, shift (False)."""

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        w = {}
        for i, sub in enumerate(spec.params["mixers"]):
            for name, ws in MIXERS.get(sub.kind).weight_specs(sub).items():
                w[f"{i}.{name}"] = ws
        w.update(ProjectedMixer.shift_specs(spec))
        return w

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.scales = [float(s) for s in p["scales"]]
        self.mixers: List[ProjectedMixer] = []
        for i, sub in enumerate(p["mixers"]):
            cls = MIXERS.get(sub.kind)
            if not issubclass(cls, ProjectedMixer) or sub.params.get("shift"):
                raise ValueError(f"side_by_side: '{sub.kind}' must be a mixer between two products, without a shift of its own")
            local = {k[len(f"{i}."):]: t for k, t in weights.items() if k.startswith(f"{i}.")}
            self.mixers.append(cls(sub, local, rt))
            self.mixers[-1].standalone = False
            setattr(self, f"mixer_{i}", self.mixers[-1])      # a part of its own for whoever walks the parts
        if len(self.scales) != len(self.mixers) or not self.mixers:
            raise ValueError("side_by_side: one scale for every mixer")
        if sum(1 for m in self.mixers if m.cache_request() is not None) > 1:
            raise ValueError("side_by_side: at most one mixer may keep pages in the cache")
        self.w_in = torch.cat([m.w_in for m in self.mixers], dim=0).contiguous()
        self.w_out = torch.cat([m.w_out for m in self.mixers], dim=1).contiguous()
        self.state_floats = sum(int(m.state_floats) for m in self.mixers)
        self.init_shift(spec, weights)

    def cache_request(self) -> Optional[KVCacheRequest]:
        for m in self.mixers:
            rq = m.cache_request()
            if rq is not None:
                return rq
        return None

    def planner(self):
        for m in self.mixers:
            pl = m.planner()
            if pl is not None:
                return pl
        return None

    def mix(self, proj, batch, memory, state, y, scale):
        r = c = s = 0
        for m, a in zip(self.mixers, self.scales):
            rows, cols, floats = m.w_in.shape[0], m.w_out.shape[1], int(m.state_floats)
            m.mix(proj[:, r:r + rows], batch, memory, state[:, s:s + floats] if floats else None, y[:, c:c + cols], scale * a)
            r, c, s = r + rows, c + cols, s + floats
