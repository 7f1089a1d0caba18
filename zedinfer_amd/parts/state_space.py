"""A selective state-space mixer (the state-space-duality form: one decay a head and token)."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.forward_config import PartSpec
from ..weights.loader import WeightSpec
from .base import LayerMemory, Mixer, Runtime, StateRequest, register_mixer
from .rows import ProductRows


@register_mixer("state_space")
class StateSpace(Mixer):
    """(z | u | B | C | dt) = W_in x, inner = heads * vdim, N = state, G = groups.  u, B and C pass a causal
    convolution per channel (``conv`` taps, with a bias) and SiLU; dt <- softplus(dt + dt_bias).  Per head h (it
    reads B and C of group h / (heads / G)):

        S_t = exp(-exp(A_log_h) dt_t) S_{t-1} + dt_t B_t u_t^T      (S is N x vdim, float32, zero at the start)
        y_t = S_t^T C_t + D_h u_t

    The heads side by side are multiplied by silu(z), RMS-normed in ``norm_groups`` equal parts (a gain a channel)
    and projected.  The state per request is the convolution's last ``conv`` - 1 input rows and the matrices S; the
    recurrence runs token by token in prompts too, so its sums do not depend on how a prompt is cut.

    One stacked input product with float32 results, ``ops.ssm_prepare`` (convolution, SiLU, dt, decay),
    ``ops.conv_tail``, the linear-attention kernel with keys B, queries C, values dt u and the decay a (token, head),
    ``ops.ssm_finish`` (skip, gate, norm), one output product.

    params: hidden_size, heads, vdim, state, groups, conv, norm_groups, eps."""

    graph_safe = True
    tape_safe = True
    padding_safe = False      # padding tokens would move the state on
    writes_into = True

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        p = spec.params
        H, nh, vd, N, G, taps = (int(p[k]) for k in ("hidden_size", "heads", "vdim", "state", "groups", "conv"))
        inner, C = nh * vd, nh * vd + 2 * G * N
        return {"in": WeightSpec((2 * inner + 2 * G * N + nh, H)), "conv": WeightSpec((C, taps)),
                "conv_bias": WeightSpec((C,), init="zeros"), "dt_bias": WeightSpec((nh,), init="zeros"),
                "A_log": WeightSpec((nh,), init="zeros"), "D": WeightSpec((nh,), init="ones"),
                "norm": WeightSpec((inner,), init="ones"), "o": WeightSpec((H, inner))}

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden, self.nh, self.vd, self.N, self.G, self.taps, self.parts = (
            int(p[k]) for k in ("hidden_size", "heads", "vdim", "state", "groups", "conv", "norm_groups"))
        self.eps = float(p.get("eps", 1e-6))
        if self.nh % self.G:
            raise ValueError(f"state_space: {self.nh} heads are not a multiple of {self.G} groups")
        self.inner = self.nh * self.vd
        if self.inner % self.parts:
            raise ValueError(f"state_space: {self.inner} channels do not divide into {self.parts} equal parts")
        if not (1 <= self.taps <= ops.hybrid.SSM_MAX_TAPS) or self.N > 512:
            raise ValueError("state_space: conv must lie in 1..16 and state be at most 512")
        self.gn = self.G * self.N
        self.channels = self.inner + 2 * self.gn
        self.width = 2 * self.inner + 2 * self.gn + self.nh
        w = weights["in"]
        stacked = torch.zeros((-(-self.width // 8) * 8, self.hidden), dtype=w.dtype, device=w.device)   # rows to a multiple of 8
        stacked[:self.width] = w
        self.w_in = stacked
        self.conv_w = weights["conv"].float().contiguous()
        self.conv_b = weights["conv_bias"].float().contiguous()
        self.dt_bias, self.a_log = weights["dt_bias"].float().contiguous(), weights["A_log"].float().contiguous()
        self.skip, self.norm = weights["D"].float().contiguous(), weights["norm"].float().contiguous()
        self.o = weights["o"]
        self.tail = (self.taps - 1) * self.channels

    def state_request(self) -> Optional[StateRequest]:
        return StateRequest((max(1, ops.ssm_state_floats(self.nh, self.vd, self.N, self.G, self.taps)),), torch.float32)

    def step_rows(self, rows: int, kind: str) -> int:
        return ProductRows.step_rows(rows, kind)

    def forward(self, x: torch.Tensor, batch, memory: LayerMemory, out=None) -> torch.Tensor:
        n, rt, inner, gn = x.shape[0], self.rt, self.inner, self.gn
        state = memory.state
        full = ops.linear(x, self.w_in, out=rt.buffer("ssm_proj", (n, self.w_in.shape[0]), torch.float32))
        proj = full[:, :self.width]
        prep = rt.buffer("ssm_prepared", (n, self.width), torch.float32)
        ops.ssm_prepare(proj, self.conv_w, self.conv_b, self.dt_bias, self.a_log, state, batch.tok_seq, batch.entry_start,
                        batch.entry_slot, self.nh, self.vd, self.N, self.G, self.taps, out=prep)
        if self.taps > 1:
            ops.conv_tail(state, proj[:, inner:inner + self.channels], None, batch.entry_start, batch.entry_len,
                          batch.entry_slot, self.taps)
        C = self.channels
        y = rt.buffer("ssm_read", (n, inner), torch.float32)
        ops.linear_attention_grouped(prep[:, inner + gn:C], prep[:, inner:inner + gn], prep[:, C:C + inner],
                                     prep[:, C + inner:], state[:, self.tail:], batch.entry_start, batch.entry_len,
                                     batch.entry_past, batch.entry_slot, self.nh, self.nh // self.G, self.N, self.vd, out=y,
                                     single_tokens=bool(batch.single_tokens))
        g = rt.buffer("ssm_gated", (n, inner))
        ops.ssm_finish(y, prep[:, :inner], proj[:, :inner], self.skip, self.norm, self.nh, self.vd, self.parts, self.eps, out=g)
        if out is None:
            if ops.linear_sums_supported(g, self.o):      # few rows: the partial sums go to the norm that follows
                S = ops.linear_splits(n, self.hidden, inner)
                return ops.linear_sums(g, self.o, out=rt.buffer("ssm_out_sums", (S, n, self.hidden), torch.float32))
            out = rt.buffer("ssm_out", (n, self.hidden))
        return ops.linear(g, self.o, out=out)
