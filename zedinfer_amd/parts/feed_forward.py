"""Feed-forward parts."""
from __future__ import annotations

import os
from typing import Dict

import torch

from .. import ops
from ..config.forward_config import PartSpec
from ..weights.loader import WeightSpec
from .base import FeedForward, Runtime, register_feed_forward
from .rows import ProductRows


def stack_rows(tensors):
    """Concatenate [n_i, k] matrices along rows when they share a storage type; else None."""
    if len({t.dtype for t in tensors}) != 1:
        return None
    return torch.cat(list(tensors), dim=0).contiguous()


def interleave_rows(a: torch.Tensor, b: torch.Tensor, block: int) -> torch.Tensor:
    """[a rows 0..block-1, b rows 0..block-1, a rows block..2*block-1, ...] for two [n, k] matrices."""
    n, k = a.shape
    return torch.stack([a.view(n // block, block, k), b.view(n // block, block, k)], dim=1).reshape(2 * n, k).contiguous()


GATE_UP_BLOCK = 8    # gate and up rows alternate in blocks of 8: one matrix-core tile holds both for 8 columns


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    """down(up(x) * silu(gate(x))), no biases (reference:
    src/frontend/models/transformer_forward.cpp:128-137; src/backend/ops/swiglu/cpu/swiglu_cpu.cpp:9-23).
    gate and up are stacked into one [2I, H] matrix at load: one product instead of two, the same
    sums per output element.  In bfloat16 (and with I a multiple of 8) their rows alternate in
    blocks of 8, so that the few-rows product can apply the activation in its epilogue.
    params: hidden_size, intermediate_size."""

    graph_safe = True
    tape_safe = True
    # For many rows the gate/up product is the library's, and at some sizes it makes the transposed
    # result, W . x^T, faster than x . W^T (measured at the 1.5B sizes: 100 against 119 us at 2,048 rows,
    # 31 against 37 at 512, 73 against 67 at 1,024).  The transposed result goes through the activation
    # kernel that turns it back; the two ways differ by rounding.  Which one a step of n rows takes is
    # read from ``rt.choices[("gate_up_transposed", n, 2I, H)]``: absent, the straight product (or what
    # ZEDINFER_GATE_UP_TRANSPOSED=0/1 says).  ``tune(n)`` measures both outside of any step and records
    # the winner there; nothing is measured while a step runs.
    TRANSPOSED_MIN_ROWS = 128

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        H, I = int(spec.params["hidden_size"]), int(spec.params["intermediate_size"])
        return {"gate": WeightSpec((I, H)), "up": WeightSpec((I, H)), "down": WeightSpec((H, I))}

    def _choice_key(self, n: int) -> tuple:
        return ("gate_up_transposed", int(n), 2 * self.inter, self.hidden)

    def _can_transpose(self, n: int) -> bool:
        return (self.interleave == GATE_UP_BLOCK and self.rt.dtype == torch.bfloat16
                and n >= self.TRANSPOSED_MIN_ROWS and n % 8 == 0)

    def _gate_up_straight(self, x: torch.Tensor, act: torch.Tensor) -> None:
        gu = self.rt.buffer("ffn_gate_up", (x.shape[0], 2 * self.inter))
        ops.linear(x, self.gate_up, out=gu)
        ops.swiglu(gu, out=act, interleave=self.interleave)

    def _gate_up_transposed(self, x: torch.Tensor, act: torch.Tensor) -> None:
        n, I = x.shape[0], self.inter
        gut = self.rt.buffer("ffn_gate_up", (n, 2 * I)).view(-1)[:2 * I * n].view(2 * I, n)      # the same memory
        ops.linear_transposed(x, self.gate_up, out=gut)
        ops.swiglu_t(gut, out=act)

    def _gate_up_many_rows(self, x: torch.Tensor, act: torch.Tensor) -> None:
        """act = swiglu of the gate/up product of x, bfloat16, interleaved weights, more rows than the
        few-rows kernels take."""
        n = x.shape[0]
        if self._can_transpose(n) and x.is_contiguous():
            wins = self.rt.choices.get(self._choice_key(n))
            if wins is None:
                wins = os.environ.get("ZEDINFER_GATE_UP_TRANSPOSED", "") == "1"
            if wins:
                return self._gate_up_transposed(x, act)
        return self._gate_up_straight(x, act)

    def step_rows(self, rows: int, kind: str) -> int:
        return ProductRows.step_rows(rows, kind)

    def tune(self, num_tokens: int) -> None:
        """For steps of ``num_tokens`` rows: the library's algorithms for the gate/up and down products, then the
        orientation of the gate/up product: three runs each of product plus activation; the transposed one must
        win by 5 %."""
        n, key = int(num_tokens), self._choice_key(num_tokens)
        x = self.rt.buffer("norm_out", (n, self.hidden))
        act = self.rt.buffer("ffn_act", (n, self.inter))
        # first the library's algorithm for each product, then the way round with those
        if self.gate_up is not None:
            self.rt.tune_linear(x, self.gate_up)
            if self._can_transpose(n):
                self.rt.tune_linear(x, self.gate_up, transposed=True)
        self.rt.tune_linear(act, self.down)
        forced = os.environ.get("ZEDINFER_GATE_UP_TRANSPOSED", "")
        if key in self.rt.choices or not self._can_transpose(n) or forced in ("0", "1"):
            return

        def clock(fn):
            fn(x, act)
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(3):
                fn(x, act)
            b.record()
            b.synchronize()
            return a.elapsed_time(b)
        self.rt.choices[key] = bool(clock(self._gate_up_transposed) < 0.95 * clock(self._gate_up_straight))

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        self.hidden = int(spec.params["hidden_size"])
        self.inter = int(spec.params["intermediate_size"])
        g, u = weights["gate"], weights["up"]
        self.interleave = 0
        self.gate = self.up = None
        if g.dtype == u.dtype == torch.bfloat16 and self.inter % GATE_UP_BLOCK == 0:
            self.gate_up = interleave_rows(g, u, GATE_UP_BLOCK)
            self.interleave = GATE_UP_BLOCK
        else:
            self.gate_up = stack_rows([g, u])
            if self.gate_up is None:
                self.gate, self.up = g, u
        self.down = weights["down"]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        n, I = x.shape[0], self.inter
        act = self.rt.buffer("ffn_act", (n, I))
        if self.interleave and ops.linear_swiglu_supported(x, self.gate_up):
            ops.linear_swiglu(x, self.gate_up, out=act)
        elif self.interleave and ops.linear_sums_supported(x, self.gate_up, ops.FEW_ROWS):
            S = ops.linear_splits(n, 2 * I, self.hidden)
            sums = ops.linear_sums(x, self.gate_up, out=self.rt.buffer("ffn_gate_up_sums", (S, n, 2 * I), torch.float32))
            ops.swiglu(sums, out=act, interleave=self.interleave)
        elif self.interleave == GATE_UP_BLOCK and x.dtype == torch.bfloat16:
            self._gate_up_many_rows(x, act)
        else:
            gu = self.rt.buffer("ffn_gate_up", (n, 2 * I))
            if self.gate_up is not None:
                ops.linear(x, self.gate_up, out=gu)
            else:
                ops.linear(x, self.gate, out=gu[:, :I])
                ops.linear(x, self.up, out=gu[:, I:])
            if self.interleave:
                ops.swiglu(gu, out=act, interleave=self.interleave)
            else:
                ops.swiglu(gu[:, :I], gu[:, I:], out=act)
        if ops.linear_sums_supported(act, self.down):
            S = ops.linear_splits(n, self.hidden, I)
            return ops.linear_sums(act, self.down, out=self.rt.buffer("ffn_out_sums", (S, n, self.hidden), torch.float32))
        out = self.rt.buffer("ffn_out", (n, self.hidden))
        return ops.linear(act, self.down, out=out)


@register_feed_forward("none")
class NoFeedForward(FeedForward):
    """A layer without a feed-forward: block arrangements that know the kind leave the term out."""

    graph_safe = True
    tape_safe = True
    writes_into = True

    def forward(self, x: torch.Tensor, out=None):
        return None


@register_feed_forward("gated_mlp")
class GatedMLP(FeedForward):
    """down(act(gate(x)) * up(x)), no biases, with the activation as a parameter: "silu", "gelu_tanh"
    (0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))) or "gelu_erf".  gate and up are stacked into one [2I, H]
    matrix at load (one product); the activation and the product of the halves are one kernel in float32
    arithmetic.  With ``out=`` the result goes there (float32 for a float32 residual term).
    params: hidden_size, intermediate_size, activation."""

    graph_safe = True
    tape_safe = True
    writes_into = True

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        H, I = int(spec.params["hidden_size"]), int(spec.params["intermediate_size"])
        return {"gate": WeightSpec((I, H)), "up": WeightSpec((I, H)), "down": WeightSpec((H, I))}

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        self.hidden = int(spec.params["hidden_size"])
        self.inter = int(spec.params["intermediate_size"])
        self.activation = str(spec.params.get("activation", "silu"))
        if self.activation not in ("silu", "gelu_tanh", "gelu_erf"):
            raise ValueError(f"gated_mlp: unknown activation {self.activation!r}")
        # the up rows begin at a multiple of 8 rows, so that both halves of the product's rows stay aligned
        self.up_at = -(-self.inter // 8) * 8
        g, u = weights["gate"], weights["up"]
        if g.dtype != u.dtype:
            u = u.to(g.dtype)
        stacked = torch.zeros((self.up_at + self.inter, self.hidden), dtype=g.dtype, device=g.device)
        stacked[:self.inter] = g
        stacked[self.up_at:] = u
        self.gate_up = stacked
        self.down = weights["down"]

    def step_rows(self, rows: int, kind: str) -> int:
        return ProductRows.step_rows(rows, kind)

    def tune(self, num_tokens: int) -> None:
        n = int(num_tokens)
        self.rt.tune_linear(self.rt.buffer("norm_out", (n, self.hidden)), self.gate_up)

    def forward(self, x: torch.Tensor, out=None) -> torch.Tensor:
        n, I = x.shape[0], self.inter
        gu = self.rt.buffer("ffn_gate_up", (n, self.up_at + I))
        ops.linear(x, self.gate_up, out=gu)
        act = self.rt.buffer("ffn_act", (n, I))
        ops.gated_act(gu[:, :I], gu[:, self.up_at:], self.activation, out=act)
        if out is None:
            out = self.rt.buffer("ffn_out", (n, self.hidden))
        return ops.linear(act, self.down, out=out)


@register_feed_forward("routed_experts")
class RoutedExperts(FeedForward):
    """A mixture of small feed-forwards down_e(gelu_erf(up_e(x))), no biases, of which every token uses ``top``.

    Router: z = W_router x in float32, s = softmax(z) over all experts; the ``top`` experts with the largest
    s + correction are chosen (the correction steers the choice only), their weights are s * ``scale``, not
    renormalised; the result is the weighted sum of the chosen experts' outputs, in float32.

    Everything runs on the device (``csrc/moe.hip``): the (token, choice) pairs are sorted by expert there, and the
    two products walk tiles of rows of one expert each, so the launches of a step do not depend on what the
    tokens choose.  The experts' matrices are stacked [E, ff, H] and [E, H, ff] at load.
    params: hidden_size, experts, top, ff, scale."""

    graph_safe = True
    tape_safe = True
    writes_into = True

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        H, E, ff = int(spec.params["hidden_size"]), int(spec.params["experts"]), int(spec.params["ff"])
        w = {"router": WeightSpec((E, H)), "correction": WeightSpec((E,), init="zeros")}
        for e in range(E):
            w[f"up_{e}"] = WeightSpec((ff, H))
            w[f"down_{e}"] = WeightSpec((H, ff))
        return w

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden, self.experts, self.top, self.ff = int(p["hidden_size"]), int(p["experts"]), int(p["top"]), int(p["ff"])
        self.scale = float(p.get("scale", 1.0))
        if not (0 < self.top <= self.experts):
            raise ValueError(f"routed_experts: top {self.top} of {self.experts} experts")
        self.router = weights["router"]
        self.correction = weights["correction"].float().contiguous()
        self.up = torch.stack([weights[f"up_{e}"] for e in range(self.experts)]).contiguous()
        self.down = torch.stack([weights[f"down_{e}"] for e in range(self.experts)]).contiguous()

    def step_rows(self, rows: int, kind: str) -> int:
        return ProductRows.step_rows(rows, kind)

    def forward(self, x: torch.Tensor, out=None) -> torch.Tensor:
        n, E, top, rt = x.shape[0], self.experts, self.top, self.rt
        pairs = n * top
        z = ops.linear(x, self.router, out=rt.buffer("moe_logits", (n, E), torch.float32))
        idx = rt.buffer("moe_choice", (n, top), torch.int32)
        wt = rt.buffer("moe_weight", (n, top), torch.float32)
        ops.moe_route(z, self.correction, top, self.scale, idx, wt)
        rows = ops.moe_tile_rows(x.dtype, self.up.dtype, (self.hidden, self.ff), pairs, E)
        tiles = ops.moe_max_tiles(pairs, E, rows)
        plan = rt.buffer("moe_plan", (1 + 3 * tiles,), torch.int32)
        order = rt.buffer("moe_order", (pairs,), torch.int32)
        place_of = rt.buffer("moe_place", (pairs,), torch.int32)
        ops.moe_group(idx, E, rows, plan, order, place_of)
        act = rt.buffer("moe_act", (pairs, self.ff))
        ops.moe_linear(x, self.up, plan, rows, tiles, out=act, source=order, source_div=top, activation="gelu_erf")
        y = rt.buffer("moe_out_rows", (pairs, self.hidden), torch.float32)
        ops.moe_linear(act, self.down, plan, rows, tiles, out=y)
        if out is None:
            out = rt.buffer("moe_out", (n, self.hidden), torch.float32)
        return ops.moe_combine(y, wt, place_of, out)


def _float_result(rt: Runtime, name: str, x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """x . weight^T with float32 results for a norm to read: partial sums [S, n, N] for few rows, else [n, N]."""
    n, N = x.shape[0], weight.shape[0]
    if ops.linear_sums_supported(x, weight):
        S = ops.linear_splits(n, N, x.shape[1])
        return ops.linear_sums(x, weight, out=rt.buffer(name + "_sums", (S, n, N), torch.float32))
    return ops.linear(x, weight, out=rt.buffer(name, (n, N), torch.float32))


@register_feed_forward("relu2_mlp")
class ReluSquaredMLP(FeedForward):
    """down(relu(up(x))^2), no gate, no biases.  The result is float32 (partial sums for few rows): a norm reads it.
    params: hidden_size, intermediate_size."""

    graph_safe = True
    tape_safe = True

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        H, I = int(spec.params["hidden_size"]), int(spec.params["intermediate_size"])
        return {"up": WeightSpec((I, H)), "down": WeightSpec((H, I))}

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        self.hidden = int(spec.params["hidden_size"])
        self.inter = int(spec.params["intermediate_size"])
        self.up, self.down = weights["up"], weights["down"]

    def step_rows(self, rows: int, kind: str) -> int:
        return ProductRows.step_rows(rows, kind)

    def tune(self, num_tokens: int) -> None:
        n = int(num_tokens)
        self.rt.tune_linear(self.rt.buffer("resid_copy", (n, self.hidden)), self.up)
        self.rt.tune_linear(self.rt.buffer("ffn_act", (n, self.inter)), self.down, out_dtype=torch.float32)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        n, I, rt = x.shape[0], self.inter, self.rt
        act = rt.buffer("ffn_act", (n, I))
        if ops.linear_sums_supported(x, self.up):
            S = ops.linear_splits(n, I, self.hidden)
            z = ops.linear_sums(x, self.up, out=rt.buffer("ffn_up_sums", (S, n, I), torch.float32))
        else:
            z = ops.linear(x, self.up, out=rt.buffer("ffn_up", (n, I)))
        ops.relu_squared(z, out=act)
        return _float_result(rt, "ffn_out_f32", act, self.down)


class _ClampedGated:
    """One feed-forward of the clamped gated form, down(g sigmoid(1.702 g) (u + 1)) with g = min(gate x, limit) and
    u = clamp(up x, -limit, limit): gate and up stacked into one product (the up rows begin at a multiple of 8)."""

    def __init__(self, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor, limit: float):
        self.inter, self.hidden = int(gate.shape[0]), int(gate.shape[1])
        self.up_at = -(-self.inter // 8) * 8
        stacked = torch.zeros((self.up_at + self.inter, self.hidden), dtype=gate.dtype, device=gate.device)
        stacked[:self.inter] = gate
        stacked[self.up_at:] = up.to(gate.dtype)
        self.gate_up, self.down, self.limit = stacked, down, float(limit)

    def forward(self, rt: Runtime, x: torch.Tensor, name: str) -> torch.Tensor:
        n, I = x.shape[0], self.inter
        act = rt.buffer(name + "_act", (n, I))
        if ops.linear_sums_supported(x, self.gate_up):
            S = ops.linear_splits(n, self.up_at + I, self.hidden)
            gu = ops.linear_sums(x, self.gate_up, out=rt.buffer(name + "_gate_up_sums", (S, n, self.up_at + I), torch.float32))
            ops.clamped_glu(gu[:, :, :I], gu[:, :, self.up_at:], self.limit, out=act)
        else:
            gu = ops.linear(x, self.gate_up, out=rt.buffer(name + "_gate_up", (n, self.up_at + I), torch.float32))
            ops.clamped_glu(gu[:, :I], gu[:, self.up_at:], self.limit, out=act)
        return act


@register_feed_forward("clamped_experts")
class ClampedExperts(FeedForward):
    """A mixture of small clamped gated feed-forwards (see ``_ClampedGated``; no biases) of which every token uses
    ``top``, plus, optionally, a shared one that every token uses.

    Router: z = W_router x + b in float32; the ``top`` experts with the largest z are chosen (the lowest index among
    equals) and weighted by the softmax over the chosen logits only.  The result is the weighted sum of the chosen
    experts' outputs plus the shared expert's, handed on as a stack of float32 terms [routed, shared].

    Routing, grouping and the experts' products run on the device as for ``routed_experts`` (``csrc/moe.hip``): the
    launches of a step do not depend on what the tokens choose.  The experts' matrices are stacked [E, 2 ff, H] (gate
    rows, then up rows) and [E, H, ff] at load.
    params: hidden_size, experts, top, ff, limit, shared_ff (0: none), shared_limit."""

    graph_safe = True
    tape_safe = True

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        p = spec.params
        H, E, ff, sff = int(p["hidden_size"]), int(p["experts"]), int(p["ff"]), int(p.get("shared_ff", 0) or 0)
        w = {"router": WeightSpec((E, H)), "router_bias": WeightSpec((E,), init="zeros")}
        for e in range(E):
            w[f"gate_{e}"] = WeightSpec((ff, H))
            w[f"up_{e}"] = WeightSpec((ff, H))
            w[f"down_{e}"] = WeightSpec((H, ff))
        if sff:
            w.update({"shared_gate": WeightSpec((sff, H)), "shared_up": WeightSpec((sff, H)),
                      "shared_down": WeightSpec((H, sff))})
        return w

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden, self.experts, self.top, self.ff = int(p["hidden_size"]), int(p["experts"]), int(p["top"]), int(p["ff"])
        self.limit = float(p["limit"])
        if not (0 < self.top <= self.experts):
            raise ValueError(f"clamped_experts: top {self.top} of {self.experts} experts")
        self.router = weights["router"]
        self.router_bias = weights["router_bias"].float().contiguous()
        E = self.experts
        self.gate_up = torch.stack([torch.cat([weights[f"gate_{e}"], weights[f"up_{e}"].to(weights[f"gate_{e}"].dtype)])
                                    for e in range(E)]).contiguous()
        self.down = torch.stack([weights[f"down_{e}"] for e in range(E)]).contiguous()
        self.shared = None
        if int(p.get("shared_ff", 0) or 0):
            self.shared = _ClampedGated(weights["shared_gate"], weights["shared_up"], weights["shared_down"],
                                        float(p["shared_limit"]))

    def step_rows(self, rows: int, kind: str) -> int:
        return ProductRows.step_rows(rows, kind)

    def tune(self, num_tokens: int) -> None:
        n = int(num_tokens)
        if self.shared is not None:
            self.rt.tune_linear(self.rt.buffer("resid_copy", (n, self.hidden)), self.shared.gate_up, out_dtype=torch.float32)
            self.rt.tune_linear(self.rt.buffer("moe_shared_act", (n, self.shared.inter)), self.shared.down,
                                out_dtype=torch.float32)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        n, E, top, ff, rt = x.shape[0], self.experts, self.top, self.ff, self.rt
        pairs = n * top
        # the terms of the result: the routed experts' sum, then the shared expert's output (as the partial sums of
        # its last product when that has few rows); whoever reads the stack adds them
        shared_sums = 0
        if self.shared is not None:
            probe = rt.buffer("moe_shared_act", (n, self.shared.inter))
            shared_sums = ops.linear_splits(n, self.hidden, self.shared.inter) if ops.linear_sums_supported(probe, self.shared.down) else 0
        terms = rt.buffer("moe_terms", (1 + (shared_sums or (1 if self.shared is not None else 0)), n, self.hidden), torch.float32)
        z = ops.linear(x, self.router, out=rt.buffer("moe_logits", (n, E), torch.float32))
        idx = rt.buffer("moe_choice", (n, top), torch.int32)
        wt = rt.buffer("moe_weight", (n, top), torch.float32)
        ops.moe_route_top(z, self.router_bias, top, idx, wt)
        rows = ops.moe_tile_rows(x.dtype, self.gate_up.dtype, (self.hidden, ff), pairs, E)
        tiles = ops.moe_max_tiles(pairs, E, rows)
        plan = rt.buffer("moe_plan", (1 + 3 * tiles,), torch.int32)
        order = rt.buffer("moe_order", (pairs,), torch.int32)
        place_of = rt.buffer("moe_place", (pairs,), torch.int32)
        ops.moe_group(idx, E, rows, plan, order, place_of)
        gu = rt.buffer("moe_gate_up", (pairs, 2 * ff), torch.float32)
        ops.moe_linear(x, self.gate_up, plan, rows, tiles, out=gu, source=order, source_div=top)
        act = rt.buffer("moe_act", (pairs, ff))
        ops.clamped_glu(gu[:, :ff], gu[:, ff:], self.limit, out=act)
        y = rt.buffer("moe_out_rows", (pairs, self.hidden), torch.float32)
        ops.moe_linear(act, self.down, plan, rows, tiles, out=y)
        ops.moe_combine(y, wt, place_of, terms[0])
        if self.shared is not None:
            act_s = self.shared.forward(rt, x, "moe_shared")
            if shared_sums:
                ops.linear_sums(act_s, self.shared.down, out=terms[1:])
            else:
                ops.linear(act_s, self.shared.down, out=terms[1])
        return terms


@register_feed_forward("table_experts")
class TableExperts(FeedForward):
    """A mixture of small gated feed-forwards down_e(act(gate_e x) * up_e x), no biases, without a router: an
    integer table [vocab_size, top] names the experts of every token id (the entries of a row differ); each counts
    1 / top, and the result is the weighted sum in float32.

    Grouping, the experts' products and the sum are the routed mixtures' kernels (``csrc/moe.hip``); the table is
    read on the device by the step's token ids, so the launches of a step do not depend on its tokens.
    params: hidden_size, vocab_size, experts, top, ff, activation ("silu")."""

    graph_safe = True
    tape_safe = True
    writes_into = True
    reads_batch = True

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        p = spec.params
        H, V, E, top, ff = (int(p[k]) for k in ("hidden_size", "vocab_size", "experts", "top", "ff"))
        w = {"table": WeightSpec((V, top), kind="int", high=E)}
        for e in range(E):
            w[f"gate_{e}"] = WeightSpec((ff, H))
            w[f"up_{e}"] = WeightSpec((ff, H))
            w[f"down_{e}"] = WeightSpec((H, ff))
        return w

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden, self.experts, self.top, self.ff = int(p["hidden_size"]), int(p["experts"]), int(p["top"]), int(p["ff"])
        self.activation = str(p.get("activation", "silu"))
        if not (0 < self.top <= self.experts):
            raise ValueError(f"table_experts: top {self.top} of {self.experts} experts")
        self.table = weights["table"].to(torch.int32).contiguous()
        E = self.experts
        self.gate_up = torch.stack([torch.cat([weights[f"gate_{e}"], weights[f"up_{e}"].to(weights[f"gate_{e}"].dtype)])
                                    for e in range(E)]).contiguous()
        self.down = torch.stack([weights[f"down_{e}"] for e in range(E)]).contiguous()

    def step_rows(self, rows: int, kind: str) -> int:
        return ProductRows.step_rows(rows, kind)

    def forward(self, x: torch.Tensor, batch=None, out=None) -> torch.Tensor:
        if batch is None:
            raise ValueError("table_experts: the step's token ids are needed")
        n, E, top, ff, rt = x.shape[0], self.experts, self.top, self.ff, self.rt
        pairs = n * top
        idx = rt.buffer("moe_choice", (n, top), torch.int32)
        wt = rt.buffer("moe_weight", (n, top), torch.float32)
        ops.moe_route_table(batch.token_ids, self.table, E, idx, wt)
        rows = ops.moe_tile_rows(x.dtype, self.gate_up.dtype, (self.hidden, ff), pairs, E)
        tiles = ops.moe_max_tiles(pairs, E, rows)
        plan = rt.buffer("moe_plan", (1 + 3 * tiles,), torch.int32)
        order = rt.buffer("moe_order", (pairs,), torch.int32)
        place_of = rt.buffer("moe_place", (pairs,), torch.int32)
        ops.moe_group(idx, E, rows, plan, order, place_of)
        gu = rt.buffer("moe_gate_up", (pairs, 2 * ff), torch.float32)
        ops.moe_linear(x, self.gate_up, plan, rows, tiles, out=gu, source=order, source_div=top)
        act = rt.buffer("moe_act", (pairs, ff))
        ops.gated_act(gu[:, :ff], gu[:, ff:], self.activation, out=act)
        y = rt.buffer("moe_out_rows", (pairs, self.hidden), torch.float32)
        ops.moe_linear(act, self.down, plan, rows, tiles, out=y)
        if out is None:
            out = rt.buffer("moe_out", (n, self.hidden), torch.float32)
        return ops.moe_combine(y, wt, place_of, out)


@register_feed_forward("scored_experts")
class ScoredExperts(FeedForward):
    """A mixture of small gated feed-forwards down_e(silu(gate_e h) * up_e h), no biases, of which every token uses
    ``top``, plus, optionally, a shared one that every token uses.

    Router: z = W_router x in float32, s = sigmoid(z): every expert is scored by itself.  The ``top`` experts with the
    largest scores are chosen (the lowest index among equals); their weights are the scores, not renormalised.  The
    weight multiplies the expert's INPUT: the result is the sum of expert_e(s_e x) over the chosen experts.  An
    expert is linear before its activation, so the kernels compute silu(s g) * (s u) from g = gate_e x and u = up_e x
    (``ops.moe_weighted_glu``) instead of scaling rows of x.  The shared expert's output is multiplied by
    sigmoid(w_sg . x), one number a token (``shared_gate``); its row is stacked under the router's, one product.

    Routing, grouping and the experts' products run on the device as for the other mixtures (``csrc/moe.hip``): the
    launches of a step do not depend on what the tokens choose.  The result is float32 [n, hidden].
    params: hidden_size, experts, top, ff, shared_ff (0: none), shared_gate (whether the shared expert is gated)."""

    graph_safe = True
    tape_safe = True
    writes_into = True

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        p = spec.params
        H, E, ff, sff = int(p["hidden_size"]), int(p["experts"]), int(p["ff"]), int(p.get("shared_ff", 0) or 0)
        w = {"router": WeightSpec((E, H))}
        for e in range(E):
            w[f"gate_{e}"] = WeightSpec((ff, H))
            w[f"up_{e}"] = WeightSpec((ff, H))
            w[f"down_{e}"] = WeightSpec((H, ff))
        if sff:
            w.update({"shared_gate": WeightSpec((sff, H)), "shared_up": WeightSpec((sff, H)),
                      "shared_down": WeightSpec((H, sff))})
            if p.get("shared_gate", False):
                w["shared_sg"] = WeightSpec((1, H))
        return w

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden, self.experts, self.top, self.ff = int(p["hidden_size"]), int(p["experts"]), int(p["top"]), int(p["ff"])
        if not (0 < self.top <= self.experts):
            raise ValueError(f"scored_experts: top {self.top} of {self.experts} experts")
        E = self.experts
        self.sff = int(p.get("shared_ff", 0) or 0)
        self.gated_shared = bool(self.sff and p.get("shared_gate", False))
        # the router's rows, then the shared expert's gate row, padded to a multiple of 8 rows: one product
        rows = E + (1 if self.gated_shared else 0)
        r = weights["router"]
        stacked = torch.zeros((-(-rows // 8) * 8, self.hidden), dtype=r.dtype, device=r.device)
        stacked[:E] = r
        if self.gated_shared:
            stacked[E] = weights["shared_sg"].reshape(-1).to(r.dtype)
        self.router = stacked
        self.gate_up = torch.stack([torch.cat([weights[f"gate_{e}"], weights[f"up_{e}"].to(weights[f"gate_{e}"].dtype)])
                                    for e in range(E)]).contiguous()
        self.down = torch.stack([weights[f"down_{e}"] for e in range(E)]).contiguous()
        self.shared = None
        if self.sff:
            self.shared = GatedMLP(PartSpec("gated_mlp", {"hidden_size": self.hidden, "intermediate_size": self.sff,
                                                          "activation": "silu"}),
                                   {"gate": weights["shared_gate"], "up": weights["shared_up"], "down": weights["shared_down"]}, rt)

    def step_rows(self, rows: int, kind: str) -> int:
        return ProductRows.step_rows(rows, kind)

    def forward(self, x: torch.Tensor, out=None) -> torch.Tensor:
        n, E, top, ff, rt = x.shape[0], self.experts, self.top, self.ff, self.rt
        pairs = n * top
        z = ops.linear(x, self.router, out=rt.buffer("moe_logits", (n, self.router.shape[0]), torch.float32))
        idx = rt.buffer("moe_choice", (n, top), torch.int32)
        wt = rt.buffer("moe_weight", (n, top), torch.float32)
        ops.moe_route_sigmoid(z, E, top, idx, wt)
        rows = ops.moe_tile_rows(x.dtype, self.gate_up.dtype, (self.hidden, ff), pairs, E)
        tiles = ops.moe_max_tiles(pairs, E, rows)
        plan = rt.buffer("moe_plan", (1 + 3 * tiles,), torch.int32)
        order = rt.buffer("moe_order", (pairs,), torch.int32)
        place_of = rt.buffer("moe_place", (pairs,), torch.int32)
        ops.moe_group(idx, E, rows, plan, order, place_of)
        gu = rt.buffer("moe_gate_up", (pairs, 2 * ff), torch.float32)
        ops.moe_linear(x, self.gate_up, plan, rows, tiles, out=gu, source=order, source_div=top)
        act = rt.buffer("moe_act", (pairs, ff))
        ops.moe_weighted_glu(gu, wt, order, ff, out=act)
        y = rt.buffer("moe_out_rows", (pairs, self.hidden), torch.float32)
        ops.moe_linear(act, self.down, plan, rows, tiles, out=y)
        shared = None
        if self.shared is not None:
            shared = self.shared.forward(x, out=rt.buffer("moe_shared_out", (n, self.hidden), torch.float32))
        if out is None:
            out = rt.buffer("moe_out", (n, self.hidden), torch.float32)
        return ops.moe_sum_shared(y, place_of, top, out, shared=shared, gate=z[:, E] if self.gated_shared else None)
