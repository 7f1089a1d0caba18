"""Normalisation parts."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.forward_config import PartSpec
from ..weights.loader import WeightSpec
from .base import Norm, Runtime, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    """y = w * x * rsqrt(mean(x^2) + eps); with ``add_one`` the weight is (1 + w)
    (reference: src/backend/ops/rms_norm/cpu/rms_norm_cpu.cpp:14-29).
    With ``scalar`` the checkpoint holds ONE number (a tensor without axes) that multiplies every coordinate; it is
    spread over ``dim`` values at load, so the kernels are the same.  ``out_dtype`` "float32": the normed rows leave
    in float32 whatever the engine's activation type (for a reader that works on them in float32 before any product).
    params: dim, eps, add_one (default False), scalar (False), out_dtype (None)."""

    graph_safe = True
    tape_safe = True

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        # a gain: 1 in random-weights mode (0 when the norm multiplies by 1 + w)
        shape = () if spec.params.get("scalar", False) else (int(spec.params["dim"]),)
        return {"weight": WeightSpec(shape, init="zeros" if spec.params.get("add_one", False) else "ones")}

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        self.dim = int(spec.params["dim"])
        self.eps = float(spec.params["eps"])
        self.add_one = bool(spec.params.get("add_one", False))
        self.weight = weights["weight"]
        if spec.params.get("scalar", False):
            self.weight = self.weight.reshape(1).expand(self.dim).contiguous()
        self.out_dtype = torch.float32 if spec.params.get("out_dtype") == "float32" else None

    def forward(self, x: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        out = self.rt.buffer("norm_out", (x.shape[0], self.dim), out_dtype or self.out_dtype or self.rt.dtype)
        return ops.rms_norm(x, self.weight, self.eps, out=out, add_one=self.add_one)

    def add_forward(self, resid: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
        out = self.rt.buffer("norm_out", (resid.shape[0], self.dim), self.out_dtype or self.rt.dtype)
        return ops.add_rms_norm(resid, delta, self.weight, self.eps, out=out, add_one=self.add_one)


    def add_normed(self, resid: torch.Tensor, y: torch.Tensor, then: Optional["RMSNorm"] = None) -> Optional[torch.Tensor]:
        """The norm on a sublayer's OUTPUT: resid (float32, in place) += norm(y); y is [n, dim] or a stack [S, n, dim]
        of float32 terms that are added first.  With ``then`` (the norm the next sublayer reads, of this norm's kind)
        the new rows of the stream come back normed by it, from the same launch."""
        out = None
        if then is not None:
            if then.add_one != self.add_one or then.weight.dtype != self.weight.dtype:
                raise ValueError("rmsnorm: the two norms of one launch must be of one kind")
            out = self.rt.buffer("norm_out", (resid.shape[0], self.dim), then.out_dtype or self.rt.dtype)
        return ops.normed_add_norm(resid, y, self.weight, self.eps, self.add_one, w2=then.weight if then is not None else None,
                                   eps2=then.eps if then is not None else 0.0, out=out)


@register_norm("none")
class NoNorm(Norm):
    """Stands where a block arrangement names a norm that a layer does not have (the norm before a feed-forward
    that is not there); it is never run."""

    graph_safe = True
    tape_safe = True

    def forward(self, x, out_dtype=None):
        raise ValueError("a layer without this norm was asked to run it")

    add_forward = forward


@register_norm("layernorm")
class LayerNorm(Norm):
    """y = (x - mean) / sqrt(var + eps) * w + b, var the mean of the squared deviations, all in float32.
    params: dim, eps.  Beside the norm's two usual forms it has a third, ``add_normed(resid, y)``: the norm sits on a
    sublayer's OUTPUT, resid += norm(y), and the new residual rows come back in the activation type (what the next
    sublayer's products read)."""

    graph_safe = True
    tape_safe = True

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        dim = int(spec.params["dim"])
        return {"weight": WeightSpec((dim,), init="ones"), "bias": WeightSpec((dim,), init="zeros")}

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        self.dim = int(spec.params["dim"])
        self.eps = float(spec.params["eps"])
        self.weight = weights["weight"]
        self.bias = weights["bias"].to(self.weight.dtype)

    def forward(self, x: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        out = self.rt.buffer("norm_out", (x.shape[-2], self.dim), out_dtype or self.rt.dtype)
        return ops.layer_norm(x, self.weight, self.bias, self.eps, out=out)

    def add_forward(self, resid: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
        for term in (delta if delta.dim() == 3 else (delta,)):
            ops.add(resid, term, out=resid)
        return self.forward(resid)

    def add_normed(self, resid: torch.Tensor, y: torch.Tensor, want_copy: bool = True) -> Optional[torch.Tensor]:
        """resid (float32, in place) += norm(y); y is [n, dim] or a stack [S, n, dim] of float32 terms that are added
        first.  Returns the new residual rows in the activation type, or nothing when that type is float32 (the
        stream itself serves) or no copy is wanted."""
        out = None
        if want_copy and self.rt.dtype != torch.float32:
            out = self.rt.buffer("resid_copy", (resid.shape[0], self.dim), self.rt.dtype)
        ops.layer_norm(y, self.weight, self.bias, self.eps, out=out, resid=resid)
        return out
