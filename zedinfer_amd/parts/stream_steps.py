"""What a design does to the residual stream between two layers (``ScheduleStep.enter``)."""
from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.forward_config import PartSpec
from ..weights.loader import WeightSpec
from .base import Runtime, StreamStep, register_stream_step


@register_stream_step("reenter")
class Reenter(StreamStep):
    """x <- x + (the embedding output as it was before the first layer, when ``add_embedded``) + rows[row] (one row
    of a learned table ``rows`` [count, hidden_size], when ``count``): what stands at the start of every pass of a
    run of layers that is repeated with the same weights.  The addition still pending from the layer before is
    folded into the stream in the same kernel, all in float32.
    params: hidden_size, add_embedded (False), count (0: no table), row."""

    graph_safe = True
    tape_safe = True

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        count = int(spec.params.get("count", 0) or 0)
        return {"rows": WeightSpec((count, int(spec.params["hidden_size"])))} if count else {}

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        self.needs_embedded = bool(spec.params.get("add_embedded", False))
        count = int(spec.params.get("count", 0) or 0)
        self.row = None
        if count:
            r = int(spec.params["row"])
            if not (0 <= r < count):
                raise ValueError(f"reenter: row {r} of a table of {count}")
            self.row = weights["rows"][r].contiguous()

    def forward(self, resid, delta, embedded):
        if self.needs_embedded and embedded is None:
            raise ValueError("reenter: the embedding output was not kept")
        ops.stream_reenter(resid, delta, embedded if self.needs_embedded else None, self.row)
        return None
