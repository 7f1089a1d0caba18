"""Token embedding and the output head."""
from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.forward_config import PartSpec
from ..weights.loader import WeightSpec
from .base import Part, Runtime, register_embedding, register_head


@register_embedding("token")
class TokenEmbedding(Part):
    """h[i,:] = table[ids[i],:], unscaled, widened into the float32 residual stream
    (reference: src/frontend/models/transformer_forward.cpp:54-60).  With ``norm_eps`` the rows are then RMS-normed
    in place, in float32, with the gain ``norm`` [hidden_size].

    Two more terms can be added to the row, in the same kernel: with ``pair`` ({"buckets", "mul_prev", "mul_cur"}) the
    row (previous id * mul_prev + id * mul_cur) mod buckets of a second table ``pair`` [buckets + 1, hidden_size] (its
    last row for a sequence's first token); the id before a step's first one is state of the request (one int32 a
    slot, which the cache manager hands to the embedding as it hands mixers theirs), so such a model's steps are not
    padded.  With ``sinusoid`` (a base, 10000 in the classic form) the fixed position vector whose entries 2i and
    2i+1 are sin and cos of position * base^(-2i/hidden_size); the frequencies are made in double precision on the
    host and the angle and its sine in double on the device.
    params: vocab_size, hidden_size, norm_eps (None), pair (None), sinusoid (None)."""

    graph_safe = True
    tape_safe = True

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        w = {"weight": WeightSpec((int(spec.params["vocab_size"]), int(spec.params["hidden_size"])))}
        if spec.params.get("norm_eps") is not None:
            w["norm"] = WeightSpec((int(spec.params["hidden_size"]),), init="ones")
        if spec.params.get("pair") is not None:
            w["pair"] = WeightSpec((int(spec.params["pair"]["buckets"]) + 1, int(spec.params["hidden_size"])))
        return w

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        self.weight = weights["weight"]
        self.vocab, self.hidden = self.weight.shape
        self.norm_eps = spec.params.get("norm_eps")
        self.norm = weights["norm"] if self.norm_eps is not None else None
        pair = spec.params.get("pair")
        self.pair = weights["pair"] if pair is not None else None
        self.buckets, self.mul_prev, self.mul_cur = ((int(pair[k]) for k in ("buckets", "mul_prev", "mul_cur"))
                                                     if pair is not None else (0, 0, 0))
        if pair is not None and self.buckets <= 0:
            raise ValueError("embedding: the pair table needs a positive number of buckets")
        base = spec.params.get("sinusoid")
        self.freq = None
        if base:
            f = [float(base) ** (-2.0 * i / self.hidden) for i in range((self.hidden + 1) // 2)]
            self.freq = torch.tensor(f, dtype=torch.float64, device=self.weight.device)
        # the step's entries and positions are read when there is more than the table
        self.reads_batch = self.pair is not None or self.freq is not None
        self.padding_safe = self.pair is None      # a padding entry would rewrite the slot it names

    def state_request(self):
        """One int32 per request (the id of the token before) when the pair table is there."""
        from .base import StateRequest
        return StateRequest((1,), torch.int32) if self.pair is not None else None

    def forward(self, ids: torch.Tensor, batch=None, memory=None) -> torch.Tensor:
        out = self.rt.buffer("resid", (ids.numel(), self.hidden), torch.float32)
        if self.reads_batch:
            if batch is None or (self.pair is not None and (memory is None or memory.state is None)):
                raise ValueError("embedding: the step's entries and the request's state are needed")
            ops.embedding_sum(ids, self.weight, out, batch.positions, pair=self.pair, buckets=self.buckets,
                              mul_prev=self.mul_prev, mul_cur=self.mul_cur,
                              state=memory.state if self.pair is not None else None, tok_seq=batch.tok_seq,
                              entry_start=batch.entry_start, entry_len=batch.entry_len, entry_slot=batch.entry_slot,
                              freq=self.freq)
        else:
            ops.embedding(ids, self.weight, out=out)
        if self.norm is not None:
            ops.rms_norm(out, self.norm, float(self.norm_eps), out=out)      # a thread rewrites what it read itself
        return out


@register_head("linear")
class LinearHead(Part):
    """logits = x . W^T in float32, no bias (reference: transformer_forward.cpp:155-156).  With
    ``tied_to`` in the spec's weights the checkpoint may leave the tensor out and the embedding
    table stands in (reference: src/frontend/models/base.cpp:410-416).
    With ``softcap`` c the logits are then bounded smoothly: c * tanh(logits / c).
    params: vocab_size, hidden_size, tied_to (tensor name or None), softcap (None)."""

    graph_safe = True
    tape_safe = True

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        return {"weight": WeightSpec((int(spec.params["vocab_size"]), int(spec.params["hidden_size"])),
                                     fallback=spec.params.get("tied_to"))}

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        self.weight = weights["weight"]
        self.vocab = self.weight.shape[0]
        cap = spec.params.get("softcap")
        self.softcap = float(cap) if cap else None

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        out = self.rt.buffer("logits", (x.shape[0], self.vocab), torch.float32)
        ops.linear(x, self.weight, out=out)
        if self.softcap is not None:
            ops.softcap(out, self.softcap)
        return out
