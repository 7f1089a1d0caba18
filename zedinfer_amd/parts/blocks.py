"""Block arrangements."""
from __future__ import annotations

from typing import Optional

import torch

from .. import ops

from .base import Block, LayerMemory, Runtime, register_block


@register_block("prenorm")
class PreNormBlock(Block):
    """h += mixer(norm_in(h)); h += feed_forward(norm_post(h))
    (reference: src/frontend/models/transformer_forward.cpp:63-149).  The residual stream is
    float32 and every add into it happens inside the norm that follows it."""

    graph_safe = True
    tape_safe = True

    norm_names = ("input", "post_mixer")

    def __init__(self, norms, mixer, feed_forward, rt: Runtime):
        self.norm_in = norms["input"]
        self.norm_post = norms["post_mixer"]
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.has_ff = getattr(feed_forward, "kind", "") != "none"      # without one the mixer's addition is handed on
        self.rt = rt

    def forward(self, resid: torch.Tensor, delta: Optional[torch.Tensor], batch, memory: LayerMemory):
        x = self.norm_in.add_forward(resid, delta) if delta is not None else self.norm_in.forward(resid)
        a = self.mixer.forward(x, batch, memory)
        if not self.has_ff:
            return a
        y = self.norm_post.add_forward(resid, a)
        if self.feed_forward.reads_batch:
            return self.feed_forward.forward(y, batch=batch)
        return self.feed_forward.forward(y)


@register_block("parallel")
class ParallelBlock(Block):
    """n = norm(h); h += mixer(n) + feed_forward(n): one norm, and both sublayers read its output.  The two
    additions are handed on as a stack of float32 terms that the next norm adds into the float32 residual stream,
    mixer first.  A sublayer that takes ``out=`` (``writes_into``) writes its term in place; any other result is
    brought into the stack (a stack of partial sums added up, a bfloat16 result widened).  The feed-forward may be
    the kind "none"."""

    graph_safe = True
    tape_safe = True

    norm_names = ("input",)

    def __init__(self, norms, mixer, feed_forward, rt: Runtime):
        self.norm_in = norms["input"]
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.has_ff = getattr(feed_forward, "kind", "") != "none"
        self.rt = rt
        # a term that has to be copied into the stack is copied by a torch operator, which a tape does not hold
        self.tape_safe = all(getattr(p, "writes_into", False) for p in ((mixer, feed_forward) if self.has_ff else (mixer,)))

    def _term(self, slot: torch.Tensor, part, *args):
        if getattr(part, "writes_into", False):
            part.forward(*args, out=slot)
            return
        y = part.forward(*args)
        if y.dim() == 3:
            ops.reduce_sums(y, out=slot)
        else:
            slot.copy_(y)

    def forward(self, resid: torch.Tensor, delta: Optional[torch.Tensor], batch, memory: LayerMemory):
        x = self.norm_in.add_forward(resid, delta) if delta is not None else self.norm_in.forward(resid)
        n, H = resid.shape
        terms = self.rt.buffer("parallel_terms", (2 if self.has_ff else 1, n, H), torch.float32)
        self._term(terms[0], self.mixer, x, batch, memory)
        if self.has_ff:
            if self.feed_forward.reads_batch:
                raise ValueError("the parallel block hands its feed-forward the rows alone")
            self._term(terms[1], self.feed_forward, x)
        return terms


@register_block("output_norm")
class OutputNormBlock(Block):
    """h += norm_mixer(mixer(h)); h += norm_ff(feed_forward(h)): the sublayers read the residual stream itself (its
    rounding to the activation type, where that is not float32) and the norm sits on each sublayer's output.  The
    norms must offer ``add_normed`` (the layer norm does).  Nothing is left pending: the stream is whole when the
    block returns.  The rounded copy of the stream that the last norm left is handed to the next block of the kind
    through ``batch.shared``, which holds for one run of the model.  The feed-forward may be the kind "none"."""

    graph_safe = True
    tape_safe = True

    norm_names = ("mixer_out", "ff_out")
    SHARED = "output_norm_block.resid_copy"

    def __init__(self, norms, mixer, feed_forward, rt: Runtime):
        self.norm_mixer = norms["mixer_out"]
        self.norm_ff = norms["ff_out"]
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.has_ff = getattr(feed_forward, "kind", "") != "none"
        self.rt = rt

    def _copy_of(self, resid: torch.Tensor, batch) -> torch.Tensor:
        if self.rt.dtype == torch.float32:
            return resid
        shared = getattr(batch, "shared", None)
        x = shared.get(self.SHARED) if shared is not None else None
        if x is None:
            x = ops.convert(resid, self.rt.buffer("resid_copy", tuple(resid.shape), self.rt.dtype))
        return x

    def forward(self, resid: torch.Tensor, delta: Optional[torch.Tensor], batch, memory: LayerMemory):
        if delta is not None:       # a block of another kind before this one left an addition pending
            for term in (delta if delta.dim() == 3 else (delta,)):
                ops.add(resid, term, out=resid)
        x = self._copy_of(resid, batch)
        a = self.mixer.forward(x, batch, memory)
        x = self.norm_mixer.add_normed(resid, a)
        if self.has_ff:
            kw = {"batch": batch} if self.feed_forward.reads_batch else {}
            f = self.feed_forward.forward(x if x is not None else resid, **kw)
            x = self.norm_ff.add_normed(resid, f)
        shared = getattr(batch, "shared", None)
        if shared is not None:
            shared[self.SHARED] = x
        return None


@register_block("sandwich")
class SandwichBlock(Block):
    """h += norm_mixer_out(mixer(norm_in(h))); h += norm_ff_out(feed_forward(norm_ff_in(h))): a norm before and a
    norm after each sublayer.  The norms on the outputs must offer ``add_normed`` (the RMS norm does): the output's
    norm, the addition into the float32 stream and the norm that the feed-forward reads are one launch.  Nothing is
    left pending: the stream is whole when the block returns.  The feed-forward may be the kind "none" (its two
    norms are then the kind "none" too).  When the model says which norm the next block runs first
    (``batch.shared["next_input_norm"]``) and that norm is of the same kind, the block's last launch makes it too and
    hands the rows on (``batch.shared[SHARED]``: the norm and its rows), which the next block of the kind takes up."""

    graph_safe = True
    tape_safe = True

    norm_names = ("input", "mixer_out", "ff_in", "ff_out")
    SHARED = "sandwich_block.normed_input"

    def __init__(self, norms, mixer, feed_forward, rt: Runtime):
        self.norm_in, self.norm_mixer_out = norms["input"], norms["mixer_out"]
        self.norm_ff_in, self.norm_ff_out = norms["ff_in"], norms["ff_out"]
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.has_ff = getattr(feed_forward, "kind", "") != "none"
        self.rt = rt

    def forward(self, resid: torch.Tensor, delta: Optional[torch.Tensor], batch, memory: LayerMemory):
        shared = getattr(batch, "shared", None)
        ready = shared.pop(self.SHARED, None) if shared is not None else None
        if delta is not None:
            x = self.norm_in.add_forward(resid, delta)
        elif ready is not None and ready[0] is self.norm_in:
            x = ready[1]                      # the block before made this norm in its last launch
        else:
            x = self.norm_in.forward(resid)
        then = shared.get("next_input_norm") if shared is not None else None
        if then is not None and not self._same_kind(then):
            then = None
        a = self.mixer.forward(x, batch, memory)
        if not self.has_ff:
            out = self.norm_mixer_out.add_normed(resid, a, then=then)
        else:
            y = self.norm_mixer_out.add_normed(resid, a, then=self.norm_ff_in)
            kw = {"batch": batch} if self.feed_forward.reads_batch else {}
            f = self.feed_forward.forward(y, **kw)
            out = self.norm_ff_out.add_normed(resid, f, then=then)
        if then is not None:
            shared[self.SHARED] = (then, out)
        return None

    def _same_kind(self, norm) -> bool:
        last = self.norm_ff_out if self.has_ff else self.norm_mixer_out
        return (type(norm) is type(last) and getattr(norm, "add_one", None) == getattr(last, "add_one", None)
                and getattr(norm, "weight", None) is not None and norm.weight.dtype == last.weight.dtype
                and getattr(norm, "out_dtype", None) is None)
