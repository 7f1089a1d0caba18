"""Windowed softmax attention that sees the positions before its window as means of blocks."""
from __future__ import annotations

import math
from typing import Dict, Optional

import numpy as np
import torch

from .. import ops
from ..config.forward_config import PartSpec
from ..weights.loader import WeightSpec
from .base import KEY_BOUND_PLANNER, PAGE, KVCacheRequest, LayerMemory, Mixer, PageTensor, Runtime, StepPlanner, register_mixer
from .rows import ProductRows


def ramped_frequencies(dims: int, base: float, scaling) -> tuple:
    """(f_i for the dims / 2 pairs as float32, the magnitude of cos and sin).  f_i = base^(-2i / dims); with
    ``scaling`` (factor, original, fast, slow) the pairs that turn few times within ``original`` positions are slowed
    by ``factor``, those that turn many times are kept, with a linear ramp over the pair index between the two: with
    dim(t) = dims ln(original / (2 pi t)) / (2 ln base), lo = max(floor(dim(fast)), 0), hi = min(ceil(dim(slow)),
    dims - 1), ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), f_i <- f_i / factor * ramp_i + f_i (1 - ramp_i);
    the magnitude is 0.1 ln(factor) + 1.  Computed in double precision, rounded once."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = np.power(float(base), -2.0 * i / dims)
    if not scaling:
        return f.astype(np.float32), 1.0
    missing = [k for k in ("factor", "original", "fast", "slow") if k not in scaling]
    if missing:
        raise ValueError("rotation scaling lacks " + ", ".join(missing))
    factor, orig, fast, slow = (float(scaling[k]) for k in ("factor", "original", "fast", "slow"))
    if not (factor > 0 and orig > 0 and fast > 0 and slow > 0 and base > 1):
        raise ValueError("rotation scaling: factor, original, fast and slow must be positive")

    def dim_of(turns: float) -> float:
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(dim_of(fast)), 0)
    hi = min(math.ceil(dim_of(slow)), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return (f / factor * ramp + f * (1.0 - ramp)).astype(np.float32), 0.1 * math.log(factor) + 1.0


def halves_order(size: int, turned: int) -> torch.Tensor:
    """The order that brings a head whose first ``turned`` dims pair as (2i, 2i + 1) into the layout whose pairs are
    (i, i + turned / 2): new[j] = old[order[j]]."""
    return torch.tensor(list(range(0, turned, 2)) + list(range(1, turned, 2)) + list(range(turned, size)), dtype=torch.long)


@register_mixer("pooled_window_attention")
class PooledWindowAttention(Mixer):
    """Grouped-query softmax attention: position i sees j with 0 <= i - j < window and, beside these, one key and one
    value for each block of ``pool`` positions that lies wholly before the window (b pool + pool - 1 <= i - window):
    the means of the block's keys and values as the cache holds them.  Tokens and blocks share one softmax; positions
    that have left the window and whose block is not yet whole behind it are not seen.

    Keys have ``dim`` values a head and values ``vdim``.  Optional: an RMS norm of every query and key head with one
    gain vector each (``qk_norm``); a rotation of the first ``rotary_dim`` dims of q and k (frequencies from ``theta``,
    stretched by ``scaling``, see ``ramped_frequencies``); a rotation of every value by its own position over all its
    dims, undone on the head's result by the query's position (``rotate_values``: what a head then sums are values in
    the query's own frame).  ``pairing`` says which dims a checkpoint pairs: "halves" (i with i + R/2, what the
    kernels turn) or "interleaved" (2i with 2i + 1: the rows of the projections and the gains are reordered at load,
    which changes no score and no result).

    The token cache is a window's (pages return as the window passes; it also keeps a block's positions until the
    block is whole); the blocks' means live in a cache of one row for every ``pool`` positions, kept for good.

    params: hidden_size, heads, kv_heads, dim, vdim, scale, window (0: all positions), pool (0: no blocks), qk_norm,
    eps, rotary_dim (0: none), theta, scaling, rotate_values, pairing."""

    graph_safe = True
    tape_safe = True
    padding_safe = True      # padding has no place in either cache and no real token sees it
    writes_into = True
    # Where the matrix-core kernel takes the sizes: entries that bring at least this many tokens (portions of prompts)
    # a tile of queries a workgroup; shorter ones (decoded tokens), which fit one tile, with their keys cut over
    # workgroups and merged.  Everything else goes to the kernel that deals a token's keys over four wavefronts.
    LONG_ENTRY = 8

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        p = spec.params
        H, nh, nkv, d, vd = (int(p[k]) for k in ("hidden_size", "heads", "kv_heads", "dim", "vdim"))
        w = {"q": WeightSpec((nh * d, H)), "k": WeightSpec((nkv * d, H)), "v": WeightSpec((nkv * vd, H)),
             "o": WeightSpec((H, nh * vd))}
        if p.get("qk_norm", False):
            w.update({"q_norm": WeightSpec((d,), init="ones"), "k_norm": WeightSpec((d,), init="ones")})
        return w

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden, self.nh, self.nkv, self.d, self.vd = (int(p[k]) for k in ("hidden_size", "heads", "kv_heads", "dim", "vdim"))
        if self.nh % self.nkv:
            raise ValueError(f"pooled_window_attention: {self.nh} heads are not a multiple of {self.nkv} key/value heads")
        self.scale = float(p["scale"])
        self.window, self.pool = int(p.get("window", 0) or 0), int(p.get("pool", 0) or 0)
        if self.window <= 0:
            self.pool = 0       # all positions are seen themselves
        self.eps = float(p.get("eps", 1e-6))
        self.rot = int(p.get("rotary_dim", 0) or 0)
        self.rotate_values = bool(p.get("rotate_values", False))
        if self.rot % 2 or self.rot > self.d or (self.rotate_values and self.vd % 2):
            raise ValueError("pooled_window_attention: rotated dims must be even and within the head")
        pairing = str(p.get("pairing", "halves"))
        if pairing not in ("halves", "interleaved"):
            raise ValueError(f"pooled_window_attention: unknown pairing {pairing!r}")
        q, k, v, o = weights["q"], weights["k"], weights["v"], weights["o"]
        self.q_gain = self.k_gain = None
        if p.get("qk_norm", False):
            self.q_gain, self.k_gain = weights["q_norm"].float(), weights["k_norm"].float()
        if pairing == "interleaved":
            if self.rot:
                order = halves_order(self.d, self.rot).to(q.device)
                q = q.view(self.nh, self.d, self.hidden)[:, order].reshape(self.nh * self.d, self.hidden)
                k = k.view(self.nkv, self.d, self.hidden)[:, order].reshape(self.nkv * self.d, self.hidden)
                if self.q_gain is not None:
                    self.q_gain, self.k_gain = self.q_gain[order], self.k_gain[order]
            if self.rotate_values:
                order = halves_order(self.vd, self.vd).to(v.device)
                v = v.view(self.nkv, self.vd, self.hidden)[:, order].reshape(self.nkv * self.vd, self.hidden)
                o = o.view(self.hidden, self.nh, self.vd)[:, :, order].reshape(self.hidden, self.nh * self.vd)
        if self.q_gain is not None:
            self.q_gain, self.k_gain = self.q_gain.contiguous(), self.k_gain.contiguous()
        width = (self.nh + self.nkv) * self.d + self.nkv * self.vd
        stacked = torch.zeros((-(-width // 8) * 8, self.hidden), dtype=q.dtype, device=q.device)     # rows to a multiple of 8
        stacked[:width] = torch.cat([q, k.to(q.dtype), v.to(q.dtype)])
        self.qkv, self.width, self.o = stacked, width, o.contiguous()
        self.cores = rt.device.type == "cuda" and ops.pooled_attention_cores_supported(rt.dtype, self.nh, self.nkv, self.d, self.vd)
        self.long_entry = min(self.LONG_ENTRY, ops.hybrid.POOLED_ROWS // (self.nh // self.nkv) + 1)
        self.units = ops.compute_units() if rt.device.type == "cuda" else 256
        self.table_key = self.vtable_key = None
        if self.rot:
            theta, scaling = float(p["theta"]), p.get("scaling")
            freqs, self.magnitude = ramped_frequencies(self.rot, theta, scaling)
            self.inv_freq = torch.from_numpy(freqs).to(rt.device)
            self.table_key = ("ramped_rotation", self.rot, theta, tuple(sorted((str(a), float(b)) for a, b in scaling.items())) if scaling else None)
        if self.rotate_values:
            theta = float(p["theta"])
            self.v_inv_freq = torch.from_numpy(ramped_frequencies(self.vd, theta, None)[0]).to(rt.device)
            self.vtable_key = ("ramped_rotation", self.vd, theta, None)

    # ---- what the cache manager has to provide ---------------------------------------------------------------------
    def cache_request(self) -> Optional[KVCacheRequest]:
        tensors = (("k", PageTensor((PAGE, self.nkv, self.d))), ("v", PageTensor((PAGE, self.nkv, self.vd))))
        if self.window <= 0:
            return KVCacheRequest("full", 0, tensors)
        # a block's positions stay until the block is whole: the cache's window is at least a block long
        return KVCacheRequest("window", max(self.window, self.pool), tensors)

    def side_cache_requests(self) -> Dict[str, KVCacheRequest]:
        if self.pool <= 0:
            return {}
        return {"blocks": KVCacheRequest("full", 0, (("k", PageTensor((PAGE, self.nkv, self.d), torch.float32)),
                                                     ("v", PageTensor((PAGE, self.nkv, self.vd), torch.float32))),
                                         stride=self.pool)}

    def step_rows(self, rows: int, kind: str) -> int:
        return ProductRows.step_rows(rows, kind)

    def planner(self) -> Optional[StepPlanner]:
        return KEY_BOUND_PLANNER

    def _table(self, batch, key, inv_freq, magnitude):
        table = batch.shared.get(key)
        if table is None:
            out = self.rt.buffer("rotation_table_" + repr(key), (batch.num_tokens, inv_freq.numel(), 2), torch.float32)
            table = batch.shared[key] = ops.rope_table_scaled(batch.positions, inv_freq, magnitude, out=out)
        return table

    def forward(self, x: torch.Tensor, batch, memory: LayerMemory, out=None) -> torch.Tensor:
        n, rt = x.shape[0], self.rt
        view = batch.groups[memory.group]
        kc, vc = memory.tensors["k"], memory.tensors["v"]
        table = self._table(batch, self.table_key, self.inv_freq, self.magnitude) if self.rot else None
        vtable = self._table(batch, self.vtable_key, self.v_inv_freq, 1.0) if self.rotate_values else None
        if ops.linear_sums_supported(x, self.qkv) and self.qkv.shape[0] == self.width:
            # few rows: the kernel that norms and stores adds the product's partial sums itself
            S = ops.linear_splits(n, self.width, self.hidden)
            proj = ops.linear_sums(x, self.qkv, out=rt.buffer("pooled_qkv_sums", (S, n, self.width), torch.float32))
        else:
            proj = ops.linear(x, self.qkv, out=rt.buffer("pooled_qkv", (n, self.qkv.shape[0]), torch.float32))[:, :self.width]
        q = rt.buffer("pooled_q", (n, self.nh * self.d))
        writes = memory.writes
        ops.norm_rope_store(proj, self.q_gain, self.k_gain, self.eps, table, vtable,
                            view.slots if writes else None, kc if writes else None, vc if writes else None,
                            self.nh, self.nkv, self.d, self.vd, q_out=q)
        blocks = memory.sides.get("blocks") if self.pool > 0 else None
        kp = vp = ptab = None
        if blocks is not None:
            bview = batch.groups[blocks.group]
            kp, vp, ptab = blocks.tensors["k"], blocks.tensors["v"], bview.block_tables
            if writes:
                ops.pool_blocks(kc, vc, kp, vp, bview.slots, batch.tok_seq, batch.positions, view.block_tables, self.nkv,
                                self.d, self.vd, self.pool)
        heads = rt.buffer("pooled_heads", (n, self.nh * self.vd))
        lens = batch.host_len
        args = (self.nh, self.nkv, self.d, self.vd, self.window, self.pool, self.scale)
        if not self.cores or lens is None:
            ops.pooled_attention(q, kc, vc, kp, vp, batch.tok_seq, batch.positions, view.block_tables, ptab, *args, out=heads,
                                 vtable=vtable)
        else:
            longest, shortest = int(lens.max()), int(lens.min())
            if longest >= self.long_entry:
                ops.pooled_attention_cores(q, kc, vc, kp, vp, batch.entry_start, batch.entry_len, batch.entry_past, longest,
                                           view.block_tables, ptab, *args, out=heads, vtable=vtable, long_len=self.long_entry)
            if shortest < self.long_entry:
                max_keys = batch.plans[KEY_BOUND_PLANNER.key].sizes["max_keys"]
                chunks, per = ops.pooled_attention_cores_cut(max_keys, self.window, self.pool, self.long_entry - 1, self.units,
                                                             batch.num_entries * self.nkv)
                ws = rt.buffer("pooled_chunks", (ops.pooled_attention_cores_workspace(n, self.nh, self.vd, chunks),), torch.float32)
                ops.pooled_attention_cores(q, kc, vc, kp, vp, batch.entry_start, batch.entry_len, batch.entry_past, longest,
                                           view.block_tables, ptab, *args, out=heads, vtable=vtable, long_len=self.long_entry,
                                           chunks=chunks, chunk_blocks=per, workspace=ws, tok_seq=batch.tok_seq)
        if out is None:
            if ops.linear_sums_supported(heads, self.o):      # few rows: the partial sums go to the norm that follows
                S = ops.linear_splits(n, self.hidden, self.nh * self.vd)
                return ops.linear_sums(heads, self.o, out=rt.buffer("pooled_out_sums", (S, n, self.hidden), torch.float32))
            out = rt.buffer("pooled_out", (n, self.hidden))
        return ops.linear(heads, self.o, out=out)
