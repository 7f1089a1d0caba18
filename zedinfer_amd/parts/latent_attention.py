"""Latent attention: keys and values made from one short latent per token."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.forward_config import PartSpec
from ..weights.loader import WeightSpec
from .base import (KEY_BOUND_PLANNER, PAGE, KVCacheRequest, LayerMemory, Mixer, PageTensor, POSITION_ENCODINGS, Runtime,
                   StepPlanner, register_mixer)
from .rows import ProductRows


def latent_cache_request(kind: str, rank: int, rot: int, window: int = 0) -> KVCacheRequest:
    """What latent attention keeps in a page: the normed latents [slot][rank] and the rotated key parts
    [slot][rot] that all heads share."""
    return KVCacheRequest(kind, int(window), (("latent", PageTensor((PAGE, int(rank)))),
                                              ("key_part", PageTensor((PAGE, int(rot))))))


@register_mixer("latent_attention")
class LatentAttention(Mixer):
    """Causal softmax attention, over all keys or a sliding window, whose keys and values are made from a latent.

    Per token: (d_1 .. d_rank+rot) = W_dkv x; c = rms_norm(d_1..rank) * g is the latent, the last ``rot`` values,
    turned by the position, are a key part kr shared by all heads.  Head h's query is (q_plain [dim], q_rot [rot],
    turned), its key for token j (W_uk_h c_j, kr_j), its value W_uv_h c_j; score = (q . k) * scale; the window lets
    position i see j with 0 <= i - j < window.  Only c and kr are cached.  The kernels never make keys or values:
    q_plain is carried through W_uk_h once a token and head, the attended latents through W_uv_h afterwards
    (``csrc/latent.hip``).  Scores, softmax and the sums over positions are float32; the cache holds the
    activation type.

    A layer built with ``shares_cache`` has no W_dkv: its run of the schedule names the cache of the layer whose
    latents it reads (``ScheduleStep.writes_cache`` False), and it brings its own W_uk, W_uv, queries, window.

    With ``q_rank`` the queries come through a latent of their own: c_q = rms_norm(W_dq x) * g_q, q = W_uq c_q
    (two products and a norm instead of the one product W_q x).

    ``pairing`` says which of the rot_dim dims a checkpoint pairs: "interleaved" (2i with 2i + 1, what the kernels
    turn; the default) or "halves" (i with i + rot_dim / 2: the turned rows of the query and key projections are
    reordered at load, the same way in both, which changes no score).

    params: hidden_size, heads, dim, rot_dim, vdim, kv_rank, scale, window (0: all keys), eps, shares_cache, q_rank
    (0: none), pairing, position (a PartSpec of an encoding that hands over ``pair_table``: neighbouring pairs turn)."""

    graph_safe = True
    tape_safe = True
    padding_safe = True      # padding has no place in the cache and no real token sees it
    writes_into = True

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        p = spec.params
        H, nh, dim, rot, vdim, rank = (int(p[k]) for k in ("hidden_size", "heads", "dim", "rot_dim", "vdim", "kv_rank"))
        w = {"uk": WeightSpec((nh * dim, rank)), "uv": WeightSpec((nh * vdim, rank)), "o": WeightSpec((H, nh * vdim))}
        q_rank = int(p.get("q_rank", 0) or 0)
        if q_rank:
            w.update({"dq": WeightSpec((q_rank, H)), "dq_norm": WeightSpec((q_rank,), init="ones"),
                      "uq": WeightSpec((nh * (dim + rot), q_rank))})
        else:
            w["q"] = WeightSpec((nh * (dim + rot), H))
        if not p.get("shares_cache", False):
            w["dkv"] = WeightSpec((rank + rot, H))
            w["dkv_norm"] = WeightSpec((rank,), init="ones")
        return w

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden, self.nh, self.dim, self.rot, self.vdim, self.rank = (
            int(p[k]) for k in ("hidden_size", "heads", "dim", "rot_dim", "vdim", "kv_rank"))
        self.scale = float(p["scale"])
        self.window = int(p.get("window", 0) or 0)
        self.eps = float(p.get("eps", 1e-6))
        self.shares_cache = bool(p.get("shares_cache", False))
        if self.rot % 2:
            raise ValueError(f"latent_attention: rot_dim {self.rot} must be even")
        pos_spec: PartSpec = p["position"]
        self.position = POSITION_ENCODINGS.get(pos_spec.kind)(pos_spec, {}, rt)
        if self.rot and (not hasattr(self.position, "pair_table") or self.position.rotary_dim != self.rot):
            raise ValueError("latent_attention: the position encoding must turn neighbouring pairs of all rot_dim dims")
        self.uk, self.uv, self.o = weights["uk"], weights["uv"], weights["o"]
        self.q_rank = int(p.get("q_rank", 0) or 0)
        pairing = str(p.get("pairing", "interleaved"))
        if pairing not in ("interleaved", "halves"):
            raise ValueError(f"latent_attention: unknown pairing {pairing!r}")
        # pairs (i, i + rot/2) of a checkpoint become the neighbours (2i, 2i + 1) that the kernels turn
        order = None
        if pairing == "halves" and self.rot:
            half = self.rot // 2
            order = torch.tensor([j // 2 + (j % 2) * half for j in range(self.rot)], dtype=torch.long, device=self.uk.device)
        q_w = weights["uq"] if self.q_rank else weights["q"]
        if order is not None:
            per_head = q_w.view(self.nh, self.dim + self.rot, q_w.shape[1]).clone()
            per_head[:, self.dim:] = per_head[:, self.dim:][:, order]
            q_w = per_head.reshape(self.nh * (self.dim + self.rot), q_w.shape[1]).contiguous()
        self.q = q_w
        if self.q_rank:
            self.dq, self.dq_norm = weights["dq"], weights["dq_norm"]
        # a bfloat16 cache of sizes the matrix-core kernel takes goes there; everything else to the plain kernel
        self.cores = (rt.device.type == "cuda" and rt.dtype == torch.bfloat16
                      and ops.latent_attention_cores_supported(rt.dtype, self.rank, self.rot))
        self.units = ops.compute_units() if rt.device.type == "cuda" else 256
        # the heads' blocks of W_uk with the contraction running fastest, for the matrix cores
        self.uk_t = None
        if self.uk.dtype == torch.bfloat16 and self.dim % 8 == 0:
            self.uk_t = self.uk.view(self.nh, self.dim, self.rank).transpose(1, 2).contiguous()
        if not self.shares_cache:
            self.dkv = weights["dkv"]
            if order is not None:
                self.dkv = torch.cat([self.dkv[:self.rank], self.dkv[self.rank:][order]]).contiguous()
            self.dkv_norm = weights["dkv_norm"]

    def cache_request(self) -> Optional[KVCacheRequest]:
        return latent_cache_request("window" if self.window > 0 else "full", self.rank, self.rot, self.window)

    def step_rows(self, rows: int, kind: str) -> int:
        return ProductRows.step_rows(rows, kind)

    def planner(self) -> Optional[StepPlanner]:
        """Without a window the cut of a tile's keys over workgroups is sized by the most keys a token sees."""
        return KEY_BOUND_PLANNER if self.window <= 0 else None

    def forward(self, x: torch.Tensor, batch, memory: LayerMemory, out=None) -> torch.Tensor:
        n, rt = x.shape[0], self.rt
        view = batch.groups[memory.group]
        table = self.position.pair_table(batch) if self.rot else None
        c_cache, kr_cache = memory.tensors["latent"], memory.tensors["key_part"]
        if memory.writes:
            if self.shares_cache:
                raise ValueError("latent_attention: a layer without W_dkv cannot write a cache")
            dkv = ops.linear(x, self.dkv, out=rt.buffer("latent_dkv", (n, self.rank + self.rot), torch.float32))
            ops.latent_store(dkv, self.dkv_norm, self.eps, table, view.slots, c_cache, kr_cache, self.rank, self.rot)
        if self.q_rank:
            cq = ops.linear(x, self.dq, out=rt.buffer("latent_cq", (n, self.q_rank), torch.float32))
            x = ops.rms_norm(cq, self.dq_norm, self.eps, out=rt.buffer("latent_cq_normed", (n, self.q_rank)))
        q = ops.linear(x, self.q, out=rt.buffer("latent_q", (n, self.nh * (self.dim + self.rot)), torch.float32))
        qa = rt.buffer("latent_qa", (n, self.nh, self.rank + self.rot), torch.float32)
        ops.latent_query(q, self.uk, table, self.nh, self.dim, self.rank, self.rot, out=qa, w_uk_t=self.uk_t)
        o = rt.buffer("latent_attended", (n, self.nh, self.rank), torch.float32)
        if self.cores:
            max_keys = batch.plans[KEY_BOUND_PLANNER.key].sizes["max_keys"] if self.window <= 0 else 0
            waves, chunk_keys, chunks = ops.latent_attention_cores_plan(n, batch.num_entries, self.nh, self.window, self.units,
                                                                        max_keys=max_keys)
            need = ops.latent_attention_cores_workspace(n, self.nh, self.rank, chunks)
            ws = rt.buffer("latent_chunks", (need,), torch.float32) if need else None
            ops.latent_attention_cores(qa, c_cache, kr_cache, batch.entry_start, batch.entry_len, batch.entry_past,
                                       view.block_tables, self.scale, self.window, out=o, waves=waves,
                                       chunk_keys=chunk_keys, chunks=chunks, workspace=ws)
        else:
            ops.latent_attention(qa, c_cache, kr_cache, batch.tok_seq, batch.positions, view.block_tables, self.scale,
                                 self.window, out=o)
        heads = ops.latent_value(o, self.uv, self.vdim, out=rt.buffer("latent_heads", (n, self.nh * self.vdim)))
        if out is None:
            if ops.linear_sums_supported(heads, self.o):      # few rows: the partial sums go to the norm that follows
                S = ops.linear_splits(n, self.hidden, self.nh * self.vdim)
                return ops.linear_sums(heads, self.o, out=rt.buffer("latent_out_sums", (S, n, self.hidden), torch.float32))
            out = rt.buffer("latent_out", (n, self.hidden))
        return ops.linear(heads, self.o, out=out)
