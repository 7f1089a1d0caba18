"""Checked launches of the kernels behind mixers with a decayed matrix state (linear attention), behind what feeds
and shifts the residual stream (an embedding summed from several tables, the token shift, re-entry of the embedding
output), behind softmax attention with capped and biased scores over normed values, and the table that names a
token's experts."""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib
from .functional import _attention_args, _check_cache, _code, _gpu, _i32, _p, _rows, _sinks, _stream
from .mixing import MOE_MAX_EXPERTS, _f32

GATE_ACTIVATIONS = {"sigmoid": 0, "silu": 1}


def _entries(what: str, *arrays: torch.Tensor) -> int:
    E = arrays[0].numel()
    for a in arrays:
        _i32(a, what + " entries", E)
    return E


def embedding_sum(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, positions: torch.Tensor,
                  pair: Optional[torch.Tensor] = None, buckets: int = 0, mul_prev: int = 0, mul_cur: int = 0,
                  state: Optional[torch.Tensor] = None, tok_seq: Optional[torch.Tensor] = None,
                  entry_start: Optional[torch.Tensor] = None, entry_len: Optional[torch.Tensor] = None,
                  entry_slot: Optional[torch.Tensor] = None, freq: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out [n, H] float32 = table[ids] (+ pair[(previous id * mul_prev + id * mul_cur) mod buckets], row ``buckets``
    at position 0) (+ the sinusoid of the position: channel j turns with ``freq[j // 2]``, float64; even channels the
    sine, odd ones the cosine).  The id before an entry's first token is read from ``state`` [slots, >= 1] int32 at
    the entry's slot, and the entry's last id is written there."""
    _gpu("embedding_sum", ids, table, out, positions, pair, state, tok_seq, entry_start, entry_len, entry_slot, freq)
    n = ids.numel()
    _i32(ids, "embedding_sum ids")
    _i32(positions, "embedding_sum positions", n)
    if table.dim() != 2 or not table.is_contiguous():
        raise ValueError("embedding_sum: the table must be a contiguous [vocab, hidden] tensor")
    V, H = table.shape
    _f32(out, "embedding_sum out", (n, H))
    if pair is not None:
        if tuple(pair.shape) != (buckets + 1, H) or not pair.is_contiguous() or buckets <= 0:
            raise ValueError(f"embedding_sum: the pair table must be a contiguous [{buckets + 1}, {H}] tensor")
        if state is None or state.dtype != torch.int32 or state.dim() != 2 or not state.is_contiguous():
            raise ValueError("embedding_sum: the pair table needs an int32 state [slots, >= 1]")
        _i32(tok_seq, "embedding_sum tok_seq", n)
        _entries("embedding_sum", entry_start, entry_len, entry_slot)
    if freq is not None and (freq.dtype != torch.float64 or not freq.is_contiguous() or freq.numel() < (H + 1) // 2):
        raise ValueError(f"embedding_sum: freq must be a contiguous float64 tensor of {(H + 1) // 2} frequencies")
    _lib.call("zi_embedding_sum", _p(out), _p(table), _code(table, "embedding_sum table"), _p(pair),
              _code(pair, "embedding_sum pair") if pair is not None else 0, _p(ids), _p(positions), _p(tok_seq),
              _p(entry_start), _p(entry_len), _p(entry_slot), _p(state), int(state.stride(0)) if state is not None else 0,
              _p(freq), n, H, V, int(buckets), int(mul_prev), int(mul_cur), _stream())
    return out


def token_shift(x: torch.Tensor, weight: torch.Tensor, state: torch.Tensor, tok_seq: torch.Tensor,
                positions: torch.Tensor, entry_start: torch.Tensor, entry_len: torch.Tensor, entry_slot: torch.Tensor,
                out: torch.Tensor) -> torch.Tensor:
    """out[t] = x[t] + (x[t-1] - x[t]) * weight per channel; nothing stands before position 0; the row before an
    entry's first one is ``state`` [slots, >= H] float32 (a column slice is fine) at the entry's slot, which then
    takes the entry's last row of x."""
    _gpu("token_shift", x, weight, state, tok_seq, positions, entry_start, entry_len, entry_slot, out)
    ldx, H = _rows(x, "token_shift x")
    ldo, Ho = _rows(out, "token_shift out")
    n = x.shape[0]
    if tuple(out.shape) != (n, H) or weight.numel() != H or not weight.is_contiguous():
        raise ValueError("token_shift: out must be [n, H] and the weight [H]")
    if state.dtype != torch.float32 or state.dim() != 2 or state.shape[1] < H or state.stride(1) != 1:
        raise ValueError(f"token_shift: the state must be float32 [slots, >= {H}] with dense rows")
    _i32(tok_seq, "token_shift tok_seq", n)
    _i32(positions, "token_shift positions", n)
    _entries("token_shift", entry_start, entry_len, entry_slot)
    _lib.call("zi_token_shift", _p(out), _code(out, "token_shift out"), ldo, _p(x), _code(x, "token_shift x"), ldx,
              _p(weight), _code(weight, "token_shift weight"), _p(state), int(state.stride(0)), _p(tok_seq), _p(positions),
              _p(entry_start), _p(entry_len), _p(entry_slot), n, H, _stream())
    return out


def stream_reenter(resid: torch.Tensor, delta: Optional[torch.Tensor] = None, again: Optional[torch.Tensor] = None,
                   row: Optional[torch.Tensor] = None) -> torch.Tensor:
    """In place on the float32 stream [n, H]: resid += delta ([n, H] or a stack [S, n, H], added in rising order)
    + again (float32 [n, H]) + row ([H]); each may be left out."""
    _gpu("stream_reenter", resid, delta, again, row)
    _f32(resid, "stream_reenter resid")
    n, H = resid.shape
    splits = stride = 0
    if delta is not None:
        if not delta.is_contiguous() or tuple(delta.shape[-2:]) != (n, H) or delta.dim() not in (2, 3):
            raise ValueError("stream_reenter: delta must be a contiguous [n, H] or [S, n, H] tensor")
        splits, stride = (int(delta.shape[0]), n * H) if delta.dim() == 3 else (1, 0)
    if again is not None:
        _f32(again, "stream_reenter again", (n, H))
    if row is not None and (row.numel() != H or not row.is_contiguous()):
        raise ValueError(f"stream_reenter: the row must be a contiguous [{H}] tensor")
    _lib.call("zi_stream_reenter", _p(resid), _p(delta), _code(delta, "stream_reenter delta") if delta is not None else 0,
              splits, stride, _p(again), _p(row), _code(row, "stream_reenter row") if row is not None else 0, n, H, _stream())
    return resid


def lowrank_decay(u: torch.Tensor, w2: torch.Tensor, bias: Optional[torch.Tensor], tau: float, out: torch.Tensor) -> torch.Tensor:
    """out [n, C] float32 = sigmoid(u . w2^T + bias)^(1 / tau) for float32 rows u [n, rank] (a column slice is
    fine), w2 [C, rank], bias [C] of w2's type."""
    _gpu("lowrank_decay", u, w2, bias, out)
    ldu, rank = _rows(u, "lowrank_decay u")
    ldo, C = _rows(out, "lowrank_decay out")
    n = u.shape[0]
    if u.dtype != torch.float32 or out.dtype != torch.float32 or out.shape[0] != n:
        raise ValueError("lowrank_decay: u and out must be float32 with one row a token")
    if tuple(w2.shape) != (C, rank) or not w2.is_contiguous():
        raise ValueError(f"lowrank_decay: w2 must be a contiguous [{C}, {rank}] tensor")
    if bias is not None and (bias.numel() != C or bias.dtype != w2.dtype or not bias.is_contiguous()):
        raise ValueError(f"lowrank_decay: the bias must be a contiguous [{C}] tensor of the weight's type")
    if not tau > 0:
        raise ValueError("lowrank_decay: tau must be positive")
    _lib.call("zi_lowrank_decay", _p(out), ldo, _p(u), ldu, _p(w2), _p(bias), _code(w2, "lowrank_decay w2"), n, C, rank,
              float(tau), _stream())
    return out


def linear_attention_state_floats(heads: int, dim: int, vdim: int) -> int:
    return int(heads) * int(dim) * int(vdim)


def linear_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, state: torch.Tensor, entry_start: torch.Tensor,
                     entry_len: torch.Tensor, entry_past: torch.Tensor, entry_slot: torch.Tensor, heads: int, dim: int,
                     vdim: int, out: torch.Tensor, decay: Optional[torch.Tensor] = None,
                     head_decay: Optional[torch.Tensor] = None, silu: bool = False, qscale: float = 1.0) -> torch.Tensor:
    """Token by token over every entry: S <- diag(a_t) S + k_t v_t^T, out_t = S^T (q_t * qscale), per head.  q, k
    [n, heads*dim] and v [n, heads*vdim] are float32 column slices of ONE projection (one row stride); the decay a_t
    is ``decay`` [n, heads*dim] float32, or ``head_decay`` [heads] float32 (one factor a head), or 1.  ``silu``: q, k
    and v pass SiLU as they are read.  ``state`` [slots, >= heads*dim*vdim] float32 (a column slice is fine) holds S
    of every request; an entry that starts its sequence (nothing in the cache yet) starts from zero."""
    _gpu("linear_attention", q, k, v, state, entry_start, entry_len, entry_past, entry_slot, out, decay, head_decay)
    n = q.shape[0]
    ld, wq = _rows(q, "linear_attention q")
    for name, t, width in (("q", q, heads * dim), ("k", k, heads * dim), ("v", v, heads * vdim)):
        ldt, w = _rows(t, f"linear_attention {name}")
        if t.dtype != torch.float32 or w != width or t.shape[0] != n or (n > 1 and ldt != ld):
            raise ValueError(f"linear_attention: {name} must be float32 [n, {width}], a column slice of the projection q is of")
    ldo, wo = _rows(out, "linear_attention out")
    if out.dtype != torch.float32 or tuple(out.shape) != (n, heads * vdim):
        raise ValueError(f"linear_attention: out must be float32 [n, {heads * vdim}]")
    ldd = 0
    if decay is not None:
        ldd, wd = _rows(decay, "linear_attention decay")
        if decay.dtype != torch.float32 or tuple(decay.shape) != (n, heads * dim):
            raise ValueError(f"linear_attention: decay must be float32 [n, {heads * dim}]")
    if head_decay is not None:
        _f32(head_decay, "linear_attention head_decay", (heads,))
    if decay is not None and head_decay is not None:
        raise ValueError("linear_attention: a decay per token or one per head, not both")
    if state.dtype != torch.float32 or state.dim() != 2 or state.stride(1) != 1 or state.shape[1] < heads * dim * vdim:
        raise ValueError(f"linear_attention: the state must be float32 [slots, >= {heads * dim * vdim}] with dense rows")
    E = _entries("linear_attention", entry_start, entry_len, entry_past, entry_slot)
    _lib.call("zi_linear_attention", _p(out), ldo, _p(q), _p(k), _p(v), max(ld, 1), _p(decay), ldd, _p(head_decay),
              _p(state), int(state.stride(0)), _p(entry_start), _p(entry_len), _p(entry_past), _p(entry_slot), E, heads, dim,
              vdim, int(bool(silu)), float(qscale), _stream())
    return out


def gate_heads(x: torch.Tensor, gate: torch.Tensor, head: int, x_head: int, activation: str, out: torch.Tensor,
               scale: float = 1.0) -> torch.Tensor:
    """out [n, W] = x * act(gate) * scale, act "sigmoid" or "silu"; gate float32 [n, W]; x holds heads of ``x_head``
    values of which the first ``head`` count (W = heads * head)."""
    _gpu("gate_heads", x, gate, out)
    ldx, wx = _rows(x, "gate_heads x")
    ldg, W = _rows(gate, "gate_heads gate")
    ldo, wo = _rows(out, "gate_heads out")
    n = x.shape[0]
    if gate.dtype != torch.float32 or W % head or wx != (W // head) * x_head or wo != W or gate.shape[0] != n \
            or out.shape[0] != n or x_head < head:
        raise ValueError("gate_heads: shapes do not agree")
    if activation not in GATE_ACTIVATIONS:
        raise ValueError(f"gate_heads: unknown activation {activation!r}")
    _lib.call("zi_gate_heads", _p(out), _code(out, "gate_heads out"), ldo, _p(x), _code(x, "gate_heads x"), ldx, x_head,
              _p(gate), ldg, n, W, head, GATE_ACTIVATIONS[activation], float(scale), _stream())
    return out


def gated_rms_norm_act(o: torch.Tensor, weight: torch.Tensor, gate: torch.Tensor, groups: int, size: int, eps: float,
                       activation: str, out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """out [n, groups * size] (dense rows; a column slice is fine) = o / rms(o over each group's ``size`` values) *
    weight [size] * act(gate) * scale; o float32 contiguous, gate float32 [n, groups * size] with dense rows."""
    _gpu("gated_rms_norm_act", o, weight, gate, out)
    n = o.shape[0]
    _f32(o, "gated_rms_norm_act o", (n, groups * size))
    if weight.numel() != size or not weight.is_contiguous():
        raise ValueError(f"gated_rms_norm_act: the weight must be a contiguous [{size}] tensor")
    ldg, gw = _rows(gate, "gated_rms_norm_act gate")
    ldo, wo = _rows(out, "gated_rms_norm_act out")
    if gate.dtype != torch.float32 or gw != groups * size or gate.shape[0] != n or wo != groups * size or out.shape[0] != n:
        raise ValueError("gated_rms_norm_act: gate and out must be [n, groups * size], the gate float32")
    if activation not in GATE_ACTIVATIONS:
        raise ValueError(f"gated_rms_norm_act: unknown activation {activation!r}")
    _lib.call("zi_gated_rmsnorm_act", _p(out), _code(out, "gated_rms_norm_act out"), ldo, _p(o), _p(weight),
              _code(weight, "gated_rms_norm_act weight"), _p(gate), ldg, n, groups, size, float(eps),
              1 if activation == "sigmoid" else 0, float(scale), _stream())
    return out


def normed_kv_store(proj: torch.Tensor, q_at: int, k_at: int, v_at: int, q_out: torch.Tensor,
                    slots: Optional[torch.Tensor], kcache: Optional[torch.Tensor], vcache: Optional[torch.Tensor],
                    nh: int, nkv: int, dim: int, vdim: int, head: int, eps: float, norm_values: bool = True) -> torch.Tensor:
    """From float32 rows of one projection (queries [nh*dim] at column ``q_at``, keys [nkv*dim] at ``k_at``, values
    [nkv*vdim] at ``v_at``): the queries into ``q_out`` [n, nh*head], keys into the paged cache at ``slots`` and
    values, each head divided by its root mean square over vdim when ``norm_values``, into the transposed value
    cache; heads of the cache hold ``head`` >= dim, vdim values, the rest zero.  A token whose slot is negative
    stores nothing; without caches only the queries are written."""
    _gpu("normed_kv_store", proj, q_out, slots, kcache, vcache)
    ld, width = _rows(proj, "normed_kv_store proj")
    n = proj.shape[0]
    if proj.dtype != torch.float32:
        raise ValueError("normed_kv_store: the projection must be float32")
    ldq, wq = _rows(q_out, "normed_kv_store q_out")
    if tuple(q_out.shape) != (n, nh * head) or head < max(dim, vdim):
        raise ValueError(f"normed_kv_store: q_out must be [n, {nh * head}] with heads of at least {max(dim, vdim)} values")
    if min(q_at, k_at, v_at) < 0 or max(q_at + nh * dim, k_at + nkv * dim, v_at + nkv * vdim) > width:
        raise ValueError("normed_kv_store: the columns lie outside the projection")
    pages = ps = 0
    if kcache is not None:
        if slots is None:
            raise ValueError("normed_kv_store: a cache needs the tokens' slots")
        _i32(slots, "normed_kv_store slots", n)
        pages, ps = _check_cache(kcache, vcache, nkv, head, q_out.dtype, "normed_kv_store")
    _lib.call("zi_normed_kv_store", _p(q_out), _code(q_out, "normed_kv_store q_out"), ldq, _p(kcache),
              _p(vcache if kcache is not None else None), _p(proj), ld, int(q_at), int(k_at), int(v_at),
              _p(slots if kcache is not None else None), pages * ps, n, nh, nkv, dim, vdim, head, max(ps, 1), float(eps),
              int(bool(norm_values)), _stream())
    return q_out


def attention_biased(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, tok_seq: torch.Tensor,
                     tok_pos: torch.Tensor, block_tables: torch.Tensor, nh: int, nkv: int, d: int, scale: float,
                     window: int = 0, out: Optional[torch.Tensor] = None, tok_index: Optional[torch.Tensor] = None,
                     sinks: Optional[torch.Tensor] = None, softcap: float = 0.0, bias: Optional[torch.Tensor] = None,
                     keep_first: int = 0) -> torch.Tensor:
    """The plain attention kernel (``ops.attention``) with its options: scores are (q . k) * scale, then
    ``softcap`` * tanh(score / ``softcap``) when the cap is positive, then plus ``bias[head, min(distance, L - 1)]``
    (float32 [nh, L]); beside the window the first ``keep_first`` positions of the sequence stay visible."""
    out, n, count, ldq, ldo, pages, ps = _attention_args("attention", q, kcache, vcache, tok_seq, tok_pos,
                                                         block_tables, nh, nkv, d, tok_index, out)
    L = 0
    if bias is not None:
        _f32(bias, "attention bias")
        if bias.dim() != 2 or bias.shape[0] != nh or bias.device != q.device:
            raise ValueError(f"attention: the bias must be float32 [{nh}, distances] on {q.device}")
        L = int(bias.shape[1])
    _lib.call("zi_attention_generic_biased", _p(out), _p(q), _code(q, "attention"), count, ldq, ldo, _p(kcache), _p(vcache),
              _p(tok_index), _p(tok_seq), _p(tok_pos), _p(block_tables), block_tables.shape[1], pages, nh, nkv, d, ps,
              int(window), float(scale), _p(_sinks(sinks, nh, q, "attention") if sinks is not None else None),
              float(softcap), _p(bias), L, int(keep_first), _stream())
    return out


def moe_route_table(ids: torch.Tensor, table: torch.Tensor, experts: int, idx: torch.Tensor, wt: torch.Tensor) -> None:
    """Token id v uses the experts ``table[v]`` (int32 [vocab, top]), each with the weight 1 / top: ``idx`` [n, top]
    and ``wt`` [n, top] as the routers leave them."""
    _gpu("moe_route_table", ids, table, idx, wt)
    n = ids.numel()
    _i32(ids, "moe_route_table ids")
    if table.dtype != torch.int32 or table.dim() != 2 or not table.is_contiguous():
        raise ValueError("moe_route_table: the table must be a contiguous int32 [vocab, top] tensor")
    V, top = table.shape
    _f32(wt, "moe_route_table wt", (n, top))
    _i32(idx, "moe_route_table idx", n * top)
    if not (0 < top <= experts <= MOE_MAX_EXPERTS):
        raise ValueError(f"moe_route_table: top {top} of {experts} experts (at most {MOE_MAX_EXPERTS})")
    _lib.call("zi_moe_route_table", _p(idx), _p(wt), _p(ids), _p(table), n, V, experts, top, _stream())
