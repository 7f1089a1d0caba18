"""Checked launches of the kernels behind a state-space mixer with one decay a (token, head), behind windowed
attention that sees the past as means of blocks, behind norms that sit on a sublayer's output, and behind experts
whose router gives independent scores."""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib
from .functional import _code, _gpu, _i32, _p, _rows, _stream
from .mixing import MOE_MAX_EXPERTS, _f32
from .sublayers import _terms

SSM_MAX_TAPS = 16
POOLED_MAX_HEAD = 512
NORMED_ADD_MAX_HIDDEN = 15360


def rope_table_scaled(pos: torch.Tensor, inv_freq: torch.Tensor, magnitude: float, out: torch.Tensor) -> torch.Tensor:
    """(cos, sin) of pos[t] * inv_freq[k], both times ``magnitude``, as float32 [n, pairs, 2]."""
    _gpu("rope_table_scaled", pos, inv_freq, out)
    n, half = pos.numel(), inv_freq.numel()
    _i32(pos, "rope_table_scaled positions", n)
    _f32(inv_freq, "rope_table_scaled inv_freq", (half,))
    _f32(out, "rope_table_scaled out", (n, half, 2))
    _lib.call("zi_rope_table_scaled", _p(out), _p(pos), _p(inv_freq), n, half, float(magnitude), _stream())
    return out


# ---- state-space mixer ----------------------------------------------------------------------------------------
def ssm_state_floats(heads: int, vdim: int, state: int, groups: int, taps: int) -> int:
    """Floats of one request's state: the convolution's tail [taps - 1, channels] first, then the matrices
    [heads, state, vdim]."""
    return (taps - 1) * (heads * vdim + 2 * groups * state) + heads * state * vdim


def ssm_prepare(proj: torch.Tensor, conv_w: torch.Tensor, conv_b: Optional[torch.Tensor], dt_bias: torch.Tensor,
                a_log: torch.Tensor, state: torch.Tensor, tok_seq: torch.Tensor, entry_start: torch.Tensor,
                entry_slot: torch.Tensor, heads: int, vdim: int, state_size: int, groups: int, taps: int,
                out: torch.Tensor) -> torch.Tensor:
    """From proj [n, z | x | B | C | dt] (float32) the row [x | B | C | dt x | decay] (float32, same width): x, B, C
    after the causal convolution (rows before an entry's first from the tail at the start of ``state``'s rows), its
    bias and SiLU; dt = softplus(dt + dt_bias); decay = exp(-exp(a_log) dt)."""
    _gpu("ssm_prepare", proj, conv_w, conv_b, dt_bias, a_log, state, tok_seq, entry_start, entry_slot, out)
    n = proj.shape[0]
    inner, gn2 = heads * vdim, 2 * groups * state_size
    width = 2 * inner + gn2 + heads
    ld, w = _rows(proj, "ssm_prepare proj")
    ldo, wo = _rows(out, "ssm_prepare out")
    if proj.dtype != torch.float32 or out.dtype != torch.float32 or w != width or wo != width or out.shape[0] != n:
        raise ValueError(f"ssm_prepare: proj and out must be float32 [n, {width}]")
    if not (1 <= taps <= SSM_MAX_TAPS):
        raise ValueError(f"ssm_prepare: at most {SSM_MAX_TAPS} taps")
    _f32(conv_w, "ssm_prepare conv_w", (inner + gn2, taps))
    if conv_b is not None:
        _f32(conv_b, "ssm_prepare conv_b", (inner + gn2,))
    _f32(dt_bias, "ssm_prepare dt_bias", (heads,))
    _f32(a_log, "ssm_prepare a_log", (heads,))
    if state.dtype != torch.float32 or state.dim() != 2 or not state.is_contiguous() or state.shape[1] < (taps - 1) * (inner + gn2):
        raise ValueError("ssm_prepare: the state must be contiguous float32 [slots, >= the tail's floats]")
    _i32(tok_seq, "ssm_prepare tok_seq", n)
    _i32(entry_start, "ssm_prepare entry_start")
    _i32(entry_slot, "ssm_prepare entry_slot", entry_start.numel())
    _lib.call("zi_ssm_prepare", _p(out), ldo, _p(proj), ld, n, _p(conv_w), _p(conv_b), _p(dt_bias), _p(a_log), _p(state),
              int(state.stride(0)), _p(tok_seq), _p(entry_start), _p(entry_slot), heads, vdim, gn2, taps, _stream())
    return out


def ssm_finish(y: torch.Tensor, x: torch.Tensor, z: torch.Tensor, skip: torch.Tensor, gain: torch.Tensor, heads: int,
               vdim: int, parts: int, eps: float, out: torch.Tensor) -> torch.Tensor:
    """out [n, heads*vdim] = norm((y + skip_h x) * silu(z)) * gain, the norm over each of ``parts`` equal parts of a
    row; y, x, z float32 [n, heads*vdim] (column slices are fine), skip [heads], gain [heads*vdim] float32."""
    _gpu("ssm_finish", y, x, z, skip, gain, out)
    n, inner = y.shape[0], heads * vdim
    lds = []
    for name, t in (("y", y), ("x", x), ("z", z)):
        ld, w = _rows(t, f"ssm_finish {name}")
        if t.dtype != torch.float32 or w != inner or t.shape[0] != n:
            raise ValueError(f"ssm_finish: {name} must be float32 [n, {inner}]")
        lds.append(ld)
    _f32(skip, "ssm_finish skip", (heads,))
    _f32(gain, "ssm_finish gain", (inner,))
    ldo, wo = _rows(out, "ssm_finish out")
    if wo != inner or out.shape[0] != n or parts <= 0 or inner % parts:
        raise ValueError("ssm_finish: out must be [n, heads*vdim], the parts equal")
    _lib.call("zi_ssm_finish", _p(out), _code(out, "ssm_finish out"), ldo, _p(y), lds[0], _p(x), lds[1], _p(z), lds[2],
              _p(skip), _p(gain), n, heads, vdim, int(parts), float(eps), _stream())
    return out


def linear_attention_grouped(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, state: torch.Tensor,
                             entry_start: torch.Tensor, entry_len: torch.Tensor, entry_past: torch.Tensor,
                             entry_slot: torch.Tensor, heads: int, share: int, dim: int, vdim: int,
                             out: torch.Tensor, single_tokens: bool = False) -> torch.Tensor:
    """Token by token over every entry, per head: S <- a_t S + k_t v_t^T, out_t = S^T q_t, where ``share`` heads in
    a row read the same q and k ([n, (heads/share)*dim]) and the decay a_t is one number a (token, head)
    ([n, heads]).  q, k, v and the decay are float32 column slices of ONE row; ``state`` [slots, >= heads*dim*vdim]
    float32 (a column slice is fine).  ``single_tokens``: every entry brings one token (the caller knows): the kernel
    that streams every head's matrix through once takes the step; its sums differ from the other's by rounding."""
    _gpu("linear_attention_grouped", q, k, v, decay, state, entry_start, entry_len, entry_past, entry_slot, out)
    n = q.shape[0]
    if share <= 0 or heads % share:
        raise ValueError("linear_attention_grouped: the heads must divide into runs that share q and k")
    ld, _ = _rows(q, "linear_attention_grouped q")
    for name, t, width in (("q", q, heads // share * dim), ("k", k, heads // share * dim), ("v", v, heads * vdim),
                           ("decay", decay, heads)):
        ldt, w = _rows(t, f"linear_attention_grouped {name}")
        if t.dtype != torch.float32 or w != width or t.shape[0] != n or (n > 1 and ldt != ld):
            raise ValueError(f"linear_attention_grouped: {name} must be float32 [n, {width}], a column slice of q's row")
    ldo, wo = _rows(out, "linear_attention_grouped out")
    if out.dtype != torch.float32 or tuple(out.shape) != (n, heads * vdim):
        raise ValueError(f"linear_attention_grouped: out must be float32 [n, {heads * vdim}]")
    if state.dtype != torch.float32 or state.dim() != 2 or state.stride(1) != 1 or state.shape[1] < heads * dim * vdim:
        raise ValueError("linear_attention_grouped: the state row is too short")
    E = entry_start.numel()
    for t in (entry_start, entry_len, entry_past, entry_slot):
        _i32(t, "linear_attention_grouped entries", E)
    _lib.call("zi_linear_attention_grouped", _p(out), ldo, _p(q), _p(k), _p(v), max(ld, 1), _p(decay), max(ld, 1), None,
              _p(state), int(state.stride(0)), _p(entry_start), _p(entry_len), _p(entry_past), _p(entry_slot), E, heads,
              dim, vdim, 0, 1.0, int(share), 1, int(bool(single_tokens)), _stream())
    return out


# ---- windowed attention over tokens and means of blocks --------------------------------------------------------
def _token_cache(kcache: torch.Tensor, vcache: torch.Tensor, nkv: int, dim: int, vdim: int, what: str):
    """keys [pages, page_size, kv_heads, dim], values [pages, page_size, kv_heads, vdim]; (pages, page_size)."""
    if kcache.dim() != 4 or not kcache.is_contiguous() or tuple(kcache.shape[2:]) != (nkv, dim):
        raise ValueError(f"{what}: the key cache must be contiguous [pages, page_size, {nkv}, {dim}]")
    pages, ps = int(kcache.shape[0]), int(kcache.shape[1])
    if tuple(vcache.shape) != (pages, ps, nkv, vdim) or not vcache.is_contiguous() or vcache.dtype != kcache.dtype:
        raise ValueError(f"{what}: the value cache must be contiguous [{pages}, {ps}, {nkv}, {vdim}] of the keys' type")
    return pages, ps


def norm_rope_store(proj: torch.Tensor, q_gain: Optional[torch.Tensor], k_gain: Optional[torch.Tensor], eps: float,
                    table: Optional[torch.Tensor], vtable: Optional[torch.Tensor], slots: Optional[torch.Tensor],
                    kcache: Optional[torch.Tensor], vcache: Optional[torch.Tensor], nh: int, nkv: int, dim: int,
                    vdim: int, q_out: torch.Tensor) -> torch.Tensor:
    """proj [n, q | k | v] float32 (or a stack of float32 partial sums): every query and key head is RMS-normed over
    its ``dim`` values with the gain (when one is given), its first R dims turn as split halves by ``table``
    [n, R/2, 2]; values turn over all their dims by ``vtable`` [n, vdim/2, 2] when that is given.  Queries go to
    ``q_out`` [n, nh*dim]; keys and values of tokens with a slot into the caches."""
    _gpu("norm_rope_store", proj, q_gain, k_gain, table, vtable, slots, kcache, vcache, q_out)
    splits, split_stride, ld, n, width = _terms(proj, "norm_rope_store proj")
    if proj.dtype != torch.float32 or width != (nh + nkv) * dim + nkv * vdim:
        raise ValueError(f"norm_rope_store: proj must be float32 [n, {(nh + nkv) * dim + nkv * vdim}]")
    if max(dim, vdim) > POOLED_MAX_HEAD:
        raise ValueError(f"norm_rope_store: heads of at most {POOLED_MAX_HEAD} values")
    for name, g in (("q_gain", q_gain), ("k_gain", k_gain)):
        if g is not None:
            _f32(g, f"norm_rope_store {name}", (dim,))
    rot = 0
    if table is not None:
        _f32(table, "norm_rope_store table")
        if table.dim() != 3 or table.shape[0] != n or table.shape[2] != 2 or 2 * table.shape[1] > dim or not table.is_contiguous():
            raise ValueError("norm_rope_store: the table must be contiguous [n, R/2, 2] with R within the head")
        rot = 2 * int(table.shape[1])
    if vtable is not None:
        _f32(vtable, "norm_rope_store vtable", (n, vdim // 2, 2))
        if vdim % 2:
            raise ValueError("norm_rope_store: values of an odd size cannot be turned")
    ldq, wq = _rows(q_out, "norm_rope_store q_out")
    if tuple(q_out.shape) != (n, nh * dim):
        raise ValueError(f"norm_rope_store: q_out must be [n, {nh * dim}]")
    rows = 0
    if kcache is not None:
        if slots is None or vcache is None or kcache.dtype != q_out.dtype:
            raise ValueError("norm_rope_store: a cache needs the tokens' slots, and the queries' type")
        pages, ps = _token_cache(kcache, vcache, nkv, dim, vdim, "norm_rope_store")
        rows = pages * ps
        _i32(slots, "norm_rope_store slots", n)
    _lib.call("zi_norm_rope_store", _p(q_out), _code(q_out, "norm_rope_store q_out"), ldq, _p(kcache),
              _p(vcache if kcache is not None else None), _p(proj), ld, splits, split_stride, _p(q_gain), _p(k_gain),
              float(eps), _p(table), rot, _p(vtable), _p(slots if kcache is not None else None), rows, n, nh, nkv, dim,
              vdim, _stream())
    return q_out


def pool_blocks(kcache: torch.Tensor, vcache: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor,
                pool_slots: torch.Tensor, tok_seq: torch.Tensor, positions: torch.Tensor, block_tables: torch.Tensor,
                nkv: int, dim: int, vdim: int, pool: int) -> None:
    """For every token whose ``pool_slots`` entry is not negative (its position ends a block of ``pool`` positions):
    the means of the block's cached keys and values go to that row of ``kpool`` / ``vpool`` (float32
    [pages, page_size, kv_heads, dim / vdim])."""
    _gpu("pool_blocks", kcache, vcache, kpool, vpool, pool_slots, tok_seq, positions, block_tables)
    n = positions.numel()
    pages, ps = _token_cache(kcache, vcache, nkv, dim, vdim, "pool_blocks")
    if kpool.dtype != torch.float32 or vpool.dtype != torch.float32:
        raise ValueError("pool_blocks: the means are float32")
    ppages, pps = _token_cache(kpool, vpool, nkv, dim, vdim, "pool_blocks means")
    for name, t in (("pool_slots", pool_slots), ("tok_seq", tok_seq), ("positions", positions)):
        _i32(t, f"pool_blocks {name}", n)
    _i32(block_tables, "pool_blocks block_tables")
    if block_tables.dim() != 2 or pool <= 0:
        raise ValueError("pool_blocks: block tables are [entries, pages]; blocks hold at least one position")
    _lib.call("zi_pool_blocks", _p(kpool), _p(vpool), ppages * pps, _p(kcache), _p(vcache), _code(kcache, "pool_blocks cache"),
              _p(pool_slots), _p(tok_seq), _p(positions), _p(block_tables), int(block_tables.shape[1]), pages, ps, n, nkv,
              dim, vdim, int(pool), _stream())


def pooled_attention(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, kpool: Optional[torch.Tensor],
                     vpool: Optional[torch.Tensor], tok_seq: torch.Tensor, positions: torch.Tensor,
                     block_tables: torch.Tensor, pool_tables: Optional[torch.Tensor], nh: int, nkv: int, dim: int,
                     vdim: int, window: int, pool: int, scale: float, out: torch.Tensor,
                     vtable: Optional[torch.Tensor] = None, entry_len: Optional[torch.Tensor] = None,
                     long_len: int = 0) -> torch.Tensor:
    """out [n, nh*vdim]: softmax attention of q [n, nh*dim] over the positions j with 0 <= i - j < window and over the
    means of the blocks of ``pool`` positions that lie wholly before the window (window 0: all positions; pool 0 or no
    ``pool_tables``: no blocks).  ``vtable`` [n, vdim/2, 2]: the (cos, sin) by which every head's result is turned
    back (values were stored turned by their own positions).  With ``entry_len`` and ``long_len`` the tokens of entries
    that bring ``long_len`` tokens or more are left out (``pooled_attention_cores`` takes those)."""
    _gpu("pooled_attention", q, kcache, vcache, kpool, vpool, tok_seq, positions, block_tables, pool_tables, out, vtable)
    n = q.shape[0]
    ldq, wq = _rows(q, "pooled_attention q")
    ldo, wo = _rows(out, "pooled_attention out")
    if wq != nh * dim or wo != nh * vdim or out.shape[0] != n or q.dtype != kcache.dtype or out.dtype != q.dtype:
        raise ValueError("pooled_attention: q [n, nh*dim] and out [n, nh*vdim] in the cache's type")
    if nh % nkv or max(dim, vdim) > POOLED_MAX_HEAD:
        raise ValueError("pooled_attention: heads a multiple of the key/value heads, of at most 512 values")
    pages, ps = _token_cache(kcache, vcache, nkv, dim, vdim, "pooled_attention")
    _i32(tok_seq, "pooled_attention tok_seq", n)
    _i32(positions, "pooled_attention positions", n)
    _i32(block_tables, "pooled_attention block_tables")
    ppages = pps = pw = 0
    if pool_tables is not None and pool > 0:
        if kpool is None or vpool is None or kpool.dtype != torch.float32 or vpool.dtype != torch.float32:
            raise ValueError("pooled_attention: blocks need their float32 means")
        ppages, pps = _token_cache(kpool, vpool, nkv, dim, vdim, "pooled_attention means")
        _i32(pool_tables, "pooled_attention pool_tables")
        if pool_tables.shape[0] != block_tables.shape[0]:
            raise ValueError("pooled_attention: one row of either table an entry")
        pw = int(pool_tables.shape[1])
    else:
        pool_tables = None
    if vtable is not None:
        _f32(vtable, "pooled_attention vtable", (n, vdim // 2, 2))
    _lib.call("zi_pooled_attention", _p(out), ldo, _p(q), ldq, _code(q, "pooled_attention q"), _p(kcache), _p(vcache),
              _p(kpool), _p(vpool), _p(tok_seq), _p(positions), _p(block_tables), int(block_tables.shape[1]), pages, ps,
              _p(pool_tables), pw, ppages, pps, n, nh, nkv, dim, vdim, int(window), int(pool if pool_tables is not None else 0),
              float(scale), _p(vtable), _p(entry_len), int(long_len), _stream())
    return out


def pooled_attention_cores_supported(dtype: torch.dtype, nh: int, nkv: int, dim: int, vdim: int) -> bool:
    """Whether the matrix-core kernel takes these sizes (bfloat16; keys of 32, 64, 96 or 128 values, values of a
    multiple of 16 up to 128; at most 64 query heads a key/value head)."""
    if dtype != torch.bfloat16 or nkv <= 0:
        return False
    return bool(_lib.load().zi_pooled_attention_cores_supported(1, int(nh), int(nkv), int(dim), int(vdim)))


def pooled_attention_cores(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, kpool: Optional[torch.Tensor],
                           vpool: Optional[torch.Tensor], entry_start: torch.Tensor, entry_len: torch.Tensor,
                           entry_past: torch.Tensor, max_len: int, block_tables: torch.Tensor,
                           pool_tables: Optional[torch.Tensor], nh: int, nkv: int, dim: int, vdim: int, window: int,
                           pool: int, scale: float, out: torch.Tensor, vtable: Optional[torch.Tensor] = None,
                           long_len: int = 1, chunks: int = 0, chunk_blocks: int = 0,
                           workspace: Optional[torch.Tensor] = None, tok_seq: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``pooled_attention`` on the matrix cores for the tokens of the entries that bring at least ``long_len`` tokens
    (``max_len``: the most any entry brings); the rows of other tokens are not written.  With ``chunks`` > 0 instead
    for the entries that bring FEWER than ``long_len`` tokens (decoded tokens): the items every such entry sees (the
    blocks, then the window's positions) are cut into ``chunks`` chunks of ``chunk_blocks`` blocks of 32 items over
    workgroups and merged by a second kernel through ``workspace`` (``pooled_attention_cores_workspace`` floats);
    the caller chooses the cut so that it covers every entry's items (``pooled_attention_cores_cut``)."""
    _gpu("pooled_attention_cores", q, kcache, vcache, kpool, vpool, entry_start, entry_len, entry_past, block_tables,
         pool_tables, out, vtable)
    n = q.shape[0]
    ldq, wq = _rows(q, "pooled_attention_cores q")
    ldo, wo = _rows(out, "pooled_attention_cores out")
    if not pooled_attention_cores_supported(q.dtype, nh, nkv, dim, vdim):
        raise ValueError("pooled_attention_cores: sizes or a type the kernel does not take")
    if wq != nh * dim or wo != nh * vdim or out.shape[0] != n or kcache.dtype != q.dtype or out.dtype != q.dtype:
        raise ValueError("pooled_attention_cores: q [n, nh*dim] and out [n, nh*vdim] in the cache's type")
    pages, ps = _token_cache(kcache, vcache, nkv, dim, vdim, "pooled_attention_cores")
    E = entry_start.numel()
    for t in (entry_start, entry_len, entry_past):
        _i32(t, "pooled_attention_cores entries", E)
    _i32(block_tables, "pooled_attention_cores block_tables")
    if block_tables.dim() != 2 or block_tables.shape[0] < E:
        raise ValueError("pooled_attention_cores: one row of the block table an entry")
    ppages = pps = pw = 0
    if pool_tables is not None and pool > 0:
        if kpool is None or vpool is None or kpool.dtype != torch.float32 or vpool.dtype != torch.float32:
            raise ValueError("pooled_attention_cores: blocks need their float32 means")
        ppages, pps = _token_cache(kpool, vpool, nkv, dim, vdim, "pooled_attention_cores means")
        _i32(pool_tables, "pooled_attention_cores pool_tables")
        if pool_tables.shape[0] != block_tables.shape[0]:
            raise ValueError("pooled_attention_cores: one row of either table an entry")
        pw = int(pool_tables.shape[1])
    else:
        pool_tables = None
    if vtable is not None:
        _f32(vtable, "pooled_attention_cores vtable", (n, vdim // 2, 2))
    if chunks > 0:
        need = pooled_attention_cores_workspace(n, nh, vdim, chunks)
        if workspace is None or workspace.dtype != torch.float32 or workspace.numel() < need or not workspace.is_contiguous():
            raise ValueError(f"pooled_attention_cores: {need} floats of workspace are needed")
        if tok_seq is None or chunk_blocks <= 0 or (long_len - 1) * (nh // nkv) > POOLED_ROWS:
            raise ValueError("pooled_attention_cores: a cut needs every token's entry, blocks a chunk, and short entries that fit a tile")
        _i32(tok_seq, "pooled_attention_cores tok_seq", n)
    _lib.call("zi_pooled_attention_cores", _p(out), ldo, _p(q), ldq, _p(kcache), _p(vcache), _p(kpool), _p(vpool),
              _p(entry_start), _p(entry_len), _p(entry_past), E, int(max_len), _p(block_tables), int(block_tables.shape[1]),
              pages, ps, _p(pool_tables), pw, ppages, pps, nh, nkv, dim, vdim, int(window),
              int(pool if pool_tables is not None else 0), float(scale), _p(vtable), int(long_len), int(chunks),
              int(chunk_blocks), _p(workspace), int(workspace.numel()) if workspace is not None else 0, _p(tok_seq), n, _stream())
    return out


POOLED_ITEMS = 32          # items (blocks' means or positions) a block of the matrix-core kernel holds
POOLED_ROWS = 64           # rows (token, head of a group) a workgroup of it holds


def pooled_attention_cores_cut(max_keys: int, window: int, pool: int, most_tokens: int, units: int, tiles: int):
    """(chunks, blocks a chunk) for the short entries of a step none of which holds more than ``max_keys`` tokens
    once it has run and brings more than ``most_tokens``: chunks of four blocks of 32 items, of more when ``tiles``
    (entries x key/value heads) workgroups a chunk would be many more than the chip holds at a time."""
    if window > 0:
        span = min(window + most_tokens, max_keys)
        means = -(-(max_keys // pool) // POOLED_ITEMS) if pool > 0 else 0
        blocks = means + -(-span // POOLED_ITEMS) + 1     # the positions' first block starts anywhere
    else:
        blocks = -(-max_keys // POOLED_ITEMS)
    per = 4
    while per < blocks and -(-blocks // per) * max(tiles, 1) > 4 * max(units, 1):
        per *= 2
    return max(1, -(-blocks // per)), per


def pooled_attention_cores_workspace(n: int, nh: int, vdim: int, chunks: int) -> int:
    return int(chunks) * int(n) * int(nh) * (int(vdim) + 2)


# ---- a norm on a sublayer's output -----------------------------------------------------------------------------
def normed_add_norm(resid: torch.Tensor, y: torch.Tensor, w1: torch.Tensor, eps: float, add_one: bool,
                    w2: Optional[torch.Tensor] = None, eps2: float = 0.0, out: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """resid (float32, in place) += rms_norm(y) * w1 (1 + w1 with ``add_one``), y [n, H] or a stack [S, n, H] of
    float32 terms added first; with ``out``: out = rms_norm(resid) * w2 (likewise), the norm the next sublayer
    reads, in the same launch."""
    _gpu("normed_add_norm", resid, y, w1, w2, out)
    splits, split_stride, ldy, n, H = _terms(y, "normed_add_norm y")
    if resid.dtype != torch.float32 or tuple(resid.shape) != (n, H) or not resid.is_contiguous():
        raise ValueError(f"normed_add_norm: the residual stream must be a contiguous float32 [{n}, {H}] tensor")
    if H > NORMED_ADD_MAX_HIDDEN:
        raise ValueError(f"normed_add_norm: rows of at most {NORMED_ADD_MAX_HIDDEN} values")
    if w1.numel() != H or not w1.is_contiguous():
        raise ValueError(f"normed_add_norm: the gain must be a contiguous [{H}] tensor")
    if out is not None:
        if w2 is None or w2.numel() != H or not w2.is_contiguous() or w2.dtype != w1.dtype:
            raise ValueError("normed_add_norm: the second norm needs a gain of the first one's type")
        if tuple(out.shape) != (n, H) or not out.is_contiguous():
            raise ValueError("normed_add_norm: out must be contiguous [n, H]")
    _lib.call("zi_normed_add_norm", _p(out), _code(out, "normed_add_norm out") if out is not None else 0, _p(resid), _p(y),
              _code(y, "normed_add_norm y"), ldy, splits, split_stride, _p(w1), _p(w2 if out is not None else None),
              _code(w1, "normed_add_norm gain"), n, H, float(eps), float(eps2 or eps), int(bool(add_one)), _stream())
    return out


# ---- experts chosen by independent scores ----------------------------------------------------------------------
def moe_route_sigmoid(z: torch.Tensor, experts: int, top: int, idx: torch.Tensor, wt: torch.Tensor) -> None:
    """z float32 [n, >= experts] (the first ``experts`` columns count): s = sigmoid(z), the ``top`` largest (lowest
    index among equals) into idx [n, top] int32, their scores into wt [n, top] float32."""
    _gpu("moe_route_sigmoid", z, idx, wt)
    ld, w = _rows(z, "moe_route_sigmoid z")
    n = z.shape[0]
    if z.dtype != torch.float32 or w < experts or not (0 < top <= experts <= MOE_MAX_EXPERTS):
        raise ValueError("moe_route_sigmoid: z float32 [n, >= experts], 0 < top <= experts")
    _i32(idx, "moe_route_sigmoid idx", n * top)
    _f32(wt, "moe_route_sigmoid wt", (n, top))
    _lib.call("zi_moe_route_sigmoid", _p(idx), _p(wt), _p(z), ld, n, int(experts), int(top), _stream())


def moe_weighted_glu(gu: torch.Tensor, wt: torch.Tensor, order: torch.Tensor, ff: int, out: torch.Tensor) -> torch.Tensor:
    """out [pairs, ff] = silu(w g) * (w u) for the rows gu [pairs, g | u] float32 of the grouped pairs, w the weight of
    the pair at that place (wt.flatten()[order[row]])."""
    _gpu("moe_weighted_glu", gu, wt, order, out)
    ld, w = _rows(gu, "moe_weighted_glu gu")
    pairs = gu.shape[0]
    ldo, wo = _rows(out, "moe_weighted_glu out")
    if gu.dtype != torch.float32 or w != 2 * ff or wo != ff or out.shape[0] != pairs or wt.numel() != pairs:
        raise ValueError("moe_weighted_glu: gu float32 [pairs, 2 ff], out [pairs, ff], a weight a pair")
    _f32(wt, "moe_weighted_glu wt")
    _i32(order, "moe_weighted_glu order", pairs)
    _lib.call("zi_moe_weighted_glu", _p(out), _code(out, "moe_weighted_glu out"), ldo, _p(gu), ld, _p(wt), _p(order), pairs,
              int(ff), _stream())
    return out


def moe_sum_shared(y: torch.Tensor, place_of: torch.Tensor, top: int, out: torch.Tensor,
                   shared: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out [n, H] float32 = the sum of every token's ``top`` rows of y [pairs, H] (found through place_of) +
    sigmoid(gate[t]) * shared[t]; ``shared`` [n, H] or a stack [S, n, H] of float32 terms, ``gate`` float32 [n]
    (any stride) or None (the shared rows count whole)."""
    _gpu("moe_sum_shared", y, place_of, out, shared, gate)
    n, H = out.shape
    _f32(out, "moe_sum_shared out", (n, H))
    _f32(y, "moe_sum_shared y", (n * top, H))
    _i32(place_of, "moe_sum_shared place_of", n * top)
    splits, split_stride = 1, 0
    if shared is not None:
        splits, split_stride, ld, ns, Hs = _terms(shared, "moe_sum_shared shared")
        if shared.dtype != torch.float32 or ns != n or Hs != H or ld != H:
            raise ValueError("moe_sum_shared: the shared rows must be float32 [n, H] with dense rows")
    ldg = 0
    if gate is not None:
        if gate.dtype != torch.float32 or gate.dim() != 1 or gate.numel() != n:
            raise ValueError("moe_sum_shared: the gate is one float32 a token")
        ldg = int(gate.stride(0)) if n > 1 else 1
    _lib.call("zi_moe_sum_shared", _p(out), _p(y), _p(place_of), _p(shared), splits, split_stride, _p(gate), ldg, n, int(top),
              H, _stream())
    return out
