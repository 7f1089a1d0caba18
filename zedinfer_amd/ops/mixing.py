"""Checked launches of the kernels behind the mixers and feed-forwards that are not plain attention and SwiGLU:
latent attention (a short latent and one shared rotated key part per token), the gated delta rule (a recurrent
matrix state per head), routed experts, and the gated activation in its other forms."""
from __future__ import annotations

import os
from typing import Optional

import torch

from . import _lib
from .functional import _code, _gpu, _i32, _p, _rows, _stream

ACTIVATIONS = {"silu": 0, "gelu_tanh": 1, "gelu_erf": 2}
MOE_TILE_ROWS = (16, 32, 64)
MOE_MAX_EXPERTS = 1024
DELTA_MAX_TAPS = 17


def _f32(t: torch.Tensor, what: str, shape=None) -> None:
    if t.dtype != torch.float32 or not t.is_contiguous():
        raise TypeError(f"{what}: expected a contiguous float32 tensor, got {t.dtype} with strides {t.stride()}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"{what}: expected shape {tuple(shape)}, got {tuple(t.shape)}")


def gated_act(gate: torch.Tensor, up: torch.Tensor, activation: str, out: torch.Tensor) -> torch.Tensor:
    """out = act(gate) * up for [n, I] operands with dense rows (column slices of one product are fine)."""
    _gpu("gated_act", gate, up, out)
    if activation not in ACTIVATIONS:
        raise ValueError(f"gated_act: unknown activation {activation!r}; known: {sorted(ACTIVATIONS)}")
    ldg, I = _rows(gate, "gated_act gate")
    ldu, Iu = _rows(up, "gated_act up")
    ldo, Io = _rows(out, "gated_act out")
    n = gate.shape[0]
    if gate.dtype != up.dtype or I != Iu or I != Io or up.shape[0] != n or out.shape[0] != n:
        raise ValueError("gated_act: gate, up and out must agree in shape, gate and up in type")
    _lib.call("zi_gated_act", _p(out), _code(out, "gated_act out"), ldo, _p(gate), _p(up), _code(gate, "gated_act"),
              ldg, ldu, n, I, ACTIVATIONS[activation], _stream())
    return out


def rope_pairs(x: torch.Tensor, table: torch.Tensor, heads: int, d: int) -> torch.Tensor:
    """In place: the first R dims of every head of x [n, heads * d] turn in neighbouring pairs (2i, 2i + 1) by the
    step's ``table`` of (cos, sin) [n, R/2, 2]."""
    _gpu("rope_pairs", x, table)
    ld, width = _rows(x, "rope_pairs x")
    n = x.shape[0]
    if width != heads * d:
        raise ValueError(f"rope_pairs: x must be [n, {heads * d}]")
    if table.dim() != 3 or table.shape[0] != n or table.shape[2] != 2 or 2 * table.shape[1] > d:
        raise ValueError("rope_pairs: the table must be [n, R/2, 2] with R within the head")
    _f32(table, "rope_pairs table")
    _lib.call("zi_rope_pairs", _p(x), _code(x, "rope_pairs x"), ld, _p(table), n, heads, d, 2 * int(table.shape[1]), _stream())
    return x


# ---- latent attention ----------------------------------------------------------------------------------------
def _latent_caches(c_cache: torch.Tensor, kr_cache: torch.Tensor, rank: int, rot: int, what: str):
    if c_cache.dim() != 3 or kr_cache.dim() != 3 or c_cache.shape[2] != rank or kr_cache.shape[2] != rot \
            or c_cache.shape[:2] != kr_cache.shape[:2] or c_cache.dtype != kr_cache.dtype \
            or not c_cache.is_contiguous() or not kr_cache.is_contiguous():
        raise ValueError(f"{what}: the caches must be contiguous [pages, page, {rank}] and [pages, page, {rot}] of one type")
    return int(c_cache.shape[0]), int(c_cache.shape[1])


def latent_store(dkv: torch.Tensor, norm_w: torch.Tensor, eps: float, table: Optional[torch.Tensor],
                 slots: torch.Tensor, c_cache: torch.Tensor, kr_cache: torch.Tensor, rank: int, rot: int) -> None:
    """Rows of dkv [n, rank + rot]: the first ``rank`` values RMS-normed with ``norm_w`` go to the latent cache
    at ``slots``, the last ``rot`` turned in neighbouring pairs by ``table`` [n, rot/2, 2] to the key-part cache;
    tokens whose slot is negative are skipped."""
    _gpu("latent_store", dkv, norm_w, table, slots, c_cache, kr_cache)
    ld, width = _rows(dkv, "latent_store dkv")
    n = dkv.shape[0]
    pages, ps = _latent_caches(c_cache, kr_cache, rank, rot, "latent_store")
    if width != rank + rot or dkv.dtype != torch.float32:
        raise ValueError(f"latent_store: dkv must be float32 [n, {rank + rot}]")
    if norm_w.numel() != rank or not norm_w.is_contiguous():
        raise ValueError(f"latent_store: the norm's weight must be [{rank}]")
    _i32(slots, "latent_store slots", n)
    if rot:
        _f32(table, "latent_store table", (n, rot // 2, 2))
    _lib.call("zi_latent_store", _p(dkv), _code(c_cache, "latent_store cache"), ld, n, _p(norm_w), _code(norm_w, "latent_store norm"),
              float(eps), _p(table), _p(slots), _p(c_cache), _p(kr_cache), pages * ps, rank, rot, _stream())


def latent_query(q: torch.Tensor, w_uk: torch.Tensor, table: Optional[torch.Tensor], heads: int, dim: int, rank: int,
                 rot: int, out: torch.Tensor, w_uk_t: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out [n, heads, rank + rot] float32: every head's unrotated query part carried through its block of
    ``w_uk`` [heads * dim, rank] (so that it meets latents instead of keys), then its rotated part, turned."""
    _gpu("latent_query", q, w_uk, table, out)
    ldq, width = _rows(q, "latent_query q")
    n = q.shape[0]
    if width != heads * (dim + rot):
        raise ValueError(f"latent_query: q must be [n, {heads * (dim + rot)}]")
    if tuple(w_uk.shape) != (heads * dim, rank) or not w_uk.is_contiguous():
        raise ValueError(f"latent_query: w_uk must be a contiguous [{heads * dim}, {rank}] tensor")
    _f32(out, "latent_query out", (n, heads, rank + rot))
    if rot:
        _f32(table, "latent_query table", (n, rot // 2, 2))
    if w_uk_t is not None and q.dtype == torch.float32 and q.data_ptr() % 16 == 0 \
            and _lib.load().zi_headwise_linear_supported(_code(w_uk_t, "latent_query w_uk_t"), dim, ldq, dim + rot):
        # on the matrix cores: the head's block of W_uk, transposed at load, times the unrotated query parts
        if tuple(w_uk_t.shape) != (heads, rank, dim) or not w_uk_t.is_contiguous():
            raise ValueError(f"latent_query: w_uk_t must be a contiguous [{heads}, {rank}, {dim}] tensor")
        _lib.call("zi_headwise_linear", _p(out), 0, heads * (rank + rot), rank + rot, _p(q), ldq, dim + rot, _p(w_uk_t), n,
                  heads, rank, dim, _stream())
        if rot:
            _lib.call("zi_latent_query_rot", _p(out), _p(q), _code(q, "latent_query q"), ldq, _p(table), n, heads, dim, rank,
                      rot, _stream())
        return out
    _lib.call("zi_latent_query", _p(out), _p(q), _code(q, "latent_query q"), ldq, _p(w_uk), _code(w_uk, "latent_query w_uk"),
              _p(table), n, heads, dim, rank, rot, _stream())
    return out


def latent_attention(qa: torch.Tensor, c_cache: torch.Tensor, kr_cache: torch.Tensor, tok_seq: torch.Tensor,
                     tok_pos: torch.Tensor, block_tables: torch.Tensor, scale: float, window: int, out: torch.Tensor,
                     tok_index: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out [n, heads, rank] float32 = sum_j softmax_j((qa . (c_j, kr_j)) * scale) c_j over the positions j a token
    sees: all up to its own, or the last ``window`` of them."""
    _gpu("latent_attention", qa, c_cache, kr_cache, tok_seq, tok_pos, block_tables, out, tok_index)
    if qa.dim() != 3:
        raise ValueError("latent_attention: qa must be [n, heads, rank + rot]")
    n, heads, qw = qa.shape
    rank = int(c_cache.shape[2]) if c_cache.dim() == 3 else -1
    rot = qw - rank
    pages, ps = _latent_caches(c_cache, kr_cache, rank, rot, "latent_attention")
    _f32(qa, "latent_attention qa")
    _f32(out, "latent_attention out", (n, heads, rank))
    _i32(tok_seq, "latent_attention tok_seq", n)
    _i32(tok_pos, "latent_attention tok_pos", n)
    if block_tables.dim() != 2:
        raise ValueError("latent_attention: block tables must be [entries, pages]")
    _i32(block_tables, "latent_attention block_tables")
    count = n
    if tok_index is not None:
        _i32(tok_index, "latent_attention tok_index")
        count = tok_index.numel()
    _lib.call("zi_latent_attention", _p(out), _p(qa), _p(c_cache), _p(kr_cache), _code(c_cache, "latent_attention cache"),
              count, _p(tok_index), _p(tok_seq), _p(tok_pos), _p(block_tables), int(block_tables.shape[1]), pages, heads,
              rank, rot, ps, int(window), float(scale), _stream())
    return out


# keys of a chunk when a tile's keys are cut over workgroups (a multiple of the kernel's block of 32)
LATENT_CHUNK_KEYS = max(32, int(os.environ.get("ZEDINFER_LATENT_CHUNK_KEYS", "128") or 128) // 32 * 32)


def latent_attention_cores_supported(cache_dtype: torch.dtype, rank: int, rot: int) -> bool:
    """Whether the matrix-core kernel takes caches of this type and these sizes."""
    if cache_dtype != torch.bfloat16:
        return False
    return bool(_lib.load().zi_latent_attention_cores_supported(1, int(rank), int(rot)))


def latent_attention_cores_plan(n: int, entries: int, heads: int, window: int, units: int, max_keys: int = 0):
    """(wavefronts a workgroup, keys a chunk, chunks) for a step of n tokens in ``entries`` entries: 64 rows a
    workgroup when that many tiles fill the chip, else 16; a tile's keys are cut into chunks when the tiles alone
    are fewer than the chip's compute units (decoded tokens, short portions) and a window bounds them, or, without
    a window, ``max_keys`` does (no entry holds more tokens once the step has run).  A function of the step's shape."""
    lib = _lib.load()
    waves = 4 if lib.zi_latent_attention_cores_tiles(int(n), int(entries), int(heads), 4) >= units else 1
    tiles = lib.zi_latent_attention_cores_tiles(int(n), int(entries), int(heads), waves)
    if window > 0 and tiles < units:
        span = int(window) + -(-16 * waves // int(heads)) + 1
        chunks = -(-span // LATENT_CHUNK_KEYS)
        if chunks > 1:
            return waves, LATENT_CHUNK_KEYS, chunks
    if window <= 0 and max_keys > 0 and tiles < units:
        keys = LATENT_CHUNK_KEYS
        while -(-int(max_keys) // keys) * tiles > 4 * units:      # no more workgroups than four rounds of the chip
            keys *= 2
        chunks = -(-int(max_keys) // keys)
        if chunks > 1:
            return waves, keys, chunks
    return waves, 0, 1


def latent_attention_cores_workspace(n: int, heads: int, rank: int, chunks: int) -> int:
    """Floats of workspace for the chunks' partial results (0 without a cut)."""
    return int(chunks) * int(n) * int(heads) * (int(rank) + 2) if chunks > 1 else 0


def latent_attention_cores(qa: torch.Tensor, c_cache: torch.Tensor, kr_cache: torch.Tensor, entry_start: torch.Tensor,
                           entry_len: torch.Tensor, entry_past: torch.Tensor, block_tables: torch.Tensor, scale: float,
                           window: int, out: torch.Tensor, waves: int = 1, chunk_keys: int = 0, chunks: int = 1,
                           workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``latent_attention`` on the matrix cores, for all tokens of a step (bfloat16 caches): entry e brings the
    tokens entry_start[e] ... of positions entry_past[e] ...; queries are rounded to bfloat16 for the products,
    scores, softmax and sums are float32."""
    _gpu("latent_attention_cores", qa, c_cache, kr_cache, entry_start, entry_len, entry_past, block_tables, out, workspace)
    if qa.dim() != 3:
        raise ValueError("latent_attention_cores: qa must be [n, heads, rank + rot]")
    n, heads, qw = qa.shape
    rank = int(c_cache.shape[2]) if c_cache.dim() == 3 else -1
    rot = qw - rank
    pages, ps = _latent_caches(c_cache, kr_cache, rank, rot, "latent_attention_cores")
    if not latent_attention_cores_supported(c_cache.dtype, rank, rot):
        raise ValueError(f"latent_attention_cores: a {c_cache.dtype} cache with rank {rank} and rot {rot} is not taken")
    _f32(qa, "latent_attention_cores qa")
    _f32(out, "latent_attention_cores out", (n, heads, rank))
    E = entry_start.numel()
    for t in (entry_start, entry_len, entry_past):
        _i32(t, "latent_attention_cores entries", E)
    if block_tables.dim() != 2 or block_tables.shape[0] < E:
        raise ValueError("latent_attention_cores: block tables must be [entries, pages]")
    _i32(block_tables, "latent_attention_cores block_tables")
    need = latent_attention_cores_workspace(n, heads, rank, chunks)
    if need and (workspace is None or workspace.dtype != torch.float32 or workspace.numel() < need):
        raise ValueError(f"latent_attention_cores: {need} floats of workspace are needed")
    _lib.call("zi_latent_attention_cores", _p(out), _p(workspace), int(workspace.numel()) if workspace is not None else 0,
              _p(qa), _p(c_cache), _p(kr_cache), _p(entry_start), _p(entry_len), _p(entry_past), _p(block_tables), E, n,
              int(block_tables.shape[1]), pages, heads, rank, rot, ps, int(window), float(scale), int(waves),
              int(chunk_keys), int(chunks), _stream())
    return out


def latent_value(o: torch.Tensor, w_uv: torch.Tensor, vdim: int, out: torch.Tensor) -> torch.Tensor:
    """out [n, heads * vdim] = every head's attended latent o [n, heads, rank] through its block of ``w_uv``
    [heads * vdim, rank]."""
    _gpu("latent_value", o, w_uv, out)
    _f32(o, "latent_value o")
    n, heads, rank = o.shape
    if tuple(w_uv.shape) != (heads * vdim, rank) or not w_uv.is_contiguous():
        raise ValueError(f"latent_value: w_uv must be a contiguous [{heads * vdim}, {rank}] tensor")
    ldo, width = _rows(out, "latent_value out")
    if tuple(out.shape) != (n, heads * vdim):
        raise ValueError(f"latent_value: out must be [{n}, {heads * vdim}]")
    if w_uv.dtype == torch.bfloat16 and _lib.load().zi_headwise_linear_supported(1, rank, heads * rank, rank) \
            and w_uv.data_ptr() % 16 == 0:
        _lib.call("zi_headwise_linear", _p(out), _code(out, "latent_value out"), ldo, vdim, _p(o), heads * rank, rank,
                  _p(w_uv), n, heads, vdim, rank, _stream())
        return out
    _lib.call("zi_latent_value", _p(out), _code(out, "latent_value out"), ldo, _p(o), _p(w_uv), _code(w_uv, "latent_value w_uv"),
              n, heads, vdim, rank, _stream())
    return out


# ---- the gated delta rule -------------------------------------------------------------------------------------
def delta_state_floats(heads: int, dim: int, vdim: int, kv_heads: int, taps: int) -> int:
    """Floats of one request's state: the matrices [heads, dim, vdim], then the convolution's tail
    [taps - 1, channels]."""
    return heads * dim * vdim + (taps - 1) * (2 * kv_heads * dim + heads * vdim)


def delta_prepare(proj: torch.Tensor, conv_w: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor,
                  state: torch.Tensor, tok_seq: torch.Tensor, entry_start: torch.Tensor, entry_slot: torch.Tensor,
                  heads: int, kv_heads: int, dim: int, vdim: int, taps: int, qk: torch.Tensor, v: torch.Tensor,
                  beta_g: torch.Tensor) -> None:
    """From the stacked projection proj [n, q | k | v | gate | b | a] (float32): the short convolution and SiLU of
    q, k, v (rows before an entry's first come from the tail kept in ``state``), q and k made unit vectors per
    head (q also times dim^-1/2) into ``qk`` [n, 2 kv_heads dim], v into ``v`` [n, heads vdim], and into
    ``beta_g`` [n, 2, heads] beta = sigmoid(b) and the decay g = exp(-exp(a_log) softplus(a + dt_bias))."""
    _gpu("delta_prepare", proj, conv_w, a_log, dt_bias, state, tok_seq, entry_start, entry_slot, qk, v, beta_g)
    n = proj.shape[0]
    C = 2 * kv_heads * dim + heads * vdim
    ld, width = _rows(proj, "delta_prepare proj")
    if proj.dtype != torch.float32 or width != C + heads * vdim + 2 * heads:
        raise ValueError(f"delta_prepare: proj must be float32 [n, {C + heads * vdim + 2 * heads}]")
    for t, shape, what in ((conv_w, (C, taps), "conv_w"), (a_log, (heads,), "a_log"), (dt_bias, (heads,), "dt_bias")):
        _f32(t, f"delta_prepare {what}", shape)
    _f32(qk, "delta_prepare qk", (n, 2 * kv_heads * dim))
    _f32(v, "delta_prepare v", (n, heads * vdim))
    _f32(beta_g, "delta_prepare beta_g", (n, 2, heads))
    _f32(state, "delta_prepare state")
    if state.dim() != 2 or state.shape[1] < delta_state_floats(heads, dim, vdim, kv_heads, taps):
        raise ValueError("delta_prepare: the state must be [slots, floats of one request's state]")
    _i32(tok_seq, "delta_prepare tok_seq", n)
    _i32(entry_start, "delta_prepare entry_start")
    _i32(entry_slot, "delta_prepare entry_slot", entry_start.numel())
    _lib.call("zi_delta_prepare", _p(qk), _p(v), _p(beta_g), _p(proj), ld, n, _p(conv_w), _p(a_log), _p(dt_bias), 0,
              _p(state), int(state.shape[1]), heads * dim * vdim, _p(tok_seq), _p(entry_start), _p(entry_slot), heads,
              kv_heads, dim, vdim, taps, _stream())


def delta_conv_state(state: torch.Tensor, proj: torch.Tensor, entry_start: torch.Tensor, entry_len: torch.Tensor,
                     entry_slot: torch.Tensor, heads: int, kv_heads: int, dim: int, vdim: int, taps: int) -> None:
    """The convolution's tail in ``state`` becomes the last taps - 1 rows of every entry's sequence so far."""
    _gpu("delta_conv_state", state, proj, entry_start, entry_len, entry_slot)
    C = 2 * kv_heads * dim + heads * vdim
    ld, width = _rows(proj, "delta_conv_state proj")
    if proj.dtype != torch.float32 or width < C:
        raise ValueError("delta_conv_state: proj must be float32 and hold the convolution's channels first")
    _f32(state, "delta_conv_state state")
    if taps > DELTA_MAX_TAPS:
        raise ValueError(f"delta_conv_state: at most {DELTA_MAX_TAPS} taps")
    E = entry_start.numel()
    for t in (entry_start, entry_len, entry_slot):
        _i32(t, "delta_conv_state entries", E)
    _lib.call("zi_delta_conv_state", _p(state), int(state.shape[1]), heads * dim * vdim, _p(proj), ld, _p(entry_start),
              _p(entry_len), _p(entry_slot), E, C, taps, _stream())


def delta_rule(qk: torch.Tensor, v: torch.Tensor, beta_g: torch.Tensor, state: torch.Tensor, entry_start: torch.Tensor,
               entry_len: torch.Tensor, entry_slot: torch.Tensor, heads: int, kv_heads: int, dim: int, vdim: int,
               out: torch.Tensor) -> torch.Tensor:
    """Every entry's tokens in order, per head: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q, with S
    read from and left in ``state`` [slots, ...]; out [n, heads * vdim] float32."""
    _gpu("delta_rule", qk, v, beta_g, state, entry_start, entry_len, entry_slot, out)
    n = qk.shape[0]
    _f32(qk, "delta_rule qk", (n, 2 * kv_heads * dim))
    _f32(v, "delta_rule v", (n, heads * vdim))
    _f32(beta_g, "delta_rule beta_g", (n, 2, heads))
    _f32(out, "delta_rule out", (n, heads * vdim))
    _f32(state, "delta_rule state")
    if state.dim() != 2 or state.shape[1] < heads * dim * vdim:
        raise ValueError("delta_rule: the state row is too short")
    if dim > 256:
        raise ValueError(f"delta_rule: dim {dim} is more than the kernel's 256")
    E = entry_start.numel()
    for t in (entry_start, entry_len, entry_slot):
        _i32(t, "delta_rule entries", E)
    _lib.call("zi_delta_rule", _p(out), _p(qk), _p(v), _p(beta_g), _p(state), int(state.shape[1]), _p(entry_start),
              _p(entry_len), _p(entry_slot), E, heads, kv_heads, dim, vdim, _stream())
    return out


def gated_rms_norm(o: torch.Tensor, weight: torch.Tensor, gate: torch.Tensor, heads: int, vdim: int, eps: float,
                   out: torch.Tensor) -> torch.Tensor:
    """out [n, heads * vdim] = o / rms(o over each head's vdim values) * weight [vdim] * silu(gate), gate
    [n, heads * vdim] float32 with dense rows (a column slice is fine)."""
    _gpu("gated_rms_norm", o, weight, gate, out)
    n = o.shape[0]
    _f32(o, "gated_rms_norm o", (n, heads * vdim))
    _f32(weight, "gated_rms_norm weight", (vdim,))
    ldg, gw = _rows(gate, "gated_rms_norm gate")
    if gate.dtype != torch.float32 or gw != heads * vdim or gate.shape[0] != n:
        raise ValueError("gated_rms_norm: the gate must be float32 [n, heads * vdim]")
    if tuple(out.shape) != (n, heads * vdim) or not out.is_contiguous():
        raise ValueError("gated_rms_norm: out must be contiguous [n, heads * vdim]")
    _lib.call("zi_gated_rmsnorm", _p(out), _code(out, "gated_rms_norm out"), _p(o), _p(weight), 0, _p(gate), ldg, n, heads,
              vdim, float(eps), _stream())
    return out


# ---- routed experts -------------------------------------------------------------------------------------------
def moe_route(z: torch.Tensor, correction: torch.Tensor, top: int, scale: float, idx: torch.Tensor,
              wt: torch.Tensor) -> None:
    """z [n, E] float32 router logits: s = softmax(z); the ``top`` experts with the largest s + correction (the
    lowest index among equals) into ``idx`` [n, top], their s * scale into ``wt``."""
    _gpu("moe_route", z, correction, idx, wt)
    _f32(z, "moe_route z")
    n, E = z.shape
    _f32(correction, "moe_route correction", (E,))
    _f32(wt, "moe_route wt", (n, top))
    _i32(idx, "moe_route idx", n * top)
    if not (0 < top <= E <= MOE_MAX_EXPERTS):
        raise ValueError(f"moe_route: top {top} of {E} experts (at most {MOE_MAX_EXPERTS})")
    _lib.call("zi_moe_route", _p(idx), _p(wt), _p(z), _p(correction), n, E, top, float(scale), _stream())


def moe_max_tiles(pairs: int, experts: int, tile_rows: int) -> int:
    """Most row tiles ``moe_group`` can make of ``pairs`` (token, choice) pairs."""
    return -(-pairs // tile_rows) + min(experts, pairs)


def moe_group(idx: torch.Tensor, experts: int, tile_rows: int, plan: torch.Tensor, order: torch.Tensor,
              place_of: torch.Tensor) -> None:
    """Sort the pairs by expert on the device: ``order`` [pairs] lists them expert by expert, ``place_of`` is its
    inverse, ``plan`` = [tiles, then (expert, first row, rows) of every tile of at most ``tile_rows`` rows]."""
    _gpu("moe_group", idx, plan, order, place_of)
    pairs = idx.numel()
    _i32(idx, "moe_group idx")
    _i32(order, "moe_group order", pairs)
    _i32(place_of, "moe_group place_of", pairs)
    _i32(plan, "moe_group plan", 1 + 3 * moe_max_tiles(pairs, experts, tile_rows))
    _lib.call("zi_moe_group", _p(plan), _p(order), _p(place_of), _p(idx), pairs, experts, tile_rows, _stream())


def moe_tile_rows(x_dtype: torch.dtype, w_dtype: torch.dtype, widths, pairs: int, experts: int) -> int:
    """Rows of a tile of the experts' products: 16 for the plain kernel; on the matrix cores (bfloat16, every
    inner size a multiple of 8) 16, 32 or 64, the more rows an expert gets on average the larger."""
    cores = x_dtype == torch.bfloat16 and w_dtype == torch.bfloat16 and all(int(k) % 8 == 0 for k in widths)
    if not cores:
        return 16
    mean = pairs / max(experts, 1)
    return 64 if mean >= 96 else 32 if mean >= 24 else 16


def moe_linear(x: torch.Tensor, w: torch.Tensor, plan: torch.Tensor, tile_rows: int, max_tiles: int,
               out: torch.Tensor, source: Optional[torch.Tensor] = None, source_div: int = 1,
               activation: Optional[str] = None) -> torch.Tensor:
    """out[r] = act(w[expert of row r] . x[source row of r]) for the rows of the sorted order; w [E, N, K].
    ``source`` (the order of ``moe_group``) with ``source_div`` = top reads row r from token order[r] // top;
    without it row r reads x[r]."""
    _gpu("moe_linear", x, w, plan, out, source)
    ldx, K = _rows(x, "moe_linear x")
    ldo, N = _rows(out, "moe_linear out")
    if w.dim() != 3 or w.shape[1] != N or w.shape[2] != K or not w.is_contiguous():
        raise ValueError(f"moe_linear: w must be a contiguous [experts, {N}, {K}] tensor")
    if activation not in (None, "gelu_erf"):
        raise ValueError("moe_linear: the activation is None or 'gelu_erf'")
    if tile_rows not in MOE_TILE_ROWS:
        raise ValueError(f"moe_linear: tile_rows must be one of {MOE_TILE_ROWS}")
    _i32(plan, "moe_linear plan", 1 + 3 * max_tiles)
    if source is not None:
        _i32(source, "moe_linear source", out.shape[0])
    _lib.call("zi_moe_linear", _p(out), _code(out, "moe_linear out"), ldo, _p(x), _code(x, "moe_linear x"), ldx, _p(w),
              _code(w, "moe_linear w"), _p(plan), _p(source), int(source_div), int(max_tiles), int(tile_rows), N, K,
              1 if activation else 0, _stream())
    return out


def moe_combine(y: torch.Tensor, wt: torch.Tensor, place_of: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t] = sum_k wt[t, k] * y[place_of[t * top + k]], float32, k rising."""
    _gpu("moe_combine", y, wt, place_of, out)
    n, top = wt.shape
    _f32(wt, "moe_combine wt")
    _f32(y, "moe_combine y")
    H = y.shape[1]
    if y.shape[0] < n * top:
        raise ValueError("moe_combine: y has fewer rows than pairs")
    _f32(out, "moe_combine out", (n, H))
    _i32(place_of, "moe_combine place_of", n * top)
    _lib.call("zi_moe_combine", _p(out), _p(y), _p(wt), _p(place_of), n, top, H, _stream())
    return out
