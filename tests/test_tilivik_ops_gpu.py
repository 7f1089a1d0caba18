"""The kernels behind the Tilivik design, each alone against the plain implementation's function of the same
mechanism: the summed embedding and its carried token, the token shift and its carried row, the low-rank decay gate,
linear attention with fixed and gated decay (in portions, in slots that others left), capped and biased softmax
attention over a window and kept first positions through every attention kernel (keys far away, at the borders of
pages, windows and kept positions), and the table that names a token's experts."""
import math

import pytest
import torch

from plain import tilivik_plain as plain
from zedinfer_amd import ops
from zedinfer_amd.parts.linear_mixers import distance_bias_table

pytestmark = pytest.mark.gpu
DEV = "cuda"
F = torch.float64


def _close(got, want, tol, what=""):
    got, want = got.double().cpu(), want.double().cpu()
    scale = max(1.0, float(want.abs().max()))
    err = float((got - want).abs().max())
    assert err <= tol * scale, (what, err, scale)


def _i32(x):
    return torch.tensor(x, dtype=torch.int32, device=DEV)


def _entries(lens, slots, past):
    """The arrays that describe a step: entry e brings lens[e] tokens of the request in state slot slots[e] that holds
    past[e] tokens already."""
    start, tok_seq, pos, at = [], [], [], 0
    for e, n in enumerate(lens):
        start.append(at)
        tok_seq += [e] * n
        pos += list(range(past[e], past[e] + n))
        at += n
    return dict(entry_start=_i32(start), entry_len=_i32(lens), entry_past=_i32(past), entry_slot=_i32(slots),
                tok_seq=_i32(tok_seq), positions=_i32(pos))


# ---- the embedding ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("H, buckets, dtype", [(96, 97, torch.float32), (84, 7, torch.bfloat16), (130, 509, torch.float32)])
def test_the_summed_embedding_carries_the_token_before_from_step_to_step(H, buckets, dtype):
    V, mp, mc = 150, 29, 11
    g = torch.Generator().manual_seed(H)
    embed, pair = torch.randn(V, H, generator=g).to(dtype), torch.randn(buckets + 1, H, generator=g).to(dtype)
    a = torch.randint(0, V, (23,), generator=g).tolist()
    b = torch.randint(0, V, (9,), generator=g).tolist()
    hash_cfg = dict(buckets=buckets, mul_prev=mp, mul_cur=mc)
    want = {"a": plain.embedding(a, embed.double(), pair.double(), hash_cfg),
            "b": plain.embedding(b, embed.double(), pair.double(), hash_cfg)}
    freq = torch.tensor([10000.0 ** (-2.0 * i / H) for i in range((H + 1) // 2)], dtype=torch.float64, device=DEV)
    state = torch.full((3, 1), 77, dtype=torch.int32, device=DEV)      # what others left in the slots
    got = {"a": [], "b": []}
    fed = {"a": 0, "b": 0}
    # a in slot 2, b in slot 0; portions of unequal sizes, b joins later and is left out of a step
    for step in ([("a", 5)], [("a", 1), ("b", 4)], [("a", 7)], [("b", 1), ("a", 10)], [("b", 4)]):
        ids, lens, slots, past = [], [], [], []
        for rid, n in step:
            toks = a if rid == "a" else b
            ids += toks[fed[rid]:fed[rid] + n]
            lens.append(n)
            slots.append(2 if rid == "a" else 0)
            past.append(fed[rid])
        en = _entries(lens, slots, past)
        out = torch.empty(len(ids), H, device=DEV)
        ops.embedding_sum(_i32(ids), embed.to(DEV), out, en["positions"], pair=pair.to(DEV), buckets=buckets, mul_prev=mp,
                          mul_cur=mc, state=state, tok_seq=en["tok_seq"], entry_start=en["entry_start"],
                          entry_len=en["entry_len"], entry_slot=en["entry_slot"], freq=freq)
        at = 0
        for rid, n in step:
            got[rid].append(out[at:at + n].cpu())
            at += n
            fed[rid] += n
    for rid in ("a", "b"):
        _close(torch.cat(got[rid]), want[rid], 2e-6, rid)
    # without the pair table and the sinusoid: the rows themselves
    out = torch.empty(4, H, device=DEV)
    ops.embedding_sum(_i32(a[:4]), embed.to(DEV), out, _i32([0, 1, 2, 3]))
    _close(out, embed.double()[a[:4]], 1e-7, "rows")


def test_the_sinusoid_at_positions_far_out():
    H = 64
    embed = torch.zeros(3, H)
    freq = torch.tensor([10000.0 ** (-2.0 * i / H) for i in range(H // 2)], dtype=torch.float64, device=DEV)
    pos = [0, 1, 4095, 100000]
    out = torch.empty(len(pos), H, device=DEV)
    ops.embedding_sum(_i32([0, 1, 2, 0]), embed.to(DEV), out, _i32(pos), freq=freq)
    want = torch.tensor([[math.sin(p * 10000.0 ** (-2.0 * (c // 2) / H)) if c % 2 == 0 else
                          math.cos(p * 10000.0 ** (-2.0 * (c // 2) / H)) for c in range(H)] for p in pos], dtype=F)
    _close(out, want, 2e-6, "angles are made in double precision")


# ---- the token shift ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("H, dtype", [(96, torch.float32), (84, torch.bfloat16), (260, torch.float32)])
def test_the_token_shift_carries_the_row_before_from_step_to_step(H, dtype):
    g = torch.Generator().manual_seed(H)
    xa, xb = torch.randn(19, H, generator=g), torch.randn(6, H, generator=g)
    w = 0.5 * torch.randn(H, generator=g)
    want = {"a": plain.token_shift(xa.double(), w.double()), "b": plain.token_shift(xb.double(), w.double())}
    state = torch.full((2, H + 5), 3.0, device=DEV)       # the shifted row is the first H floats of a wider slot
    got, fed = {"a": [], "b": []}, {"a": 0, "b": 0}
    for step in ([("b", 2)], [("a", 3), ("b", 1)], [("a", 1)], [("a", 15), ("b", 3)]):
        rows, lens, slots, past = [], [], [], []
        for rid, n in step:
            x = xa if rid == "a" else xb
            rows.append(x[fed[rid]:fed[rid] + n])
            lens.append(n)
            slots.append(1 if rid == "a" else 0)
            past.append(fed[rid])
        en = _entries(lens, slots, past)
        x = torch.cat(rows).to(DEV)
        out = torch.empty(x.shape[0], H, dtype=dtype, device=DEV)
        ops.token_shift(x, w.to(DEV), state[:, :H], en["tok_seq"], en["positions"], en["entry_start"], en["entry_len"],
                        en["entry_slot"], out=out)
        at = 0
        for rid, n in step:
            got[rid].append(out[at:at + n].float().cpu())
            at += n
            fed[rid] += n
    assert float(state[:, H:].min()) == 3.0 == float(state[:, H:].max())          # nothing beyond the row is touched
    for rid in ("a", "b"):
        _close(torch.cat(got[rid]), want[rid], 2e-6 if dtype == torch.float32 else 1e-2, rid)


# ---- the decay gate -------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("C, rank, tau, dtype", [(48, 8, 16.0, torch.float32), (64, 1, 1.0, torch.bfloat16), (20, 33, 4.0, torch.float32)])
def test_the_decay_is_the_root_of_a_sigmoid_also_far_out(C, rank, tau, dtype):
    g = torch.Generator().manual_seed(C)
    u = torch.randn(7, rank + 3, generator=g) * 3
    u[0] *= 40                                                   # sigmoids of -100 and +100
    w2, b = torch.randn(C, rank, generator=g).to(dtype), (2 * torch.randn(C, generator=g)).to(dtype)
    z = u[:, :rank].double() @ w2.double().T + b.double()
    want = torch.exp(torch.nn.functional.logsigmoid(z) / tau)
    out = torch.empty(7, C, device=DEV)
    ops.lowrank_decay(u.to(DEV)[:, :rank], w2.to(DEV), b.to(DEV), tau, out=out)
    _close(out, want, 3e-6, "decay")
    assert float(out.min()) >= 0.0 and float(out.max()) <= 1.0 and bool(torch.isfinite(out).all())


# ---- linear attention ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("heads, dim, vdim, gated, silu", [
    (3, 16, 24, True, False), (4, 32, 32, False, True), (1, 48, 16, True, False), (2, 40, 24, False, True),
    (5, 12, 12, False, True), (2, 64, 128, True, False), (1, 144, 136, False, True), (1, 128, 64, True, False),
    (2, 8, 8, True, True), (1, 300, 20, True, False), (1, 520, 8, False, False)])
def test_linear_attention_in_portions_and_used_slots_is_the_plain_recurrence(heads, dim, vdim, gated, silu):
    if dim > 512:
        with pytest.raises(ops.KernelLibraryError):
            _linear_attention_case(heads, dim, vdim, gated, silu)
        return
    _linear_attention_case(heads, dim, vdim, gated, silu)


def _linear_attention_case(heads, dim, vdim, gated, silu):
    g = torch.Generator().manual_seed(heads * 1000 + dim)
    qk, vd = heads * dim, heads * vdim
    lens_of = {"a": 71, "b": 18, "c": 5}
    proj = {r: torch.randn(n, 2 * qk + vd + 3, generator=g) * 0.7 for r, n in lens_of.items()}      # q | k | v | other columns
    decay = {r: (0.5 + 0.5 * torch.rand(n, qk, generator=g)) for r, n in lens_of.items()}
    for r in decay:
        decay[r][::7] *= 0.1                                     # some strong forgetting
    head_decay = torch.tensor([0.5, 0.93, 0.999, 1.0, 0.8][:heads])
    qscale = dim ** -0.5 if gated else 1.0
    act = plain.silu if silu else (lambda z: z)
    want = {}
    for r, n in lens_of.items():
        p = proj[r].double()
        q, k, v = act(p[:, :qk]) * qscale, act(p[:, qk:2 * qk]), act(p[:, 2 * qk:2 * qk + vd])
        o = torch.zeros(n, heads, vdim, dtype=F)
        for h in range(heads):
            a = decay[r].double()[:, h * dim:(h + 1) * dim] if gated else torch.full((n, dim), float(head_decay[h]), dtype=F)
            o[:, h] = plain.decayed_linear_attention(q[:, h * dim:(h + 1) * dim], k[:, h * dim:(h + 1) * dim],
                                                     v[:, h * vdim:(h + 1) * vdim], a)
        want[r] = o.reshape(n, vd)
    floats = ops.linear_attention_state_floats(heads, dim, vdim)
    state = torch.full((3, floats + 4), 5.0, device=DEV)        # whoever had the slot before left something
    slot = {"a": 2, "b": 0, "c": 2}                             # c runs in a's slot after a has ended
    got, fed = {r: [] for r in lens_of}, {r: 0 for r in lens_of}
    steps = ([("a", 17)], [("a", 1), ("b", 2)], [("b", 16), ("a", 33)], [("a", 1)], [("a", 19)], [("c", 2)], [("c", 1)], [("c", 2)])
    for step in steps:
        rows, drows, lens, slots, past = [], [], [], [], []
        for rid, n in step:
            rows.append(proj[rid][fed[rid]:fed[rid] + n])
            drows.append(decay[rid][fed[rid]:fed[rid] + n])
            lens.append(n)
            slots.append(slot[rid])
            past.append(fed[rid])
        en = _entries(lens, slots, past)
        x = torch.cat(rows).to(DEV)
        out = torch.full((x.shape[0], vd), 9.0, device=DEV)
        ops.linear_attention(x[:, :qk], x[:, qk:2 * qk], x[:, 2 * qk:2 * qk + vd], state[:, 2:2 + floats], en["entry_start"],
                             en["entry_len"], en["entry_past"], en["entry_slot"], heads, dim, vdim, out=out,
                             decay=torch.cat(drows).to(DEV) if gated else None,
                             head_decay=None if gated else head_decay.to(DEV), silu=silu, qscale=qscale)
        at = 0
        for rid, n in step:
            got[rid].append(out[at:at + n].cpu())
            at += n
            fed[rid] += n
    for r in lens_of:
        _close(torch.cat(got[r]), want[r], 3e-5, r)
    assert float(state[:, :2].min()) == 5.0 == float(state[:, floats + 2:].max())      # nothing beside the state is touched
    assert float(state[1].min()) == 5.0 == float(state[1].max())                        # nor a slot of no entry


def test_a_cut_of_the_prompt_changes_no_bit_of_linear_attention():
    heads, dim, vdim, n = 2, 32, 48, 50
    g = torch.Generator().manual_seed(5)
    x = torch.randn(n, 2 * heads * dim + heads * vdim, generator=g).to(DEV)
    a = (0.6 + 0.4 * torch.rand(n, heads * dim, generator=g)).to(DEV)
    qk = heads * dim
    outs = []
    for cuts in ([50], [1] * 50, [3, 16, 1, 17, 13], [16, 16, 16, 2]):
        state = torch.zeros(1, ops.linear_attention_state_floats(heads, dim, vdim), device=DEV)
        out, at = torch.empty(n, heads * vdim, device=DEV), 0
        for c in cuts:
            en = _entries([c], [0], [at])
            ops.linear_attention(x[at:at + c, :qk], x[at:at + c, qk:2 * qk], x[at:at + c, 2 * qk:], state, en["entry_start"],
                                 en["entry_len"], en["entry_past"], en["entry_slot"], heads, dim, vdim, out=out[at:at + c],
                                 decay=a[at:at + c])
            at += c
        outs.append((out.clone(), state.clone()))
    for o, s in outs[1:]:
        assert torch.equal(o, outs[0][0]) and torch.equal(s, outs[0][1])


@pytest.mark.parametrize("groups, size, act, dtype", [(1, 120, "sigmoid", torch.bfloat16), (3, 24, "silu", torch.float32),
                                                      (8, 8, "silu", torch.bfloat16), (2, 136, "sigmoid", torch.float32)])
def test_the_read_out_is_normed_per_group_and_gated(groups, size, act, dtype):
    g = torch.Generator().manual_seed(size)
    n, W = 11, groups * size
    o, gate, w = torch.randn(n, W, generator=g) * 4, torch.randn(n, W + 2, generator=g), 1 + 0.2 * torch.randn(size, generator=g)
    normed = plain.rms(o.double().view(n, groups, size), 1e-5) * w.double()
    gd = gate.double()[:, :W]
    want = normed.reshape(n, W) * (torch.sigmoid(gd) if act == "sigmoid" else plain.silu(gd)) * 0.7
    out = torch.zeros(n, W + 6, dtype=dtype, device=DEV)
    ops.gated_rms_norm_act(o.to(DEV), w.to(DEV), gate.to(DEV)[:, :W], groups, size, 1e-5, act, out=out[:, 3:3 + W], scale=0.7)
    _close(out[:, 3:3 + W], want, 2e-6 if dtype == torch.float32 else 1e-2, "read-out")
    assert float(out[:, :3].abs().max()) == 0.0 and float(out[:, 3 + W:].abs().max()) == 0.0


# ---- capped and biased attention -------------------------------------------------------------------------------------
def _paged(n_tokens, ps, seed, spare=3):
    """A block table that scatters the pages of one sequence over a pool, and every token's slot."""
    pages = -(-n_tokens // ps)
    perm = torch.randperm(pages + spare, generator=torch.Generator().manual_seed(seed))[:pages]
    table = perm.to(torch.int32)
    pos = torch.arange(n_tokens)
    slots = (table[pos // ps].long() * ps + pos % ps).to(torch.int32)
    return table.view(1, -1), slots, pages + spare


def _plain_attention(q, k, v, m, rel, eps):
    """The plain mixer's attention alone: projections that hand q, k and v through, a gate of one half that the
    output matrix doubles."""
    T, H, G, dim, vdim = q.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    h = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], dim=1).double()
    W, qd, kd, vd = h.shape[1], H * dim, G * dim, G * vdim
    eye = torch.eye(W, dtype=F)
    w = {"q": eye[:qd], "k": eye[qd:qd + kd], "v": eye[qd + kd:], "g": torch.zeros(H * vdim, W, dtype=F),
         "o": 2.0 * torch.eye(H * vdim, dtype=F)}
    if rel is not None:
        w["rel"] = rel.double()
    return plain.biased_window_attention(h, w, m, eps)


CASES = [
    # T, heads, kv_heads, dim, vdim, page, window, keep_first, softcap, bias rows, far distance
    (300, 4, 2, 32, 16, 8, 20, 3, 8.0, 12, 40),
    (700, 8, 4, 48, 64, 16, 90, 7, 25.0, 24, 150),
    (450, 2, 1, 128, 96, 16, 200, 130, 50.0, 32, 1000),        # kept positions over more than a block of keys
    (333, 3, 3, 24, 24, 8, 0, 0, 0.0, 8, 64),                   # a bias alone, all keys
    (280, 12, 1, 16, 16, 32, 16, 1, 2.0, 16, 24),
    (260, 5, 5, 20, 12, 4, 9, 4, 5.0, 0, 0),                    # no bias; heads that no matrix-core kernel takes
    (2500, 2, 2, 64, 64, 16, 2300, 5, 20.0, 6, 3000),           # a window longer than a cut of the keys
    (1100, 4, 1, 64, 32, 16, 600, 40, 0.0, 4, 50),              # kept positions without a cap
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_capped_biased_windowed_attention_through_every_kernel(case, dtype):
    T, H, G, dim, vdim, ps, window, keep, cap, rows, far = case
    g = torch.Generator().manual_seed(T)
    q = torch.randn(T, H, dim, generator=g).to(dtype).float()
    k = torch.randn(T, G, dim, generator=g).to(dtype).float()
    v = torch.randn(T, G, vdim, generator=g) * 2
    # queries near the end ask for one key each with a score that stands out: one far back inside the window's first
    # place, one just outside it, one among the kept positions and the first position after them
    marks = {T - 1: max(T - window, 0) if window else 1, T - 2: max(T - 2 - window, 0) if window else 2,
             T - 3: max(keep - 1, 0), T - 4: keep, T - 40: max(T - 39 - window, 0) if window else 3}
    for qi, kj in marks.items():
        for a in range(H):
            q[qi, a] = (6.0 / dim ** 0.5) * k[kj, a // (H // G)] / k[kj, a // (H // G)].norm() * dim ** 0.5
    q = q.to(dtype).float()
    scale = 1.0 / dim ** 0.5
    m = dict(heads=H, kv_heads=G, dim=dim, vdim=vdim, scale=scale)
    if cap:
        m["softcap"] = cap
    if window:
        m["mask"] = dict(size=window, keep_first=keep)
    rel = None
    if rows:
        m["bias_max"] = far
        rel = 1.5 * torch.randn(rows, H, generator=g)
    eps = 1e-5
    d = max(dim, vdim)
    if dtype == torch.bfloat16 and d <= 128:
        d = -(-d // 16) * 16
    # the values are normed and rounded as the cache holds them
    table, slots, pages = _paged(T, ps, seed=T)
    proj = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], dim=1).to(DEV)
    kc = torch.full((pages, G, ps, d), 7.0, dtype=dtype, device=DEV)
    vc = torch.full((pages, G, d, ps), 7.0, dtype=dtype, device=DEV)
    qd, kd = H * dim, G * dim
    q_dev = torch.empty(T, H * d, dtype=dtype, device=DEV)
    ops.normed_kv_store(proj, 0, qd, qd + kd, q_dev, slots.to(DEV), kc, vc, H, G, dim, vdim, d, eps)
    want = _plain_attention(q, k, v, dict(m), rel, eps)
    bias = distance_bias_table(rel.to(DEV), float(far)) if rows else None
    tol = 2e-5 if dtype == torch.float32 else 2.5e-2
    pos = torch.arange(T, dtype=torch.int32, device=DEV)
    seq0 = torch.zeros(T, dtype=torch.int32, device=DEV)
    tab = table.to(DEV)
    extras = dict(softcap=cap, bias=bias, keep_first=keep)

    def heads_of(att):
        return att.float().view(T, H, d)[:, :, :vdim].reshape(T, H * vdim)

    # the plain kernel (every type and size)
    att = torch.zeros(T, H * d, dtype=dtype, device=DEV)
    ops.attention_biased(q_dev, kc, vc, seq0, pos, tab, H, G, d, scale, window, out=att, **extras)
    _close(heads_of(att), want, tol, "plain kernel")
    if not (ops.attention_decode_supported(dtype, H, G, d, ps) and ops.attention_prefill_supported(dtype, H, G, d, ps)):
        return
    # every token alone, its keys split over wavefronts and chunks
    att = torch.zeros(T, H * d, dtype=dtype, device=DEV)
    ops.attention_decode(q_dev, kc, vc, seq0, pos, tab, H, G, d, scale, T, window, out=att, **extras)
    _close(heads_of(att), want, tol, "single tokens")
    # a few tokens of the list only
    some = _i32([T - 1, T - 3, 5, T - 40])
    att2 = torch.zeros(T, H * d, dtype=dtype, device=DEV)
    ops.attention_decode(q_dev, kc, vc, seq0, pos, tab, H, G, d, scale, T, window, out=att2, tok_index=some, **extras)
    assert torch.equal(att2[some.long()], att[some.long()]) and float(att2[6].abs().max()) == 0.0
    # portions of the prompt as tiles of queries: the whole prompt, and a portion that continues it
    tile = ops.attention_prefill_tile_min()
    for past in (0, T - 150, T - 70):
        n = T - past
        offs = list(range(0, n, tile))
        att = torch.zeros(n, H * d, dtype=dtype, device=DEV)
        ops.attention_prefill(q_dev[past:], kc, vc, _i32([0] * len(offs)), _i32(offs), _i32([0]), _i32([n]), _i32([past]), tab,
                              H, G, d, scale, window, out=att, max_keys=T, tile=tile, **extras)
        got = att.float().view(n, H, d)[:, :, :vdim].reshape(n, H * vdim)
        _close(got, want[past:], tol, ("tiles", past))


def test_the_marked_keys_do_carry_the_weight():
    """The test above is blind to a window that is one key off unless the keys at the edges matter: with the plain
    functions alone, moving the window or the kept positions by one changes the marked rows."""
    T, H, G, dim, vdim, window, keep = 120, 2, 1, 16, 8, 20, 3
    g = torch.Generator().manual_seed(1)
    q, k, v = torch.randn(T, H, dim, generator=g), torch.randn(T, G, dim, generator=g), torch.randn(T, G, vdim, generator=g)
    for qi, kj in ((T - 1, T - window), (T - 3, keep - 1)):
        for a in range(H):
            q[qi, a] = 6.0 * k[kj, 0] / k[kj, 0].norm()
    m = dict(heads=H, kv_heads=G, dim=dim, vdim=vdim, scale=1.0, mask=dict(size=window, keep_first=keep))
    base = _plain_attention(q, k, v, m, None, 1e-6)
    narrower = _plain_attention(q, k, v, dict(m, mask=dict(size=window - 1, keep_first=keep)), None, 1e-6)
    fewer = _plain_attention(q, k, v, dict(m, mask=dict(size=window, keep_first=keep - 1)), None, 1e-6)
    assert float((base[T - 1] - narrower[T - 1]).abs().max()) > 0.3
    assert float((base[T - 3] - fewer[T - 3]).abs().max()) > 0.3
    assert float((base[T - 2] - fewer[T - 2]).abs().max()) < 0.05


# ---- the experts' table ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("V, E, top", [(50, 5, 2), (211, 16, 4), (9, 3, 3), (30, 7, 1)])
def test_the_table_names_every_tokens_experts_with_equal_weights(V, E, top):
    g = torch.Generator().manual_seed(V)
    table = torch.rand(V, E, generator=g).argsort(dim=1)[:, :top].to(torch.int32).contiguous()
    ids = torch.randint(0, V, (37,), generator=g).to(torch.int32)
    idx = torch.empty(37 * top, dtype=torch.int32, device=DEV)
    wt = torch.empty(37, top, device=DEV)
    ops.moe_route_table(ids.to(DEV), table.to(DEV), E, idx, wt)
    assert torch.equal(idx.view(37, top).cpu(), table[ids.long()])
    assert torch.equal(wt.cpu(), torch.full((37, top), 1.0 / top))
