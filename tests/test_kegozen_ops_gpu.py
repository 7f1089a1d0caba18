"""Every new mechanism of the Kegozen design alone, on the GPU, against the plain functions of
``tests/plain/kegozen_plain.py``: the state-space recurrence with its convolution and gated norm (whole, and cut into
steps through the state), the rotation tables, the store into the token cache with norm and rotation, the blocks'
means, attention over window and blocks through shuffled pages, the norm on a sublayer's output, and the experts with
scored inputs.  Sizes are the tests' own."""
import math

import numpy as np
import pytest
import torch

from plain import kegozen_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda"
F64 = torch.float64


def _i32(x):
    return torch.tensor(x, dtype=torch.int32, device=DEV)


def _close(got, want, tol, what=""):
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    err = float((got - want).abs().max())
    assert err <= tol * max(1.0, float(want.abs().max())), (what, err, float(want.abs().max()))


@pytest.mark.parametrize("heads,vdim,N,G,taps,parts,cuts", [
    (4, 16, 16, 2, 4, 2, [37]), (4, 16, 16, 2, 4, 2, [5, 1, 2, 20, 9]), (3, 24, 8, 1, 3, 1, [1, 1, 1, 30, 1, 1]), (2, 72, 40, 2, 4, 1, [1, 1, 1, 1, 5, 1]),
    (5, 20, 12, 5, 2, 5, [2, 2, 33]), (2, 64, 128, 1, 4, 1, [17, 3]), (6, 8, 40, 3, 1, 6, [11, 11])])
def test_state_space_mechanism_whole_and_through_the_state(heads, vdim, N, G, taps, parts, cuts):
    from zedinfer_amd import ops
    g = torch.Generator().manual_seed(heads * 100 + N)
    inner, gn = heads * vdim, G * N
    C, width, T = inner + 2 * gn, 2 * inner + 2 * gn + heads, sum(cuts)
    proj = torch.randn((T, width), generator=g)
    conv_w, conv_b = 0.5 * torch.randn((C, taps), generator=g), 0.2 * torch.randn((C,), generator=g)
    dt_bias, a_log = torch.randn((heads,), generator=g) - 1.0, torch.log(0.2 + 3 * torch.rand((heads,), generator=g))
    skip, gain = 1 + 0.5 * torch.randn((heads,), generator=g), 1 + 0.2 * torch.randn((inner,), generator=g)
    eps = 1e-5
    # the plain mechanism on the whole sequence
    p64 = proj.to(F64)
    rest = plain.silu(plain.causal_convolution(p64[:, inner:inner + C], conv_w.to(F64), conv_b.to(F64)))
    u = rest[:, :inner].reshape(T, heads, vdim)
    B, Cc = rest[:, inner:inner + gn].reshape(T, G, N), rest[:, inner + gn:].reshape(T, G, N)
    dt = plain.softplus(p64[:, inner + C:] + dt_bias.to(F64))
    y = torch.zeros((T, heads, vdim), dtype=F64)
    for a in range(heads):
        y[:, a] = plain.state_space_head(u[:, a], B[:, a // (heads // G)], Cc[:, a // (heads // G)], dt[:, a],
                                         float(a_log[a]), float(skip[a]))
    want = y.reshape(T, inner) * plain.silu(p64[:, :inner])
    want = plain.rms(want.reshape(T, parts, inner // parts), eps).reshape(T, inner) * gain.to(F64)
    # the kernels, step by step, the state in slot 2 of 4 (slot 1 holds garbage that a fresh entry must not read...
    # a fresh request's slot is zeroed by the cache manager, so the slot starts at zero here as well)
    floats = ops.ssm_state_floats(heads, vdim, N, G, taps)
    state = torch.randn((4, max(1, floats)), device=DEV)
    state[2].zero_()
    tail = (taps - 1) * C
    d = lambda t: t.to(DEV).contiguous()      # noqa: E731
    got = torch.zeros((T, inner), device=DEV)
    at = 0
    for n in cuts:
        pr = d(proj[at:at + n])
        prep = torch.empty((n, width), device=DEV)
        es, el, ep, sl = _i32([0]), _i32([n]), _i32([at]), _i32([2])
        ops.ssm_prepare(pr, d(conv_w), d(conv_b), d(dt_bias), d(a_log), state, _i32([0] * n), es, sl, heads, vdim, N, G, taps, out=prep)
        if taps > 1:
            ops.conv_tail(state, pr[:, inner:inner + C], None, es, el, sl, taps)
        yy = torch.empty((n, inner), device=DEV)
        ops.linear_attention_grouped(prep[:, inner + gn:C], prep[:, inner:inner + gn], prep[:, C:C + inner], prep[:, C + inner:],
                                     state[:, tail:], es, el, ep, sl, heads, heads // G, N, vdim, out=yy,
                                     single_tokens=(n == 1 and at % 2 == 0))      # decoded tokens: either kernel
        ops.ssm_finish(yy, prep[:, :inner], pr[:, :inner], d(skip), d(gain), heads, vdim, parts, eps, out=got[at:at + n])
        at += n
    _close(got, want, 2e-4, "state space")


def test_rotation_tables_follow_the_ramp():
    from zedinfer_amd import ops
    from zedinfer_amd.parts.pooled_attention import halves_order, ramped_frequencies
    for dims, base, scaling in ((16, 5000.0, dict(factor=8.0, original=64, fast=16.0, slow=2.0)), (24, 300.0, None),
                                (64, 1e6, dict(factor=4.0, original=32, fast=8.0, slow=1.0)),
                                (10, 100.0, dict(factor=2.0, original=16, fast=4.0, slow=1.0))):
        f, mag = ramped_frequencies(dims, base, scaling)
        wf, wmag = plain.pair_frequencies(dims, base, scaling)
        assert np.allclose(f, np.array(wf, dtype=np.float32), rtol=1e-6) and abs(mag - wmag) < 1e-12
        if scaling:
            assert mag > 1.0 and f[-1] < wf[-1] * 1.0001 and f[0] == np.float32(1.0)
        pos = _i32([0, 1, 7, 300])
        table = torch.empty((4, dims // 2, 2), device=DEV)
        ops.rope_table_scaled(pos, torch.from_numpy(f).to(DEV), mag, out=table)
        for r, p in enumerate([0, 1, 7, 300]):
            for i in range(dims // 2):
                assert abs(float(table[r, i, 0]) - math.cos(p * wf[i]) * wmag) < 3e-4
                assert abs(float(table[r, i, 1]) - math.sin(p * wf[i]) * wmag) < 3e-4
    assert halves_order(8, 4).tolist() == [0, 2, 1, 3, 4, 5, 6, 7]


def _paged(T, ps, extra=3, seed=0):
    """A block table for T rows over shuffled pages: (table [1, pages], slots [T], total pages)."""
    rng = np.random.RandomState(seed)
    need = -(-T // ps)
    ids = rng.permutation(need + extra)[:need]
    slots = [int(ids[j // ps]) * ps + j % ps for j in range(T)]
    return ids.astype(np.int32), slots, need + extra


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,vd,rot,window,pool,ps,T", [
    (4, 2, 32, 16, 16, 20, 4, 8, 70), (3, 3, 24, 24, 24, 33, 8, 4, 90), (12, 2, 128, 128, 64, 40, 8, 16, 200),
    (6, 6, 64, 48, 64, 70, 32, 16, 210), (12, 1, 32, 32, 0, 16, 16, 8, 100), (2, 2, 96, 80, 32, 0, 0, 8, 75), (5, 5, 20, 12, 10, 5, 7, 4, 40),
    (2, 1, 8, 72, 0, 1, 3, 16, 30), (2, 1, 128, 96, 64, 50, 16, 16, 120), (4, 2, 16, 16, 8, 0, 0, 8, 45),
    (1, 1, 16, 8, 16, 12, 0, 8, 40)])
def test_store_blocks_and_attention_against_the_plain_mechanism(dtype, H, G, d, vd, rot, window, pool, ps, T):
    """q | k | v rows through norm, rotation and store, the blocks' means, and attention, with the tokens fed in three
    steps so that blocks straddle steps; pages are shuffled.  The plain side works on the values the cache holds."""
    from zedinfer_amd import ops
    from zedinfer_amd.parts.pooled_attention import ramped_frequencies
    g = torch.Generator().manual_seed(H * 1000 + d + T)
    proj = torch.randn((T, (H + G) * d + G * vd), generator=g)
    qg, kg = 1 + 0.2 * torch.randn((d,), generator=g), 1 + 0.2 * torch.randn((d,), generator=g)
    eps, scale, base = 1e-5, 0.7 / math.sqrt(d), 700.0
    scaling = dict(factor=4.0, original=32, fast=8.0, slow=1.0) if rot else None
    rotate_values = rot > 0
    # plain: norm, turn (split halves here: what the kernels turn), cache rounding, attention, turn back
    p64 = proj.to(F64)
    q = plain.rms(p64[:, :H * d].reshape(T, H, d), eps) * qg.to(F64)
    k = plain.rms(p64[:, H * d:(H + G) * d].reshape(T, G, d), eps) * kg.to(F64)
    v = p64[:, (H + G) * d:].reshape(T, G, vd)
    pos = list(range(T))
    if rot:
        f, mag = plain.pair_frequencies(rot, base, scaling)
        q, k = plain.turn(q, pos, f, "halves", mag), plain.turn(k, pos, f, "halves", mag)
    if rotate_values:
        vf, _ = plain.pair_frequencies(vd, base)
        v = plain.turn(v, pos, vf, "halves")
    rnd = (lambda t: t.to(dtype).to(F64))
    q, k, v = rnd(q), rnd(k), rnd(v)
    want = torch.zeros((T, H, vd), dtype=F64)
    for a in range(H):
        want[:, a] = plain.pooled_window_softmax(q[:, a], k[:, a // (H // G)], v[:, a // (H // G)], scale, window, pool)
    if rotate_values:
        want = plain.turn(want, [-p for p in pos], vf, "halves")
    # kernels
    ids, slots, pages = _paged(T, ps, seed=T)
    kc = torch.zeros((pages, ps, G, d), dtype=dtype, device=DEV)
    vc = torch.zeros((pages, ps, G, vd), dtype=dtype, device=DEV)
    table = _i32(ids.reshape(1, -1))
    kp = vp = ptab = None
    pslots = [-1] * T
    if pool > 0 and window > 0:
        rows = T // pool
        pids, prow_slots, ppages = _paged(max(rows, 1), ps, seed=T + 1)
        kp = torch.zeros((ppages, ps, G, d), dtype=torch.float32, device=DEV)
        vp = torch.zeros((ppages, ps, G, vd), dtype=torch.float32, device=DEV)
        ptab = _i32(pids.reshape(1, -1))
        for j in range(T):
            if (j + 1) % pool == 0:
                pslots[j] = prow_slots[j // pool]
    got = torch.zeros((T, H * vd), dtype=dtype, device=DEV)
    cores_ran = [0]
    cuts = [T // 3, 1, 3, T - T // 3 - 4]
    at = 0
    for n in cuts:
        positions = _i32(list(range(at, at + n)))
        tab = vtab = None
        if rot:
            fr, mg = ramped_frequencies(rot, base, scaling)
            tab = ops.rope_table_scaled(positions, torch.from_numpy(fr).to(DEV), mg, out=torch.empty((n, rot // 2, 2), device=DEV))
        if rotate_values:
            fr, _ = ramped_frequencies(vd, base, None)
            vtab = ops.rope_table_scaled(positions, torch.from_numpy(fr).to(DEV), 1.0, out=torch.empty((n, vd // 2, 2), device=DEV))
        qo = torch.empty((n, H * d), dtype=dtype, device=DEV)
        seqs = _i32([0] * n)
        ops.norm_rope_store(proj[at:at + n].to(DEV).contiguous(), qg.to(DEV), kg.to(DEV), eps, tab, vtab, _i32(slots[at:at + n]),
                            kc, vc, H, G, d, vd, q_out=qo)
        if kp is not None:
            ops.pool_blocks(kc, vc, kp, vp, _i32(pslots[at:at + n]), seqs, positions, table, G, d, vd, pool)
        ops.pooled_attention(qo, kc, vc, kp, vp, seqs, positions, table, ptab, H, G, d, vd, window, pool, scale,
                             out=got[at:at + n], vtable=vtab)
        if ops.pooled_attention_cores_supported(dtype, H, G, d, vd):
            # the matrix-core kernel on the same step: the entry as one portion, and beside two entries that it leaves
            # alone (one too short, one of no tokens)
            again = torch.full((n, H * vd), float("nan"), dtype=dtype, device=DEV)
            wide = torch.cat([table, table, table])
            wide_p = torch.cat([ptab, ptab, ptab]) if ptab is not None else None
            ops.pooled_attention_cores(qo, kc, vc, kp, vp, _i32([0, 0, 0]), _i32([n, 1, 0]), _i32([at, at, 0]), n, wide, wide_p,
                                       H, G, d, vd, window, pool, scale, out=again, vtable=vtab, long_len=min(n, 2))
            _close(again.float(), got[at:at + n].float(), 2e-2, "matrix cores against the plain kernel")
            cores_ran[0] += 1
            if n <= 64 // (H // G):
                # ... and as a short entry: its items cut into chunks over workgroups, merged by the second kernel
                for max_keys in (at + n, at + n + 300):
                    chunks, per = ops.pooled_attention_cores_cut(max_keys, window, pool, n, 256, G)
                    ws = torch.full((ops.pooled_attention_cores_workspace(n, H, vd, chunks),), float("nan"), device=DEV)
                    again = torch.full((n, H * vd), float("nan"), dtype=dtype, device=DEV)
                    ops.pooled_attention_cores(qo, kc, vc, kp, vp, _i32([0, 0]), _i32([n, 0]), _i32([at, 0]), n, wide[:2],
                                               wide_p[:2] if wide_p is not None else None, H, G, d, vd, window, pool, scale,
                                               out=again, vtable=vtab, long_len=n + 1, chunks=chunks, chunk_blocks=per,
                                               workspace=ws, tok_seq=seqs)
                    _close(again.float(), got[at:at + n].float(), 2e-2, "keys cut over workgroups against the plain kernel")
                cores_ran[0] += 1
        at += n
    _close(got.float().view(T, H, vd), want, 3e-4 if dtype == torch.float32 else 2e-2, "pooled attention")
    if dtype == torch.bfloat16 and d in (32, 64, 96, 128) and vd % 16 == 0 and vd <= 128:
        assert cores_ran[0] >= 2


def test_a_far_block_that_carries_the_weight():
    """One key far behind the window is large: the block that holds it must take the softmax, with a quarter of its
    value, exactly from the position at which the block is whole behind the window."""
    from zedinfer_amd import ops
    d, vd, window, pool, ps, T = 8, 8, 10, 4, 4, 300
    k = torch.zeros((T, 1, d)); v = torch.zeros((T, 1, vd)); q = torch.zeros((T, 1, d))
    q[:, 0, 0] = 1.0
    k[5, 0, 0] = 400.0           # in block 1 (positions 4..7): its mean key has 100 in dim 0
    v[5, 0, 1] = 8.0
    v[:, 0, 0] = 1.0
    want = plain.pooled_window_softmax(q[:, 0].to(F64), k[:, 0].to(F64), v[:, 0].to(F64), 1.0, window, pool)
    assert float(want[16, 1]) < 1e-9 and float(want[17, 1]) > 1.9 and float(want[299, 1]) > 1.9    # 7 <= i - 10 from i = 17 on
    ids, slots, pages = _paged(T, ps, seed=9)
    kc = torch.zeros((pages, ps, 1, d), device=DEV); vc = torch.zeros((pages, ps, 1, vd), device=DEV)
    kc.view(-1, 1, d)[slots] = k.to(DEV)
    vc.view(-1, 1, vd)[slots] = v.to(DEV)
    pids, prow, ppages = _paged(T // pool, ps, seed=10)
    kp = torch.zeros((ppages, ps, 1, d), device=DEV); vp = torch.zeros((ppages, ps, 1, vd), device=DEV)
    pslots = [prow[j // pool] if (j + 1) % pool == 0 else -1 for j in range(T)]
    positions, seqs, table = _i32(list(range(T))), _i32([0] * T), _i32(ids.reshape(1, -1))
    ops.pool_blocks(kc, vc, kp, vp, _i32(pslots), seqs, positions, table, 1, d, vd, pool)
    got = torch.empty((T, vd), device=DEV)
    ops.pooled_attention(q.view(T, d).to(DEV), kc, vc, kp, vp, seqs, positions, table, _i32(pids.reshape(1, -1)), 1, 1, d, vd,
                         window, pool, 1.0, out=got)
    _close(got, want, 1e-5, "far block")


@pytest.mark.parametrize("H,splits,then", [(96, 1, True), (84, 3, True), (256, 1, False), (2048, 2, True)])
def test_norm_on_an_output_and_the_next_norm(H, splits, then):
    from zedinfer_amd import ops
    g = torch.Generator().manual_seed(H)
    n, eps = 7, 3e-6
    y = torch.randn((splits, n, H), generator=g)
    resid = torch.randn((n, H), generator=g)
    w1, w2 = 0.3 * torch.randn((H,), generator=g), 0.3 * torch.randn((H,), generator=g)
    total = y.to(F64).sum(0)
    want_resid = resid.to(F64) + plain.one_plus_norm(total, w1.to(F64), eps)
    want_out = plain.one_plus_norm(want_resid, w2.to(F64), eps)
    r = resid.to(DEV).clone()
    out = torch.empty((n, H), device=DEV) if then else None
    ops.normed_add_norm(r, y.to(DEV) if splits > 1 else y[0].to(DEV), w1.to(DEV), eps, True, w2=w2.to(DEV) if then else None,
                        eps2=eps, out=out)
    _close(r, want_resid, 1e-5, "stream")
    if then:
        _close(out, want_out, 1e-5, "next norm")
    # bfloat16 input and output, a plain gain
    r = resid.to(DEV).clone()
    yb = total.float().to(torch.bfloat16)
    out = torch.empty((n, H), dtype=torch.bfloat16, device=DEV)
    ops.normed_add_norm(r, yb.to(DEV), w1.to(torch.bfloat16).to(DEV), eps, False, w2=w2.to(torch.bfloat16).to(DEV), eps2=eps, out=out)
    w1b, w2b = w1.to(torch.bfloat16).to(F64), w2.to(torch.bfloat16).to(F64)
    wr = resid.to(F64) + plain.rms(yb.to(F64), eps) * w1b
    _close(r, wr, 1e-5, "stream, bfloat16 rows")
    _close(out.float(), plain.rms(wr, eps) * w2b, 1e-2, "next norm, bfloat16")


@pytest.mark.parametrize("E,top,ff,shared,W,n", [(5, 2, 40, 24, 96, 33), (12, 1, 96, 0, 64, 70), (3, 3, 16, 16, 80, 5),
                                                  (70, 4, 8, 0, 48, 20)])
def test_scored_experts_against_the_plain_mixture(E, top, ff, shared, W, n):
    """The part itself (router, choice, grouping, products, weighted activation, sum, gated shared expert) in float32."""
    from zedinfer_amd.config.forward_config import PartSpec
    from zedinfer_amd.parts import FEED_FORWARDS, Runtime
    g = torch.Generator().manual_seed(E * 10 + top)
    w = {"router": torch.randn((E, W), generator=g) * (2.0 / W ** 0.5)}
    names = {"router": "router"}
    for e in range(E):
        for k, shape in (("gate", (ff, W)), ("up", (ff, W)), ("down", (W, ff))):
            w[f"{k}_{e}"] = torch.randn(shape, generator=g) / shape[1] ** 0.5
    if shared:
        w.update({"shared_gate": torch.randn((shared, W), generator=g) / W ** 0.5, "shared_up": torch.randn((shared, W), generator=g) / W ** 0.5,
                  "shared_down": torch.randn((W, shared), generator=g) / shared ** 0.5, "shared_sg": torch.randn((1, W), generator=g) / W ** 0.5})
    x = torch.randn((n, W), generator=g)
    pw = {"router": w["router"].to(F64)}
    for e in range(E):
        pw.update({f"e{e}.gate": w[f"gate_{e}"].to(F64), f"e{e}.up": w[f"up_{e}"].to(F64), f"e{e}.down": w[f"down_{e}"].to(F64)})
    mlp = dict(kind="moe", router=dict(experts=E, top=top), expert=dict(ff=ff))
    if shared:
        mlp["shared"] = dict(ff=shared)
        pw.update({"shared.gate": w["shared_gate"].to(F64), "shared.up": w["shared_up"].to(F64),
                   "shared.down": w["shared_down"].to(F64), "shared.sg": w["shared_sg"].to(F64)})
    want = plain.feed_forward(x.to(F64), pw, mlp)
    rt = Runtime(DEV, torch.float32)
    spec = PartSpec("scored_experts", {"hidden_size": W, "experts": E, "top": top, "ff": ff, "shared_ff": shared,
                                       "shared_gate": bool(shared)}, {})
    part = FEED_FORWARDS.get("scored_experts")(spec, {k: t.to(DEV) for k, t in w.items()}, rt)
    got = part.forward(x.to(DEV))
    _close(got, want, 1e-4, "scored experts")
    # the weight goes into the input: doubling a score is not doubling the expert's output
    h = x[:1].to(F64)
    one = plain.gated_expert(0.5 * h, pw, "e0.")
    assert float((one - 0.5 * plain.gated_expert(h, pw, "e0.")).abs().max()) > 1e-4
