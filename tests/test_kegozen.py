"""The Kegozen design on the CPU: its config.json reader, its description in parts, the cache manager's groups of one
row for every so many positions, the reordering of paired dims at load, and the plain implementation's own mechanisms
held against each other (a window that covers everything is plain causal attention; values turned by their own
position and turned back by the query's are values turned by the distance; a cut of a sequence through the state)."""
import copy
import math

import numpy as np
import pytest
import torch

import kegozen_models as models
from plain import kegozen_plain as plain

F64 = torch.float64


def _config(d):
    from zedinfer_amd.config import find_architecture
    arch = find_architecture(d)
    return arch, arch.config_cls.from_dict(d)


def test_the_registry_knows_the_design_and_every_size_comes_from_the_config():
    from zedinfer_amd.models import expected_weights
    for name, cfg in models.CONFIGS.items():
        arch, c = _config(cfg)
        assert arch.name == "Kegozen" and c.hidden_size == cfg["width"] and c.vocab_size == cfg["vocab"]
        fc = arch.forward_config(c)
        want = models.tensor_shapes(cfg)
        got = expected_weights(fc)
        assert set(got) == set(want)
        assert all(tuple(got[k].shape) == tuple(want[k]) for k in want), name
        assert [l.block for l in fc.layers] == ["sandwich"] * len(cfg["layers"])
        kinds = {"mamba2": "state_space", "attention": "pooled_window_attention", "latent_attention": "latent_attention"}
        assert [l.mixer.kind for l in fc.layers] == [kinds[x["type"]] for x in cfg["layers"]]
        assert c.to_dict()["layers"] == cfg["layers"]
    for seed in range(40):
        cfg = models.random_config(seed)
        arch, c = _config(cfg)
        assert set(expected_weights(arch.forward_config(c))) == set(models.tensor_shapes(cfg))


def test_constants_of_a_layer_reach_its_part():
    arch, c = _config(models.MAIN)
    fc = arch.forward_config(c)
    a = fc.layers[0].mixer.params
    assert (a["window"], a["pool"], a["rotary_dim"], a["theta"], a["pairing"]) == (20, 4, 16, 5000.0, "interleaved")
    assert a["scaling"] == dict(factor=8.0, original=64, fast=16.0, slow=2.0) and a["rotate_values"] and a["qk_norm"]
    s = fc.layers[1].mixer.params
    assert (s["heads"], s["vdim"], s["state"], s["groups"], s["conv"], s["norm_groups"]) == (4, 16, 16, 2, 4, 2)
    la = fc.layers[2].mixer.params
    assert (la["q_rank"], la["pairing"], la["window"], la["kv_rank"]) == (40, "halves", 0, 24)
    assert fc.layers[2].feed_forward.kind == "none" and fc.layers[1].feed_forward.kind == "swiglu"
    e = fc.layers[0].feed_forward.params
    assert (e["experts"], e["top"], e["ff"], e["shared_ff"], e["shared_gate"]) == (5, 2, 40, 24, True)
    assert fc.layers[3].feed_forward.params["shared_ff"] == 0
    assert all(n.params["add_one"] and n.params["eps"] == 3e-6 for n in fc.layers[0].norms.values())


@pytest.mark.parametrize("change,word", [
    (lambda c: c.pop("norm"), "norm"), (lambda c: c["layers"][0].update(type="conv"), "type"),
    (lambda c: c["layers"][0]["mixer"].pop("kv_heads"), "kv_heads"), (lambda c: c["layers"][1]["mixer"].update(groups=3), "groups"),
    (lambda c: c["layers"][1]["mixer"].update(norm_groups=5), "norm_groups"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=15), "rot"), (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=40), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"]["mask"].update(size=0), "mask.size"), (lambda c: c["layers"][2]["mixer"]["rot"].update(dims=4), "rot_dim"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), "top"), (lambda c: c["layers"][1]["mlp"].update(kind="other"), "kind"),
    (lambda c: c["layers"][0]["mlp"]["shared"].update(ff=0), "shared"), (lambda c: c["layers"][0]["mixer"].update(heads=3), "kv_heads")])
def test_a_config_that_cannot_be_built_is_refused_with_the_key_named(change, word):
    from zedinfer_amd.config import ConfigError
    cfg = copy.deepcopy(models.MAIN)
    change(cfg)
    with pytest.raises(ConfigError) as e:
        _config(cfg)
    assert word in str(e.value)


def test_a_cache_of_one_row_for_every_block_of_positions():
    """Pages of such a group are taken as blocks become whole, a token's slot is the row its position completes, and
    the pool is as much smaller as the blocks are long."""
    from zedinfer_amd.cache.manager import CacheManager
    from zedinfer_amd.parts.base import PAGE, KVCacheRequest, PageTensor
    t = (("k", PageTensor((PAGE, 1, 4))),)
    kv = {0: KVCacheRequest("window", 6, t), (0, "blocks"): KVCacheRequest("full", 0, t, stride=3),
          1: KVCacheRequest("full", 0, t)}
    cm = CacheManager(kv, {}, num_pages=30, page_size=4, max_requests=2, dtype=torch.float32, device=None)
    assert [(g.kind, g.stride) for g in cm.groups] == [("window", 1), ("full", 1), ("full", 3)]
    assert cm.groups[2].pool.total == 30 // 3 + 2 and cm.group_of_cache[(0, "blocks")] == 2
    seq = cm.open("a", 40)
    cm.ensure(seq, 2)
    assert seq.pages[2] == []                                  # no block is whole yet
    assert cm.token_slots(seq, 2, 0, 2).tolist() == [-1, -1]
    cm.commit(seq, 2)
    cm.ensure(seq, 14)                                         # blocks 0..3 become whole at positions 2, 5, 8, 11
    assert len(seq.pages[2]) == 1 and seq.pages[2][0] >= 0
    p = seq.pages[2][0]
    assert cm.token_slots(seq, 2, 2, 12).tolist() == [p * 4, -1, -1, p * 4 + 1, -1, -1, p * 4 + 2, -1, -1, p * 4 + 3, -1, -1]
    cm.commit(seq, 14)
    cm.ensure(seq, 15)                                         # position 14 completes block 4: the second page
    assert len(seq.pages[2]) == 2 and cm.token_slots(seq, 2, 14, 1).tolist() == [seq.pages[2][1] * 4]
    cm.commit(seq, 15)
    assert seq.pages[0][0] == -1 and seq.pages[0][1] == -1 and seq.pages[0][2] >= 0     # the window gave pages back
    assert all(x >= 0 for x in seq.pages[2])                                            # the blocks stay
    cm.check()
    other = cm.open("b", 10)
    cm.ensure(other, 9)
    assert set(other.pages[2]).isdisjoint(seq.pages[2])
    cm.close(seq)
    cm.close(other)
    cm.check()
    assert cm.groups[2].pool.num_held == 0
    with pytest.raises(ValueError):
        CacheManager({0: KVCacheRequest("window", 6, t, stride=2)}, {}, 8, 4, 1, torch.float32, None)


def test_the_decode_image_places_block_rows_like_the_batch_builder():
    """The host image that decode steps keep from step to step gives a token the slot of the block it completes."""
    from zedinfer_amd.cache.manager import CacheManager
    from zedinfer_amd.parts.base import PAGE, KVCacheRequest, PageTensor
    t = (("k", PageTensor((PAGE, 1, 4))),)
    cm = CacheManager({0: KVCacheRequest("full", 0, t), (0, "blocks"): KVCacheRequest("full", 0, t, stride=3)}, {},
                      num_pages=16, page_size=2, max_requests=2, dtype=torch.float32, device=None)
    seq = cm.open("a", 20)
    got = []
    for pos in range(20):
        cm.ensure(seq, pos + 1)
        got.append(int(cm.token_slots(seq, 1, pos, 1)[0]))
        cm.commit(seq, pos + 1)
    rows = [g for g in got if g >= 0]
    assert [i for i, g in enumerate(got) if g >= 0] == [2, 5, 8, 11, 14, 17]
    assert rows == [seq.pages[1][b // 2] * 2 + b % 2 for b in range(6)]


def test_reordering_paired_dims_changes_no_score():
    """A checkpoint pairs dims (2i, 2i + 1); the kernels turn (i, i + R/2).  Reordering the rows of both projections
    and the gains the same way gives the same scores after the rotation."""
    from zedinfer_amd.parts.pooled_attention import halves_order
    g = torch.Generator().manual_seed(1)
    T, H, d, R = 6, 2, 12, 8
    q, k = torch.randn((T, H, d), generator=g, dtype=F64), torch.randn((T, H, d), generator=g, dtype=F64)
    f, mag = plain.pair_frequencies(R, 50.0, dict(factor=2.0, original=8, fast=2.0, slow=1.0))
    pos = list(range(T))
    a = torch.einsum("thd,shd->hts", plain.turn(q, pos, f, "interleaved", mag), plain.turn(k, pos, f, "interleaved", mag))
    order = halves_order(d, R)
    b = torch.einsum("thd,shd->hts", plain.turn(q[:, :, order], pos, f, "halves", mag), plain.turn(k[:, :, order], pos, f, "halves", mag))
    assert float((a - b).abs().max()) < 1e-12
    # latent attention goes the other way: a checkpoint's halves become neighbours
    R2 = 6
    order2 = torch.tensor([j // 2 + (j % 2) * (R2 // 2) for j in range(R2)])
    f2, _ = plain.pair_frequencies(R2, 100.0)
    x, y = torch.randn((T, 1, R2), generator=g, dtype=F64), torch.randn((T, 1, R2), generator=g, dtype=F64)
    a = torch.einsum("thd,shd->ts", plain.turn(x, pos, f2, "halves"), plain.turn(y, pos, f2, "halves"))
    b = torch.einsum("thd,shd->ts", plain.turn(x[:, :, order2], pos, f2, "interleaved"), plain.turn(y[:, :, order2], pos, f2, "interleaved"))
    assert float((a - b).abs().max()) < 1e-12


def test_the_ramp_keeps_fast_pairs_and_slows_slow_ones():
    from zedinfer_amd.parts.pooled_attention import ramped_frequencies
    f, mag = ramped_frequencies(48, 20000.0, dict(factor=4.0, original=1024, fast=32.0, slow=1.0))
    plainf = np.power(20000.0, -2.0 * np.arange(24) / 48)
    assert f[0] == 1.0 and abs(f[-1] - plainf[-1] / 4.0) < 1e-9 and abs(mag - (0.1 * math.log(4.0) + 1.0)) < 1e-12
    ratio = f / plainf
    assert all(ratio[i] >= ratio[i + 1] - 1e-7 for i in range(23)) and ratio.min() >= 0.25 - 1e-6
    with pytest.raises(ValueError):
        ramped_frequencies(8, 100.0, dict(factor=2.0))


def test_plain_mechanisms_agree_with_each_other():
    g = torch.Generator().manual_seed(3)
    T, d, vd = 30, 8, 6
    q, k, v = (torch.randn((T, n), generator=g, dtype=F64) for n in (d, d, vd))
    # a window that covers everything is causal attention, whatever the blocks
    s = (q @ k.T) * 0.3
    s = s.masked_fill(torch.triu(torch.ones((T, T), dtype=torch.bool), diagonal=1), float("-inf"))
    assert float((plain.pooled_window_softmax(q, k, v, 0.3, T, 4) - torch.softmax(s, 1) @ v).abs().max()) < 1e-12
    assert float((plain.pooled_window_softmax(q, k, v, 0.3, 0, 4) - torch.softmax(s, 1) @ v).abs().max()) < 1e-12
    # blocks of one position are the positions themselves: a window with such blocks sees everything as well
    assert float((plain.pooled_window_softmax(q, k, v, 0.3, 5, 1) - torch.softmax(s, 1) @ v).abs().max()) < 1e-12
    # and with longer blocks it does not
    assert float((plain.pooled_window_softmax(q, k, v, 0.3, 5, 4) - torch.softmax(s, 1) @ v).abs().max()) > 1e-3
    # values turned by their own position and the sum turned back by the query's: turned by the (negative) distance
    f, _ = plain.pair_frequencies(vd, 30.0)
    turned = plain.turn(v.reshape(T, 1, vd), list(range(T)), f, "interleaved")
    back = plain.turn(turned[3:4], [-7], f, "interleaved")
    direct = plain.turn(v[3].reshape(1, 1, vd), [3 - 7], f, "interleaved")
    assert float((back - direct).abs().max()) < 1e-12
    # the recurrence cut in two through its state gives the same rows
    u, B, C = (torch.randn((T, n), generator=g, dtype=F64) for n in (5, 4, 4))
    dt = torch.rand((T,), generator=g, dtype=F64)
    whole = plain.state_space_head(u, B, C, dt, 0.3, 0.7)
    S = torch.zeros((4, 5), dtype=F64)
    rows = []
    for t in range(T):
        S = math.exp(-math.exp(0.3) * float(dt[t])) * S + float(dt[t]) * torch.outer(B[t], u[t])
        rows.append(S.T @ C[t] + 0.7 * u[t])
    assert float((whole - torch.stack(rows)).abs().max()) < 1e-12


def test_the_plain_model_reads_a_folder_and_generates(tmp_path):
    folder = models.write_model(str(tmp_path / "m"), "odd", seed=1)
    m = plain.PlainKegozen.from_folder(folder)
    toks = [3, 1, 4, 1, 5, 9, 2, 6, 5, 3, 5, 8, 9, 7]
    full = m.logits(toks)
    assert full.shape == (len(toks), models.ODD["vocab"]) and torch.isfinite(full).all()
    # causal: a prefix's logits do not depend on what follows
    assert float((m.logits(toks[:9]) - full[:9]).abs().max()) < 1e-9
    out = m.greedy_generate(toks[:5], 3)
    assert len(out) == 3 and out[0] == int(torch.argmax(m.logits(toks[:5])[-1]))
