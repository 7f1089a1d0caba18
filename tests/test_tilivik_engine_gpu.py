"""Models of the Tilivik design in the engine against the plain implementation: whole prompts, prefill against
token-by-token decoding, portions down to two tokens, batches of unequal requests with pages and state slots used again, long decoding past every window, a key at a window's edge and among the kept first
positions that carries the weight, greedy generation through the serving engine and its scheduler, the trace replay
tool and the command lines.  The configurations are the tests' own (``tilivik_models``)."""
import json
import os

import numpy as np
import pytest
import torch

import tilivik_models as models
import traces
from plain import tilivik_plain as plain
from tolerances import BF16_REL_MEAN, BF16_REL_WORST, F32_TOL

pytestmark = pytest.mark.gpu

LENGTHS = {"main": [70, 41, 3, 55, 1, 26, 64], "odd": [45, 33, 2, 70, 17], "wide": [38, 9, 61, 1, 24]}
PAGE = {"main": 8, "odd": 4, "wide": 16}


def _engine(folder, dtype, pages, page, max_live=4):
    from zedinfer_amd.config import SchedulerConfig
    from zedinfer_amd.engine import Engine
    return Engine.from_folder(folder, dtype, SchedulerConfig(num_kv_blocks=pages, kv_block_size=page,
                                                             max_batch_requests=max_live, max_batch_tokens=4096,
                                                             max_seq_len=4096))


def _setup(tmp_path, name, dtype, pages, max_live=4, seed=0):
    folder = models.write_model(str(tmp_path / name), name, seed=seed,
                                dtype=torch.float32 if dtype == "float32" else torch.bfloat16)
    return folder, plain.PlainTilivik.from_folder(folder), _engine(folder, dtype, pages, PAGE[name], max_live)


def _rows_within(worst_of_rows, mean_of_rows, scale, dtype, what):
    """float32: every row within rounding.  bfloat16: the mean within the bound, and at most one row in fifty beyond
    the bound of a row (no router chooses here, so no row may be far off: a mechanism that is wrong moves every row)."""
    worst_of_rows, mean = np.asarray(worst_of_rows), float(np.mean(mean_of_rows))
    if dtype == "float32":
        assert worst_of_rows.max() <= F32_TOL * max(1.0, scale), (what, float(worst_of_rows.max()), scale, int(worst_of_rows.argmax()))
        return
    over = int((worst_of_rows > BF16_REL_WORST * scale).sum())
    assert mean <= BF16_REL_MEAN * scale and over <= max(1, len(worst_of_rows) // 50), \
        (what, mean, scale, over, len(worst_of_rows), float(worst_of_rows.max()))


def _check(steps, out, ref, dtype, what):
    """Every written row against the plain logits at (request, position); returns the rows compared."""
    fed, worst, mean, scale = {}, [], [], 0.0
    for st in steps:
        row = 0
        for e in st["entries"]:
            base = fed.get(e["id"], 0)
            for wpos in e["want"]:
                r = ref[e["id"]][base + wpos].numpy()
                d = np.abs(out[st["step"]][row] - r)
                row += 1
                scale = max(scale, float(np.abs(r).max()))
                mean.append(float(d.mean()))
                worst.append(float(d.max()))
            fed[e["id"]] = base + len(e["tokens"])
        for rid in st["end"]:
            fed.pop(rid, None)
    _rows_within(worst, mean, scale, dtype, what)
    return len(mean)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["main", "odd", "wide"])
def test_every_way_of_cutting_and_batching_gives_the_plain_logits(tmp_path, name, dtype):
    vocab = models.CONFIGS[name]["vocab"]
    requests = {f"r{i}": traces.random_tokens(vocab, n, seed=40 + i) for i, n in enumerate(LENGTHS[name])}
    ps = PAGE[name]
    # so few pages that the batches use them again: four live requests of the longest kind, and one page more
    pages = 4 * (-(-max(LENGTHS[name]) // ps) + 1) + 1
    folder, ref_model, engine = _setup(tmp_path, name, dtype, pages)
    ref = {rid: ref_model.forward(toks).float() for rid, toks in requests.items()}
    total = sum(len(t) for t in requests.values())
    takes = [g.pool.takes for g in engine.cache.groups]
    for what, steps in (("whole", traces.whole(requests)), ("decode", traces.last_decoded(requests, tail=30)),
                        ("portions", traces.portions(requests, seed=1)),
                        ("portions of two", traces.portions(requests, seed=2, sizes=(2, 2, 3, 2, 1, 2))),
                        ("mixed", traces.mixed(requests, max_live=4, seed=3)),
                        ("mixed, three live", traces.mixed(requests, max_live=3, seed=4, decode_tail=20, max_portion=9))):
        out = traces.run_in_process(engine, steps)
        assert _check(steps, out, ref, dtype, what) == total
    for what, steps in (("last rows", traces.few_wanted(traces.mixed(requests, max_live=4, seed=5), seed=5)),
                        ("random rows", traces.random_wanted(traces.mixed(requests, max_live=4, seed=6), seed=6))):
        out = traces.run_in_process(engine, steps)
        _check(steps, out, ref, dtype, what)
    engine.cache.check()
    assert not engine.cache.live
    for g, before in zip(engine.cache.groups, takes):
        assert g.pool.takes - before > g.pool.total              # pages went round
    assert engine.cache.slots.takes > 4 * 7                       # and so did the state slots


def test_in_float32_every_cut_gives_the_same_logits_within_rounding(tmp_path):
    """A position's logits do not depend on the cut, the batch, the pages or the slots beyond float32 rounding (the
    recurrences and attention are the same sums whatever the cut; the products of few and of many rows are not)."""
    name = "main"
    vocab = models.CONFIGS[name]["vocab"]
    requests = {f"b{i}": traces.random_tokens(vocab, n, seed=140 + i) for i, n in enumerate([33, 150, 6])}
    folder, ref_model, engine = _setup(tmp_path, name, "float32", pages=96)
    rows = {}
    for what, steps in (("whole", traces.whole(requests)), ("portions", traces.portions(requests, seed=3, sizes=(2, 5, 1, 7))),
                        ("mixed", traces.mixed(requests, max_live=3, seed=9))):
        out = traces.run_in_process(engine, steps)
        fed = {}
        for st in steps:
            row = 0
            for e in st["entries"]:
                base = fed.get(e["id"], 0)
                for wpos in e["want"]:
                    rows.setdefault((e["id"], base + wpos), []).append(out[st["step"]][row].copy())
                    row += 1
                fed[e["id"]] = base + len(e["tokens"])
    assert len(rows) == 33 + 150 + 6
    for key, got in rows.items():
        assert len(got) == 3, key
        scale = max(1.0, float(np.abs(got[0]).max()))
        assert float(np.abs(got[0] - got[1]).max()) <= 2e-5 * scale and float(np.abs(got[0] - got[2]).max()) <= 2e-5 * scale, key


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_request_in_a_slot_that_another_left_starts_from_nothing(tmp_path, dtype):
    """One state slot and few pages: every request runs where the one before it ran, and must not see what it left:
    the matrices of the linear attention, the shifted row of every layer, the token before."""
    name = "main"
    vocab = models.CONFIGS[name]["vocab"]
    requests = {f"s{i}": traces.random_tokens(vocab, n, seed=70 + i) for i, n in enumerate([30, 52, 7, 30])}
    folder, ref_model, engine = _setup(tmp_path, name, dtype, pages=10, max_live=1)
    ref = {rid: ref_model.forward(toks).float() for rid, toks in requests.items()}
    for steps in (traces.whole(requests), traces.portions(requests, seed=7, sizes=(5, 1, 9, 2))):
        out = traces.run_in_process(engine, steps)
        _check(steps, out, ref, dtype, "one slot")
    assert engine.cache.slots.total == 1 and engine.cache.slots.takes == 8


@pytest.mark.parametrize("name, dtype", [("main", "float32"), ("main", "bfloat16"), ("wide", "bfloat16")])
def test_long_decoding_past_every_window(tmp_path, name, dtype):
    """Two requests decode 300 tokens each, one step a token: every window passes over decoded tokens, the pages
    behind it go back (but those of the kept first positions), and the state is carried 300 times."""
    from zedinfer_amd.engine import StepEntry
    vocab = models.CONFIGS[name]["vocab"]
    a, b = traces.random_tokens(vocab, 310, seed=81), traces.random_tokens(vocab, 321, seed=82)
    folder, ref_model, engine = _setup(tmp_path, name, dtype, pages=128)
    ref_a, ref_b = ref_model.forward(a).float(), ref_model.forward(b).float()
    sa, sb = engine.open("a"), engine.open("b")
    out = engine.step([StepEntry(sa, a[:10], [9]), StepEntry(sb, b[:21], [20])])
    worst, mean = [], []
    rows = [(out[0].cpu(), ref_a[9]), (out[1].cpu(), ref_b[20])]
    for i in range(300):
        out = engine.step([StepEntry(sa, [a[10 + i]], [0]), StepEntry(sb, [b[21 + i]], [0])]).cpu()
        rows += [(out[0], ref_a[10 + i]), (out[1], ref_b[21 + i])]
    for row, ref in rows:
        d = (row - ref).abs()
        worst.append(float(d.max()))
        mean.append(float(d.mean()))
    engine.close(sa)
    engine.close(sb)
    _rows_within(worst, mean, max(float(ref_a.abs().max()), float(ref_b.abs().max())), dtype, "long decoding")


# one layer of windowed attention whose softmax is as sharp as the test makes it, beside a linear attention that adds
# nothing, and a head that reads the values out
def _sharp_config(window, keep, cap):
    left = dict(heads=2, kv_heads=1, dim=32, vdim=32, scale=1.0, mask=dict(size=window, keep_first=keep))
    if cap:
        left["softcap"] = cap
    return dict(architecture="Tilivik", width=64, vocab=128, norm=dict(eps=1e-5),
                layers=[dict(type="parallel", mlp=None,
                             mixer=dict(left=left, left_scale=1.0, right=dict(heads=1, dim=8, vdim=8, tau=4.0, rank=2),
                                        right_scale=0.0))])


def _sharp_weights(cfg):
    """Token 5 is the only one with a large first channel; the key's first dim reads that channel, every query's
    first dim reads the last channel, which the sinusoid holds near 1 at every position: the marked key scores about
    20 against at most 5 for the others, and its value is the only one that is large on the dim that the output
    matrix lets through four-fold."""
    w = {k: torch.zeros_like(v) for k, v in models.make_weights(cfg, 0).items()}
    W, V = cfg["width"], cfg["vocab"]
    g = torch.Generator().manual_seed(3)
    w["embed"] = 0.3 * torch.randn(V, W, generator=g)
    w["embed"][:, 0] = 0.0
    w["embed"][:, W - 1] = 0.0
    w["embed"][5, 0] = 6.0                                    # the mark
    w["l0.norm1"], w["final.norm"] = torch.tensor(1.0), torch.tensor(1.0)
    w["l0.mix.right.norm"] = torch.ones(8)
    w["l0.mix.left.k"][0, 0] = 1.0
    w["l0.mix.left.q"][0, W - 1] = 3.0
    w["l0.mix.left.q"][32, W - 1] = 3.0
    w["l0.mix.left.v"][0, 0] = 1.0
    w["l0.mix.left.v"][1, 1:] = 0.3                           # every value has something on dim 1
    w["l0.mix.left.o"][0, 0], w["l0.mix.left.o"][1, 33] = 4.0, 1.0
    w["head"] = 0.2 * torch.randn(V, W, generator=g)
    return w


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("where", ["window_in", "window_out", "kept_in", "kept_out"])
def test_a_marked_key_at_the_edge_of_the_window_and_of_the_kept_positions(tmp_path, dtype, where):
    """700 tokens, a window of 300 and 5 kept positions; the marked token stands just inside or just outside what the
    last prompt token and the decoded tokens see.  Inside, it takes the softmax's weight and shows in the logits; the
    plain logits say which."""
    from zedinfer_amd.engine import StepEntry
    window, keep, T = 300, 5, 700
    cfg = _sharp_config(window, keep, 25.0)
    toks = [t if t != 5 else 6 for t in traces.random_tokens(cfg["vocab"], T + 6, seed=11)]
    # the queries run from position T - 1 (the prompt's last) to T + 5 (decoded)
    at = {"window_in": T + 5 - window + 1, "window_out": T - 1 - window, "kept_in": keep - 1, "kept_out": keep}[where]
    toks[at] = 5
    w = _sharp_weights(cfg)
    folder = models.write_config(str(tmp_path / "sharp"), cfg,
                                 {k: v.to(torch.float32 if dtype == "float32" else torch.bfloat16) for k, v in w.items()})
    ref_model = plain.PlainTilivik.from_folder(folder)
    ref = ref_model.forward(toks).float()
    engine = _engine(folder, dtype, pages=64, page=16)
    seq = engine.open("x")
    out = [engine.step([StepEntry(seq, toks[:T], [T - 40, T - 1])]).cpu()]
    for t in range(T, T + 6):
        out.append(engine.step([StepEntry(seq, [toks[t]], [0])]).cpu())
    engine.close(seq)
    got = torch.cat(out)
    rows = [T - 40, T - 1] + list(range(T, T + 6))
    err = (got.double() - ref[rows].double()).abs()
    scale = float(ref.abs().max())
    if dtype == "float32":
        assert float(err.max()) <= F32_TOL * max(1.0, scale)
    else:
        assert float(err.max()) <= BF16_REL_WORST * scale and float(err.mean()) <= BF16_REL_MEAN * scale
    # the plain model does depend on the marked token where it is seen, and only there
    other = list(toks)
    other[at] = 6
    moved = (ref_model.forward(other).float()[rows] - ref[rows]).abs().amax(dim=1)
    if where == "window_in":
        assert float(moved.min()) > 0.08 * scale
    elif where == "window_out":
        assert float(moved[1:].max()) < 1e-3 * scale and float(moved[0]) > 0.08 * scale      # T - 40 still sees it
    elif where == "kept_in":
        assert float(moved.min()) > 0.08 * scale
    else:
        assert float(moved.max()) < 1e-3 * scale


# models of one kind of layer only: no pages at all (nothing but state), and nothing but pages and state of one layer
ONLY_LINEAR = dict(
    architecture="Tilivik", width=64, vocab=90, norm=dict(eps=1e-6), loop=dict(start=0, stop=2, times=2),
    layers=[dict(type="lightning", mixer=dict(heads=2, dim=16, vdim=32, decay=[0.9, 1.0]), mlp=None),
            dict(type="lightning", mixer=dict(heads=4, dim=8, vdim=16, decay=[0.5, 0.7, 0.9, 0.99]),
                 mlp=dict(kind="moe", expert=dict(ff=24), router=dict(experts=3, top=1)))])
ONLY_SOFTMAX = dict(
    architecture="Tilivik", width=64, vocab=90, norm=dict(eps=1e-6), embedding=dict(bigram=dict(buckets=2, mul_prev=1, mul_cur=2)),
    layers=[dict(type="parallel", mlp=None,
                 mixer=dict(left=dict(heads=2, kv_heads=2, dim=32, vdim=32, scale=0.2), left_scale=1.0,
                            right=dict(heads=1, dim=8, vdim=8, tau=2.0, rank=1), right_scale=1.0))])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["only_linear", "only_softmax"])
def test_models_of_one_kind_of_layer(tmp_path, which, dtype):
    cfg = ONLY_LINEAR if which == "only_linear" else ONLY_SOFTMAX
    requests = {f"o{i}": traces.random_tokens(cfg["vocab"], n, seed=30 + i) for i, n in enumerate([50, 3, 77, 20, 9])}
    folder = models.write_config(str(tmp_path / which), cfg,
                                 models.make_weights(cfg, 6, torch.float32 if dtype == "float32" else torch.bfloat16))
    ref_model = plain.PlainTilivik.from_folder(folder)
    ref = {rid: ref_model.forward(toks).float() for rid, toks in requests.items()}
    engine = _engine(folder, dtype, pages=40, page=8, max_live=3)
    assert len(engine.cache.groups) == (0 if which == "only_linear" else 1)
    for what, steps in (("mixed", traces.mixed(requests, max_live=3, seed=2)), ("whole", traces.whole(requests)),
                        ("portions", traces.portions(requests, seed=5, sizes=(2, 9, 1, 4)))):
        out = traces.run_in_process(engine, steps)
        _check(steps, out, ref, dtype, (which, what))


LONG = dict(
    architecture="Tilivik", width=128, vocab=180, norm=dict(eps=1e-6),
    embedding=dict(bigram=dict(buckets=251, mul_prev=5, mul_cur=3)),
    layers=[dict(type="parallel", mlp=dict(kind="moe", expert=dict(ff=32), router=dict(experts=4, top=2)),
                 mixer=dict(left=dict(heads=4, kv_heads=2, dim=64, vdim=64, scale=0.125, softcap=12.0, bias_max=3000, bias_rows=16,
                                      mask=dict(size=2200, keep_first=3)),
                            left_scale=0.9, right=dict(heads=2, dim=16, vdim=32, tau=32.0, rank=4), right_scale=0.8))])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_whose_keys_are_cut_over_workgroups(tmp_path, dtype):
    """2,300 tokens under a window of 2,200 in two portions and a few decoded tokens: tiles whose keys are cut over
    several workgroups and merged, tokens whose keys are more than one chunk, the window passing the kept positions."""
    from zedinfer_amd.engine import StepEntry
    cfg = LONG
    T = 2300
    toks = traces.random_tokens(cfg["vocab"], T, seed=4)
    folder = models.write_config(str(tmp_path / "long"), cfg,
                                 models.make_weights(cfg, 2, torch.float32 if dtype == "float32" else torch.bfloat16))
    ref = plain.PlainTilivik.from_folder(folder).forward(toks).float()
    engine = _engine(folder, dtype, pages=160, page=16)
    seq = engine.open("x")
    rows = [5, 900, 999]
    out = [engine.step([StepEntry(seq, toks[:1000], rows)]).cpu()]
    more = [0, 1100, 1202, 1203, 1289]                      # positions 1000 .. 2289
    out.append(engine.step([StepEntry(seq, toks[1000:2290], more)]).cpu())
    rows += [1000 + m for m in more]
    for t in range(2290, T):
        out.append(engine.step([StepEntry(seq, [toks[t]], [0])]).cpu())
        rows.append(t)
    engine.close(seq)
    err = (torch.cat(out).double() - ref[rows].double()).abs()
    _rows_within(err.amax(dim=1).numpy(), err.mean(dim=1).numpy(), float(ref.abs().max()), dtype, "long prompt")


@pytest.mark.parametrize("name", ["main", "odd"])
def test_greedy_generation_through_the_serving_engine(tmp_path, name):
    """Several requests at once through InferenceEngine (its scheduler cuts the prompts into portions of 16 tokens and
    batches them beside decoding requests): in float32 the tokens are the plain implementation's."""
    from zedinfer_amd import GenerationConfig, InferenceEngine, SchedulerConfig
    folder = models.write_model(str(tmp_path / name), name, seed=9)
    ref_model = plain.PlainTilivik.from_folder(folder)
    vocab = models.CONFIGS[name]["vocab"]
    prompts = [traces.random_tokens(vocab, n, seed=90 + n) for n in (37, 5, 21, 50)]
    want = [ref_model.greedy_generate(p, 12) for p in prompts]
    ie = InferenceEngine.create(folder, "float32", SchedulerConfig(num_kv_blocks=64, kv_block_size=PAGE[name],
                                                                   max_batch_requests=3, max_prefill_tokens=16))
    got = [r.output_ids for r in ie.generate(prompts, GenerationConfig(max_new_tokens=12, ignore_eos=True))]
    assert got == want
    alone = ie.generate_tokens(prompts[0], GenerationConfig(max_new_tokens=12, ignore_eos=True)).output_ids
    assert alone == want[0]


def test_the_replay_tool_runs_a_model_of_the_design(tmp_path):
    name = "main"
    folder = models.write_model(str(tmp_path / name), name, seed=3, dtype=torch.bfloat16)
    ref_model = plain.PlainTilivik.from_folder(folder)
    requests = {f"q{i}": traces.random_tokens(models.CONFIGS[name]["vocab"], n, seed=20 + i)
                for i, n in enumerate([66, 19, 130, 4, 40])}
    ref = {rid: ref_model.forward(toks).float() for rid, toks in requests.items()}
    steps = traces.mixed(requests, max_live=4, seed=8)
    for dtype in ("float32", "bfloat16"):
        out = traces.run_tool(folder, dtype, steps, str(tmp_path / f"out_{dtype}"), traces.max_live_tokens(steps),
                              stderr_to=str(tmp_path / f"err_{dtype}.txt"))
        _check(steps, out, ref, dtype, "tool")
        said = open(str(tmp_path / f"err_{dtype}.txt")).read()
        assert "4 live requests" in said


def test_command_lines_take_a_model_of_the_design(tmp_path):
    """random_model writes a folder from the design's config.json, ping generates from it what the plain implementation
    generates, batch_bench runs its scheduler over it with random weights."""
    import subprocess
    import sys
    ROOT = traces.ROOT
    env = dict(os.environ, PYTHONPATH=ROOT)
    run = lambda *a: subprocess.run([sys.executable, *a], capture_output=True, text=True, env=env, timeout=300,  # noqa: E731
                                    cwd=str(tmp_path))
    (tmp_path / "cfg").mkdir()
    with open(tmp_path / "cfg" / "config.json", "w") as f:
        json.dump(models.MAIN, f)
    folder = str(tmp_path / "made")
    r = run(os.path.join(ROOT, "bin", "random_model"), str(tmp_path / "cfg"), folder, "--seed", "5", "--dtype", "float32",
            "--std", "0.1", "--noisy-norms")
    assert r.returncode == 0 and "Tilivik" in r.stdout, r.stderr
    with open(os.path.join(folder, "config.json")) as f:
        assert json.load(f) == models.MAIN
    ref_model = plain.PlainTilivik.from_folder(folder)
    assert set(ref_model.t) == set(models.tensor_shapes(models.MAIN))
    prompt = traces.random_tokens(models.MAIN["vocab"], 27, seed=3)
    r = run(os.path.join(ROOT, "bin", "ping"), folder, "--dtype", "fp32", "--prompt-ids", ",".join(map(str, prompt)),
            "--max-new-tokens", "6", "--ignore-eos", "--num-kv-blocks", "32", "--kv-block-size", "8", "--no-log-to-console")
    assert r.returncode == 0, r.stderr
    want = ref_model.greedy_generate(prompt, 6)
    assert "output_ids: " + ",".join(map(str, want)) in r.stdout, r.stdout
    r = run(os.path.join(ROOT, "bin", "batch_bench"), str(tmp_path / "cfg"), "-b", "3", "-p", "20", "-d", "6", "--num-kv-blocks",
            "64", "--kv-block-size", "8", "--random-weights", "--seed", "4", "--no-log-to-console")
    assert r.returncode == 0 and "18 tokens generated" in r.stdout, r.stderr + r.stdout


@pytest.mark.parametrize("seed", range(10))
def test_configurations_drawn_at_random(tmp_path, seed):
    """Ten models whose sizes, layer order, repeated run and constants are drawn at random, each in both engine types,
    over a batch of unequal requests with pages and slots used again and over whole prompts."""
    cfg = models.random_config(seed)
    requests = {f"z{i}": traces.random_tokens(cfg["vocab"], n, seed=seed * 10 + i) for i, n in enumerate([83, 5, 140, 31, 1, 66])}
    for dtype in ("float32", "bfloat16"):
        folder = models.write_config(str(tmp_path / dtype), cfg,
                                     models.make_weights(cfg, seed, torch.float32 if dtype == "float32" else torch.bfloat16))
        ref_model = plain.PlainTilivik.from_folder(folder)
        ref = {rid: ref_model.forward(toks).float() for rid, toks in requests.items()}
        ps = [4, 8, 16, 32][seed % 4]
        engine = _engine(folder, dtype, 3 * (-(-140 // ps) + 3) + 6, ps, max_live=3)
        for what, steps in (("mixed", traces.mixed(requests, max_live=3, seed=seed, decode_tail=25, max_portion=40)),
                            ("whole", traces.whole(requests))):
            out = traces.run_in_process(engine, steps)
            _check(steps, out, ref, dtype, (what, seed, json.dumps(cfg)))
