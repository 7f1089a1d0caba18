"""Models of the Kegozen design in the engine against the plain implementation: whole prompts, prefill against
token-by-token decoding, portions down to two tokens, batches of unequal requests with pages and state slots used
again, long decoding past every window and block, keys at a window's and a block's edge that carry the weight, random
configurations, greedy generation through the serving engine and its scheduler, and the trace replay tool.  The
configurations are the tests' own (``kegozen_models``)."""
import json
import os

import numpy as np
import pytest
import torch

import kegozen_models as models
import traces
from plain import kegozen_plain as plain
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
    return folder, plain.PlainKegozen.from_folder(folder), _engine(folder, dtype, pages, PAGE[name], max_live)


def _rows_within(worst_of_rows, mean_of_rows, scale, dtype, what):
    """float32: every row within rounding.  bfloat16: the mean within the bound, and few rows beyond the bound of a
    row (a router whose two best scores lie within bfloat16 rounding of each other may choose the other expert, which
    moves that row; a mechanism that is wrong moves every row)."""
    worst_of_rows, mean = np.asarray(worst_of_rows), float(np.mean(mean_of_rows))
    if dtype == "float32":
        assert worst_of_rows.max() <= F32_TOL * max(1.0, scale), (what, float(worst_of_rows.max()), scale, int(worst_of_rows.argmax()))
        return
    over = int((worst_of_rows > BF16_REL_WORST * scale).sum())
    assert mean <= BF16_REL_MEAN * scale and over <= max(2, len(worst_of_rows) // 20), \
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
        if g.stride == 1:
            assert g.pool.takes - before > g.pool.total          # pages went round
        elif max(LENGTHS[name]) >= g.stride:
            assert g.pool.takes - before > 0                     # the blocks' pages were taken and given back
    assert engine.cache.slots.takes > 4 * 7                       # and so did the state slots


def test_in_float32_every_cut_gives_the_same_logits_within_rounding(tmp_path):
    """A position's logits do not depend on the cut, the batch, the pages or the slots beyond float32 rounding (the
    recurrence, the blocks' means and attention are the same sums whatever the cut; the products of few and of many
    rows are not)."""
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
        assert len(got) == 3
        scale = max(1.0, float(np.abs(got[0]).max()))
        for other in got[1:]:
            assert float(np.abs(other - got[0]).max()) <= 2e-5 * scale, key


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_past_every_window_and_block(tmp_path, dtype):
    """A short prompt and then 300 tokens one by one: the windows of 20 and 33 and the blocks of 4 and 8 pass many
    times, pages of the token caches come back while the blocks' cache grows, the state is carried 300 times."""
    name = "main"
    vocab = models.CONFIGS[name]["vocab"]
    toks = traces.random_tokens(vocab, 310, seed=7)
    folder, ref_model, engine = _setup(tmp_path, name, dtype, pages=44)
    ref = {"long": ref_model.forward(toks).float()}
    steps = traces.last_decoded({"long": toks}, tail=300)
    from zedinfer_amd.engine import StepEntry
    seq = engine.open("held")
    engine.step([StepEntry(seq, toks[:300], [])])
    window_groups = [gi for gi, g in enumerate(engine.cache.groups) if g.kind == "window"]
    assert window_groups and all(seq.held[gi] <= 33 // 8 + 2 for gi in window_groups)      # of 38 pages' worth of tokens
    engine.close(seq)
    out = traces.run_in_process(engine, steps)
    assert _check(steps, out, ref, dtype, "long decoding") == 310
    assert all(engine.cache.groups[gi].pool.takes >= 2 * (310 // 8) for gi in window_groups)
    engine.cache.check()


def _loud_model(tmp_path, window, pool, dtype):
    """One attention layer whose query of every position asks for ONE token: keys are (nearly) the one-hot of the
    token id in the first dims, the query of token 1 points at token 2's key with a large weight.  A prompt of
    token-0 filler with a single token 2 somewhere makes that position carry the weight whenever it is visible."""
    cfg = dict(architecture="Kegozen", width=32, vocab=8, norm=dict(eps=1e-6),
               layers=[dict(type="attention", mixer=dict(heads=1, kv_heads=1, dim=8, vdim=8, scale=1.0,
                                                         mask=dict(size=window, pool=pool)), mlp=None)])
    w = models.make_weights(cfg, seed=3)
    E = torch.zeros((8, 32))
    for t in range(8):
        E[t, t] = 4.0
        E[t, 8 + t] = 1.0
    w["embed"] = E
    for n in ("l0.norm1", "l0.norm1b", "final.norm"):
        w[n] = torch.zeros(32)
    q = torch.zeros((8, 32)); k = torch.zeros((8, 32)); v = torch.zeros((8, 32))
    q[0, 1] = 30.0       # token 1's query: a large value in dim 0
    k[0, 2] = 30.0       # token 2's key: the same
    for t in range(8):
        v[t, t] = 3.0    # the value names the token
    w["l0.mix.q"], w["l0.mix.k"], w["l0.mix.v"] = q, k, v
    w["l0.mix.q.norm"], w["l0.mix.k.norm"] = torch.ones(8), torch.ones(8)
    w["l0.mix.o"] = torch.randn((32, 8), generator=torch.Generator().manual_seed(5))
    folder = models.write_config(str(tmp_path / f"loud_{window}_{pool}"), cfg,
                                 {n: t.to(torch.float32 if dtype == "float32" else torch.bfloat16) for n, t in w.items()})
    return folder, cfg


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_key_just_inside_and_just_outside_the_window_and_a_block_just_seen(tmp_path, dtype):
    """The loud key stands at a chosen distance from the asking token: inside the window it takes the softmax, one
    further it is not seen at all until its block is whole behind the window, then a quarter (1 / pool) of it is;
    in prompts, in portions, and decoded one by one.  The plain implementation and the engine must agree at every
    distance, and the plain logits must differ between the cases (or the test shows nothing)."""
    window, pool = 6, 4
    folder, cfg = _loud_model(tmp_path, window, pool, dtype)
    ref_model = plain.PlainKegozen.from_folder(folder)
    engine = _engine(folder, dtype, pages=64, page=4)
    seen = {}
    for at in (8, 9, 10, 11):                 # where the loud token stands; the asking token comes at the end
        for gap in (window - 1, window, window + 1, window + 2, window + 3, window + 4, window + 5):
            toks = [0] * (at + gap + 1)
            toks[at] = 2
            toks[-1] = 1
            ref = {"p": ref_model.forward(toks).float()}
            for what, steps in (("whole", traces.whole({"p": toks})),
                                ("decoded", traces.last_decoded({"p": toks}, tail=gap + 2)),
                                ("portions", traces.portions({"p": toks}, seed=at + gap, sizes=(2, 3, 5, 2)))):
                out = traces.run_in_process(engine, steps)
                _check(steps, out, ref, dtype, (what, at, gap))
            seen[(at, gap)] = ref["p"][-1]
    # the cases differ: inside the window, hidden, and seen through its block
    inside, hidden = seen[(8, window - 1)], seen[(8, window)]
    assert float((inside - hidden).abs().max()) > 0.5
    through_block = seen[(8, window + 3)]     # block 2 = positions 8..11 ends at 11 <= (8 + 9) - 6
    assert float((through_block - hidden).abs().max()) > 0.05


@pytest.mark.parametrize("seed", range(6))
def test_random_configurations_in_float32(tmp_path, seed):
    cfg = models.random_config(100 + seed)
    folder = models.write_config(str(tmp_path / "m"), cfg, models.make_weights(cfg, seed))
    ref_model = plain.PlainKegozen.from_folder(folder)
    engine = _engine(folder, "float32", pages=80, page=[4, 8, 16][seed % 3])
    requests = {f"q{i}": traces.random_tokens(cfg["vocab"], n, seed=seed * 10 + i) for i, n in enumerate([37, 5, 58, 1])}
    ref = {rid: ref_model.forward(toks).float() for rid, toks in requests.items()}
    for what, steps in (("whole", traces.whole(requests)), ("mixed", traces.mixed(requests, max_live=3, seed=seed)),
                        ("portions", traces.portions(requests, seed=seed, sizes=(2, 9, 1, 4)))):
        out = traces.run_in_process(engine, steps)
        _check(steps, out, ref, "float32", (what, json.dumps(cfg)))
    engine.cache.check()


def test_greedy_generation_through_the_serving_engine(tmp_path):
    """Requests of unequal lengths through ``InferenceEngine`` and its scheduler (prompts cut into portions of 16
    tokens beside decoding requests), more of them than state slots, and the command line: in float32 the tokens are
    the plain implementation's."""
    import subprocess
    import sys
    from zedinfer_amd import GenerationConfig, InferenceEngine, SchedulerConfig
    name = "main"
    folder = models.write_model(str(tmp_path / name), name, seed=2)
    ref_model = plain.PlainKegozen.from_folder(folder)
    vocab = models.CONFIGS[name]["vocab"]
    prompts = [traces.random_tokens(vocab, n, seed=300 + i) for i, n in enumerate([30, 7, 52, 1, 19])]
    want = [ref_model.greedy_generate(p, 12) for p in prompts]
    ie = InferenceEngine.create(folder, "float32", SchedulerConfig(num_kv_blocks=64, kv_block_size=8,
                                                                   max_batch_requests=3, max_prefill_tokens=16))
    got = [r.output_ids for r in ie.generate(prompts, GenerationConfig(max_new_tokens=12, ignore_eos=True))]
    assert got == want
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "ping"), folder, "--dtype", "fp32", "--prompt-ids",
                        ",".join(map(str, prompts[1])), "--max-new-tokens", "6", "--ignore-eos", "--num-kv-blocks", "32",
                        "--kv-block-size", "8", "--no-log-to-console"], capture_output=True, text=True, timeout=600, env=dict(os.environ, PYTHONPATH=root))
    assert r.returncode == 0, r.stderr
    assert "output_ids: " + ",".join(map(str, want[1][:6])) in r.stdout, r.stdout


def test_the_replay_tool_runs_a_model_of_the_design(tmp_path):
    name = "odd"
    folder = models.write_model(str(tmp_path / name), name, seed=4)
    ref_model = plain.PlainKegozen.from_folder(folder)
    vocab = models.CONFIGS[name]["vocab"]
    requests = {f"t{i}": traces.random_tokens(vocab, n, seed=500 + i) for i, n in enumerate([40, 3, 66, 21, 9])}
    ref = {rid: ref_model.forward(toks).float() for rid, toks in requests.items()}
    steps = traces.mixed(requests, max_live=4, seed=11)
    out = traces.run_tool(folder, "float32", steps, str(tmp_path / "out"), traces.max_live_tokens(steps))
    assert _check(steps, out, ref, "float32", "replay tool") == sum(len(t) for t in requests.values())


def test_command_lines_take_a_model_of_the_design(tmp_path):
    """random_model writes a folder from the design's config.json (the engine's own random weights: gains of zero
    around one, zero biases), ping generates from it what the plain implementation generates, batch_bench runs its
    scheduler over it."""
    import subprocess
    import sys
    root = traces.ROOT
    env = dict(os.environ, PYTHONPATH=root)
    run = lambda *a: subprocess.run([sys.executable, *a], capture_output=True, text=True, env=env, timeout=300,  # noqa: E731
                                    cwd=str(tmp_path))
    (tmp_path / "cfg").mkdir()
    with open(tmp_path / "cfg" / "config.json", "w") as f:
        json.dump(models.ODD, f)
    folder = str(tmp_path / "made")
    r = run(os.path.join(root, "bin", "random_model"), str(tmp_path / "cfg"), folder, "--seed", "5", "--dtype", "float32", "--std", "0.1", "--noisy-norms")
    assert r.returncode == 0, r.stderr + r.stdout
    ref_model = plain.PlainKegozen.from_folder(folder)
    assert set(ref_model.w) == set(models.tensor_shapes(models.ODD))
    prompt = traces.random_tokens(models.ODD["vocab"], 27, seed=3)
    r = run(os.path.join(root, "bin", "ping"), folder, "--dtype", "fp32", "--prompt-ids", ",".join(map(str, prompt)),
            "--max-new-tokens", "6", "--ignore-eos", "--num-kv-blocks", "32", "--kv-block-size", "8", "--no-log-to-console")
    assert r.returncode == 0, r.stderr
    want = ref_model.greedy_generate(prompt, 6)
    assert "output_ids: " + ",".join(map(str, want)) in r.stdout, r.stdout
    r = run(os.path.join(root, "bin", "batch_bench"), str(tmp_path / "cfg"), "-b", "3", "-p", "20", "-d", "6", "--num-kv-blocks",
            "64", "--kv-block-size", "8", "--random-weights", "--seed", "4", "--no-log-to-console")
    assert r.returncode == 0 and "18 tokens generated" in r.stdout, r.stderr + r.stdout
