"""Small Tilivik configurations of the tests and their random weights.

The sizes differ from layer to layer and between the configurations in everything the format lets differ: query heads
against key/value heads (equal, 2, 3 and 4 to 1), dim against vdim (smaller, larger, equal) in every mixer, windows
shorter and longer than the prompts, with and without kept first positions, no window at all, bias tables of few and
many rows with a far distance inside and outside the window, no bias, no cap, repeated runs of layers that start at
the first layer or later and run two or three times, no repetition, no pair table, layers without a feed-forward, one
expert of three and four of five, widths that are no multiple of 8.

Weights are drawn here (not by the engine's random-weights mode): gains away from 1, shifts of both signs, decay
gates of both signs, bias rows large enough to matter."""
import json
import os

import torch


def _left(heads, kv_heads, dim, vdim, scale, softcap=None, bias_max=None, bias_rows=None, mask=None):
    d = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if softcap is not None:
        d["softcap"] = softcap
    if bias_max is not None:
        d.update(bias_max=bias_max, bias_rows=bias_rows)
    if mask is not None:
        d["mask"] = dict(size=mask[0], keep_first=mask[1])
    return d


def _moe(experts, top, ff):
    return dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top))


MAIN = dict(
    architecture="Tilivik", width=96, vocab=211, norm=dict(eps=3e-6),
    embedding=dict(bigram=dict(buckets=97, mul_prev=13, mul_cur=7)),
    loop=dict(start=1, stop=3, times=3),
    layers=[
        dict(type="parallel",
             mixer=dict(left=_left(4, 2, 32, 16, 0.2, softcap=8.0, bias_max=40, bias_rows=12, mask=(20, 3)), left_scale=0.7,
                        right=dict(heads=3, dim=16, vdim=24, tau=8.0, rank=8), right_scale=1.3),
             mlp=_moe(5, 2, 40)),
        dict(type="lightning", mixer=dict(heads=3, dim=16, vdim=40, decay=[0.5, 0.93, 0.999]), mlp=_moe(6, 4, 24)),
        dict(type="parallel",
             mixer=dict(left=_left(6, 2, 16, 48, 0.3, softcap=20.0, bias_max=300, bias_rows=20, mask=(33, 0)), left_scale=1.0,
                        right=dict(heads=1, dim=48, vdim=16, tau=4.0, rank=5), right_scale=0.4),
             mlp=None),
        dict(type="lightning", mixer=dict(heads=2, dim=40, vdim=24, decay=[0.8, 0.99]), mlp=_moe(3, 1, 56)),
        dict(type="parallel",
             mixer=dict(left=_left(3, 3, 24, 24, 0.25, bias_max=64, bias_rows=8), left_scale=0.5,
                        right=dict(heads=2, dim=32, vdim=32, tau=16.0, rank=12), right_scale=0.9),
             mlp=_moe(5, 4, 16)),
    ])

# a width that is no multiple of 8, heads that no matrix-core kernel takes as they are, no pair table, no repetition,
# a window without bias and a bias without window
ODD = dict(
    architecture="Tilivik", width=84, vocab=150, norm=dict(eps=1e-5),
    layers=[
        dict(type="parallel",
             mixer=dict(left=_left(5, 5, 20, 12, 0.3, softcap=5.0, mask=(9, 4)), left_scale=1.1,
                        right=dict(heads=2, dim=12, vdim=20, tau=3.0, rank=3), right_scale=0.6),
             mlp=_moe(3, 3, 36)),
        dict(type="lightning", mixer=dict(heads=5, dim=12, vdim=12, decay=[0.3, 0.6, 0.9, 0.97, 1.0]), mlp=None),
        dict(type="parallel",
             mixer=dict(left=_left(2, 1, 8, 72, 0.5, bias_max=17, bias_rows=7), left_scale=0.8,
                        right=dict(heads=3, dim=20, vdim=8, tau=1.0, rank=16), right_scale=1.0),
             mlp=_moe(4, 2, 20)),
    ])

# heads of 128 and of more than any matrix-core kernel takes, many query heads a key/value head, a run of layers that
# starts at the first layer and runs twice, a window longer than every prompt of the tests
WIDE = dict(
    architecture="Tilivik", width=128, vocab=200, norm=dict(eps=1e-6),
    embedding=dict(bigram=dict(buckets=61, mul_prev=1, mul_cur=1)),
    loop=dict(start=0, stop=2, times=2),
    layers=[
        dict(type="parallel",
             mixer=dict(left=_left(2, 1, 128, 96, 0.09, softcap=50.0, bias_max=1000, bias_rows=32, mask=(500, 2)), left_scale=1.0,
                        right=dict(heads=1, dim=128, vdim=64, tau=32.0, rank=4), right_scale=1.0),
             mlp=_moe(8, 2, 32)),
        dict(type="lightning", mixer=dict(heads=1, dim=144, vdim=136, decay=[0.97]), mlp=_moe(2, 2, 64)),
        dict(type="parallel",
             mixer=dict(left=_left(12, 1, 16, 16, 0.25, softcap=2.0, bias_max=24, bias_rows=16, mask=(16, 1)), left_scale=0.3,
                        right=dict(heads=8, dim=8, vdim=8, tau=2.0, rank=2), right_scale=2.0),
             mlp=None),
        dict(type="parallel",
             mixer=dict(left=_left(1, 1, 144, 40, 0.08, bias_max=50, bias_rows=4, mask=(64, 16)), left_scale=1.0,
                        right=dict(heads=2, dim=64, vdim=128, tau=8.0, rank=32), right_scale=0.5),
             mlp=_moe(4, 1, 48)),
    ])

CONFIGS = {"main": MAIN, "odd": ODD, "wide": WIDE}


def run_order(cfg):
    """The layers in the order they run."""
    L, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return list(range(L))
    a, b = loop["start"], loop["stop"]
    return list(range(a)) + list(range(a, b)) * loop["times"] + list(range(b, L))


def tensor_shapes(cfg):
    """name -> shape of every tensor a model of ``cfg`` has."""
    W, V, out = cfg["width"], cfg["vocab"], {}
    out["embed"] = (V, W)
    bi = (cfg.get("embedding") or {}).get("bigram")
    if bi:
        out["bigram"] = (bi["buckets"] + 1, W)
    if cfg.get("loop"):
        out["loop.step"] = (cfg["loop"]["times"], W)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"], out[p + "shift"] = (), (W,)
        if layer["type"] == "lightning":
            qk, vd = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            out.update({p + "mix.q": (qk, W), p + "mix.k": (qk, W), p + "mix.v": (vd, W), p + "mix.g": (vd, W),
                        p + "mix.o": (W, vd), p + "mix.norm": (vd,)})
        else:
            le, ri = m["left"], m["right"]
            out.update({p + "mix.left.q": (le["heads"] * le["dim"], W), p + "mix.left.k": (le["kv_heads"] * le["dim"], W),
                        p + "mix.left.v": (le["kv_heads"] * le["vdim"], W), p + "mix.left.g": (le["heads"] * le["vdim"], W),
                        p + "mix.left.o": (W, le["heads"] * le["vdim"])})
            if le.get("bias_max") is not None:
                out[p + "mix.left.rel"] = (le["bias_rows"], le["heads"])
            qk, vd = ri["heads"] * ri["dim"], ri["heads"] * ri["vdim"]
            out.update({p + "mix.right.q": (qk, W), p + "mix.right.k": (qk, W), p + "mix.right.v": (vd, W),
                        p + "mix.right.g": (vd, W), p + "mix.right.o": (W, vd), p + "mix.right.norm": (ri["vdim"],),
                        p + "mix.right.a1": (ri["rank"], W), p + "mix.right.a2": (qk, ri["rank"]), p + "mix.right.a2.b": (qk,)})
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        out[p + "norm2"] = ()
        E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
        for e in range(E):
            out.update({f"{p}mlp.e{e}.gate": (ff, W), f"{p}mlp.e{e}.up": (ff, W), f"{p}mlp.e{e}.down": (W, ff)})
        out[p + "mlp.table"] = (V, mlp["router"]["top"])
    out["final.norm"], out["head"] = (), (V, W)
    return out


def make_weights(cfg, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg).items():
        parts = name.split(".")
        last = parts[-1]
        if last == "table":
            layer = cfg["layers"][int(parts[0][1:])]
            E = layer["mlp"]["router"]["experts"]
            w[name] = torch.rand((shape[0], E), generator=g).argsort(dim=1)[:, :shape[1]].to(torch.int32).contiguous()
            continue
        if last in ("norm1", "norm2") or name == "final.norm":
            t = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif last == "norm":
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif last == "shift":
            t = 0.5 * torch.randn(shape, generator=g)
        elif last == "rel":
            t = 1.5 * torch.randn(shape, generator=g)
        elif last == "b":
            t = 1.0 + 2.0 * torch.randn(shape, generator=g)     # decay gates from almost closed to almost open
        elif name in ("embed", "bigram"):
            t = torch.randn(shape, generator=g)
        elif name == "loop.step":
            t = 0.5 * torch.randn(shape, generator=g)
        elif last == "a2":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) * (1.0 / shape[-1] ** 0.5)
        w[name] = t.to(dtype)
    return w


def write_config(folder, cfg, weights):
    from zedinfer_amd.weights.safetensors_io import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    write_safetensors(os.path.join(folder, "model.safetensors"), weights, metadata={"format": "pt"})
    return folder


def write_model(folder, name, seed=0, dtype=torch.float32):
    """config.json and model.safetensors of configuration ``name``; returns the folder."""
    return write_config(folder, CONFIGS[name], make_weights(CONFIGS[name], seed, dtype))


def random_config(seed):
    """A configuration drawn at random: sizes, head counts, the order of layers, the repeated run, windows, kept
    positions, caps, bias tables, scales, decays, experts and how many are chosen, the pair table's hash, eps."""
    import random
    rng = random.Random(seed)
    width = rng.choice([48, 64, 72, 96, 128, 160])
    cfg = dict(architecture="Tilivik", width=width, vocab=rng.choice([97, 256, 411]),
               norm=dict(eps=rng.choice([1e-6, 1e-5, 3e-6])), layers=[])
    if rng.random() < 0.75:
        cfg["embedding"] = dict(bigram=dict(buckets=rng.choice([7, 101, 509]), mul_prev=rng.choice([1, 3, 29, 1009]),
                                            mul_cur=rng.choice([1, 5, 19])))
    n_layers = rng.randint(2, 5)
    for i in range(n_layers):
        r = rng.random()
        mlp = None if r < 0.2 else _moe(*(lambda e: (e, rng.randint(1, min(e, 4)), rng.choice([16, 40, 72])))(rng.choice([2, 4, 7, 16])))
        if rng.random() < 0.4:
            heads = rng.choice([1, 2, 3, 4])
            mixer = dict(heads=heads, dim=rng.choice([8, 16, 24, 32, 64]), vdim=rng.choice([8, 16, 40, 64]),
                         decay=[rng.choice([0.4, 0.8, 0.95, 0.99, 0.999]) for _ in range(heads)])
            cfg["layers"].append(dict(type="lightning", mixer=mixer, mlp=mlp))
            continue
        kvh = rng.choice([1, 2, 3])
        dim = rng.choice([8, 16, 24, 32, 48, 64, 96])
        left = _left(kvh * rng.choice([1, 2, 4]), kvh, dim, rng.choice([8, 16, 24, 40, 64]),
                     rng.choice([0.05, 0.1, 0.2]) * (32.0 / dim) ** 0.5,
                     softcap=rng.choice([None, 3.0, 15.0, 30.0]),
                     bias_max=rng.choice([None, 10, 50, 128]), bias_rows=rng.choice([2, 6, 16, 32]),
                     mask=rng.choice([None, (5, 0), (12, 2), (30, 7), (64, 64), (200, 1)]))
        right = dict(heads=rng.choice([1, 2, 4]), dim=rng.choice([8, 16, 32, 64]), vdim=rng.choice([8, 16, 32, 64]),
                     tau=rng.choice([1.0, 4.0, 16.0]), rank=rng.choice([1, 4, 16]))
        cfg["layers"].append(dict(type="parallel", mlp=mlp,
                                  mixer=dict(left=left, right=right, left_scale=rng.choice([0.5, 1.0, 1.5]),
                                             right_scale=rng.choice([0.3, 1.0, 1.2]))))
    if rng.random() < 0.7:
        a = rng.randint(0, n_layers - 1)
        cfg["loop"] = dict(start=a, stop=rng.randint(a + 1, n_layers), times=rng.randint(1, 3))
    return cfg
