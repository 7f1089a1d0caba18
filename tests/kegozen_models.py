"""Small Kegozen configurations of the tests and their random weights.

The sizes differ from layer to layer and between the configurations in everything the format lets differ: query heads
against key/value heads (equal, 2, 4 and 12 to 1), dim against vdim (smaller, larger, equal), rotated dims that are a
part of the head or all of it, stretched frequencies or plain ones, windows shorter and longer than the prompts and
than a block, blocks longer than the window, blocks of one position's worth of pages and of many, no window at all;
state-space layers with one group, several, and a group a head, 2 to 4 taps, states that are no multiple of 8, one
norm part and a part a head; latent attention with and without a latent for the queries, ranks that are no multiple
of 8; dense feed-forwards, mixtures with one to four experts chosen, with and without a shared expert, layers without
a feed-forward; widths that are no multiple of 8.

Weights are drawn here (not by the engine's random-weights mode): gains around zero, decays from slow to fast, steps
of both signs before the softplus, routers wide enough that few choices are close."""
import json
import math
import os

import torch


def _attn(heads, kv_heads, dim, vdim, rot=None, scaling=None, mask=None, scale=None):
    d = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale or 1.0 / math.sqrt(dim))
    if rot is not None:
        d["rot"] = dict(base=rot[0], dims=rot[1])
        if scaling is not None:
            d["rot"]["scaling"] = dict(factor=scaling[0], original=scaling[1], fast=scaling[2], slow=scaling[3])
    if mask is not None:
        d["mask"] = dict(size=mask[0], pool=mask[1])
    return d


def _latent(heads, dim, rot_dim, vdim, kv_rank, q_rank=None, base=10000.0, scale=None):
    d = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, rot=dict(base=base, dims=rot_dim),
             scale=scale or 1.0 / math.sqrt(dim + rot_dim))
    if q_rank:
        d["q_rank"] = q_rank
    return d


def _ssm(heads, vdim, state, groups, conv, norm_groups):
    return dict(heads=heads, vdim=vdim, state=state, groups=groups, conv=conv, norm_groups=norm_groups)


def _moe(experts, top, ff, shared=None):
    d = dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top))
    if shared:
        d["shared"] = dict(ff=shared)
    return d


def _dense(ff):
    return dict(kind="dense", ff=ff)


MAIN = dict(
    architecture="Kegozen", width=96, vocab=211, norm=dict(eps=3e-6),
    layers=[
        dict(type="attention", mixer=_attn(4, 2, 32, 16, rot=(5000.0, 16), scaling=(8.0, 64, 16.0, 2.0), mask=(20, 4)),
             mlp=_moe(5, 2, 40, shared=24)),
        dict(type="mamba2", mixer=_ssm(4, 16, 16, 2, 4, 2), mlp=_dense(64)),
        dict(type="latent_attention", mixer=_latent(3, 16, 8, 24, 24, q_rank=40), mlp=None),
        dict(type="attention", mixer=_attn(3, 3, 24, 24, rot=(300.0, 24), mask=(33, 8)), mlp=_moe(6, 4, 24)),
        dict(type="mamba2", mixer=_ssm(3, 24, 8, 1, 3, 1), mlp=_moe(3, 1, 56, shared=16)),
    ])

# a width that is no multiple of 8, a block longer than the window, a window of one, sizes no matrix-core kernel takes
ODD = dict(
    architecture="Kegozen", width=84, vocab=150, norm=dict(eps=1e-5),
    layers=[
        dict(type="mamba2", mixer=_ssm(5, 20, 12, 5, 2, 5), mlp=_moe(4, 3, 36, shared=20)),
        dict(type="attention", mixer=_attn(5, 5, 20, 12, rot=(100.0, 10), scaling=(2.0, 16, 4.0, 1.0), mask=(5, 7)), mlp=None),
        dict(type="latent_attention", mixer=_latent(2, 12, 6, 20, 20), mlp=_dense(50)),
        dict(type="attention", mixer=_attn(2, 1, 8, 72, mask=(1, 3)), mlp=_moe(2, 2, 20)),
        dict(type="latent_attention", mixer=_latent(5, 8, 4, 8, 12, q_rank=12, base=50.0), mlp=_moe(7, 1, 16)),
    ])

# heads of 128, many query heads a key/value head, a window longer than every prompt, no window, a state of 128
WIDE = dict(
    architecture="Kegozen", width=128, vocab=200, norm=dict(eps=1e-6),
    layers=[
        dict(type="attention", mixer=_attn(2, 1, 128, 96, rot=(1e6, 64), scaling=(4.0, 32, 8.0, 1.0), mask=(500, 64)),
             mlp=_moe(8, 2, 32, shared=64)),
        dict(type="mamba2", mixer=_ssm(2, 64, 128, 1, 4, 1), mlp=_dense(96)),
        dict(type="attention", mixer=_attn(12, 1, 16, 16, rot=(10000.0, 16), mask=(16, 16)), mlp=None),
        dict(type="latent_attention", mixer=_latent(2, 128, 64, 128, 64, q_rank=96, base=250000.0), mlp=_moe(4, 1, 48)),
        dict(type="attention", mixer=_attn(4, 2, 32, 32, rot=(20000.0, 32)), mlp=_dense(64)),
    ])

CONFIGS = {"main": MAIN, "odd": ODD, "wide": WIDE}


def tensor_shapes(cfg):
    """name -> shape of every tensor a model of ``cfg`` has."""
    W, V, out = cfg["width"], cfg["vocab"], {}
    out["embed"] = (V, W)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"], out[p + "norm1b"] = (W,), (W,)
        if layer["type"] == "mamba2":
            inner, gn = m["heads"] * m["vdim"], m["groups"] * m["state"]
            out.update({p + "mix.in": (2 * inner + 2 * gn + m["heads"], W), p + "mix.conv": (inner + 2 * gn, m["conv"]),
                        p + "mix.conv.b": (inner + 2 * gn,), p + "mix.dt_bias": (m["heads"],), p + "mix.A_log": (m["heads"],),
                        p + "mix.D": (m["heads"],), p + "mix.norm": (inner,), p + "mix.o": (W, inner)})
        elif layer["type"] == "attention":
            out.update({p + "mix.q": (m["heads"] * m["dim"], W), p + "mix.k": (m["kv_heads"] * m["dim"], W),
                        p + "mix.v": (m["kv_heads"] * m["vdim"], W), p + "mix.q.norm": (m["dim"],),
                        p + "mix.k.norm": (m["dim"],), p + "mix.o": (W, m["heads"] * m["vdim"])})
        else:
            hd = m["heads"] * (m["dim"] + m["rot_dim"])
            if m.get("q_rank"):
                out.update({p + "mix.dq": (m["q_rank"], W), p + "mix.dq.norm": (m["q_rank"],), p + "mix.uq": (hd, m["q_rank"])})
            else:
                out[p + "mix.q"] = (hd, W)
            out.update({p + "mix.dkv": (m["kv_rank"] + m["rot_dim"], W), p + "mix.dkv.norm": (m["kv_rank"],),
                        p + "mix.uk": (m["heads"] * m["dim"], m["kv_rank"]), p + "mix.uv": (m["heads"] * m["vdim"], m["kv_rank"]),
                        p + "mix.o": (W, m["heads"] * m["vdim"])})
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        out[p + "norm2"], out[p + "norm2b"] = (W,), (W,)
        if mlp["kind"] == "dense":
            out.update({p + "mlp.gate": (mlp["ff"], W), p + "mlp.up": (mlp["ff"], W), p + "mlp.down": (W, mlp["ff"])})
            continue
        E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
        for e in range(E):
            out.update({f"{p}mlp.e{e}.gate": (ff, W), f"{p}mlp.e{e}.up": (ff, W), f"{p}mlp.e{e}.down": (W, ff)})
        out[p + "mlp.router"] = (E, W)
        if mlp.get("shared"):
            sf = mlp["shared"]["ff"]
            out.update({p + "mlp.shared.gate": (sf, W), p + "mlp.shared.up": (sf, W), p + "mlp.shared.down": (W, sf),
                        p + "mlp.shared.sg": (1, W)})
    out["final.norm"], out["head"] = (W,), (V, W)
    return out


def make_weights(cfg, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg).items():
        parts = name.split(".")
        last = parts[-1]
        if last in ("norm1", "norm1b", "norm2", "norm2b") or name == "final.norm":
            t = 0.3 * torch.randn(shape, generator=g)                      # the stored gain is the distance from one
        elif last == "norm":
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif last == "A_log":
            t = torch.log(0.2 + 3.0 * torch.rand(shape, generator=g))        # decays from slow to fast
        elif last == "dt_bias":
            t = torch.randn(shape, generator=g) - 1.0
        elif last == "D":
            t = 1.0 + 0.5 * torch.randn(shape, generator=g)
        elif last == "conv":
            t = 0.5 * torch.randn(shape, generator=g)
        elif last == "b":
            t = 0.2 * torch.randn(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        elif last == "router":
            t = torch.randn(shape, generator=g) * (2.0 / shape[-1] ** 0.5)
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
    """A configuration drawn at random: sizes, head counts, the order of layers, windows and blocks, rotated dims,
    stretched frequencies, taps, groups, ranks, experts and how many are chosen, shared experts, eps."""
    import random
    rng = random.Random(seed)
    width = rng.choice([48, 64, 72, 96, 128, 160])
    cfg = dict(architecture="Kegozen", width=width, vocab=rng.choice([97, 256, 411]),
               norm=dict(eps=rng.choice([1e-6, 1e-5, 3e-6])), layers=[])
    for i in range(rng.randint(2, 5)):
        r = rng.random()
        if r < 0.15:
            mlp = None
        elif r < 0.4:
            mlp = _dense(rng.choice([24, 40, 96]))
        else:
            e = rng.choice([2, 4, 7, 16])
            mlp = _moe(e, rng.randint(1, min(e, 4)), rng.choice([16, 40, 72]), shared=rng.choice([None, 16, 48]))
        kind = rng.choice(["mamba2", "attention", "latent_attention"])
        if kind == "mamba2":
            groups = rng.choice([1, 2, 3])
            heads = groups * rng.choice([1, 2, 4])
            vdim = rng.choice([8, 16, 24, 40, 64])
            parts = rng.choice([p for p in (1, 2, heads) if (heads * vdim) % p == 0])
            mixer = _ssm(heads, vdim, rng.choice([8, 16, 24, 64]), groups, rng.choice([2, 3, 4]), parts)
        elif kind == "attention":
            kvh = rng.choice([1, 2, 3])
            dim = rng.choice([8, 16, 24, 32, 48, 64, 96])
            rot = rng.choice([None, (rng.choice([100.0, 10000.0, 5e5]), rng.choice([d for d in (4, 8, 16, dim) if d <= dim]))])
            scaling = rng.choice([None, (rng.choice([2.0, 4.0, 16.0]), rng.choice([16, 64, 512]), rng.choice([8.0, 32.0]), rng.choice([1.0, 2.0]))])
            mask = rng.choice([None, (5, 2), (12, 4), (30, 7), (16, 16), (7, 16), (200, 8), (24, 0)])
            mixer = _attn(kvh * rng.choice([1, 2, 4]), kvh, dim, rng.choice([8, 16, 24, 40, 64]), rot=rot,
                          scaling=scaling if rot else None, mask=mask)
        else:
            dim, rot = rng.choice([8, 16, 32, 64]), rng.choice([4, 8, 16, 32])
            mixer = _latent(rng.choice([1, 2, 3, 4]), dim, rot, rng.choice([8, 16, 40, 64]), rng.choice([8, 12, 32, 64]),
                            q_rank=rng.choice([None, 8, 24, 48]), base=rng.choice([100.0, 10000.0, 250000.0]))
        cfg["layers"].append(dict(type=kind, mixer=mixer, mlp=mlp))
    return cfg
