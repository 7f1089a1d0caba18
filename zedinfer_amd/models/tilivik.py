"""Tilivik: the description of the design in parts.

A decoder whose layers are listed one by one in config.json.  The embedding sums the token's row, a row of a second
table looked up by a hash of the token and the one before it, and a fixed sinusoid of the position.  A layer is
x <- x + mixer(shift(n1(x))), x <- x + ff(n2(x)) with RMS norms whose gain is one number, and a token shift (a learned
mix of every channel with the token before) in front of the mixer.  The mixer is linear attention with a fixed decay
per head ("lightning"), or windowed softmax attention (no rotation; capped scores, a bias by distance, normed values,
the first positions always visible, an output gate) beside gated linear attention ("parallel"), their results added
with two scales.  The feed-forward is a mixture of gated experts that a table names by the token's id.  A run of
layers may repeat with the same weights, each pass on caches and state of its own; before every pass a learned row
is added to the stream, and before every pass but the first the embedding output as well.

Tensor names: ``embed``, ``bigram``, ``loop.step``, ``l<i>.norm1`` / ``.norm2`` / ``.shift``, ``l<i>.mix.q`` / ``.k`` /
``.v`` / ``.g`` / ``.o`` / ``.norm`` (lightning), ``l<i>.mix.left.q`` / ``.k`` / ``.v`` / ``.g`` / ``.o`` / ``.rel`` and
``l<i>.mix.right.q`` / ``.k`` / ``.v`` / ``.g`` / ``.o`` / ``.norm`` / ``.a1`` / ``.a2`` / ``.a2.b`` (parallel),
``l<i>.mlp.e<j>.gate`` / ``.up`` / ``.down``, ``l<i>.mlp.table``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config.forward_config import LayerSpec, ModelForwardConfig, PartSpec, ScheduleStep
from ..config.model_config import TilivikConfig
from ..config.registry import register_architecture

SINUSOID_BASE = 10000.0      # the design fixes it


def _mixer(cfg: TilivikConfig, i: int) -> PartSpec:
    layer, p, H = cfg.layers[i], f"l{i}.mix.", cfg.hidden_size
    m = layer["mixer"]
    if layer["type"] == "lightning":
        return PartSpec(
            "lightning_attention",
            {"hidden_size": H, "heads": int(m["heads"]), "dim": int(m["dim"]), "vdim": int(m["vdim"]),
             "decay": [float(c) for c in m["decay"]], "eps": cfg.norm_eps, "shift": True},
            {"q": p + "q", "k": p + "k", "v": p + "v", "g": p + "g", "o": p + "o", "norm": p + "norm",
             "shift": f"l{i}.shift"})
    left, right = m["left"], m["right"]
    mask = left.get("mask") or {}
    soft = PartSpec(
        "biased_window_attention",
        {"hidden_size": H, "heads": int(left["heads"]), "kv_heads": int(left["kv_heads"]), "dim": int(left["dim"]),
         "vdim": int(left["vdim"]), "scale": float(left["scale"]), "softcap": float(left.get("softcap") or 0.0),
         "bias_max": float(left["bias_max"]) if left.get("bias_max") is not None else None,
         "bias_rows": int(left.get("bias_rows", 0) or 0), "window": int(mask.get("size", 0) or 0),
         "keep_first": int(mask.get("keep_first", 0) or 0), "eps": cfg.norm_eps})
    # the low-rank gate's inner size is a tensor's: it is read from the checkpoint unless the config names it
    gla = PartSpec(
        "gated_linear_attention",
        {"hidden_size": H, "heads": int(right["heads"]), "dim": int(right["dim"]), "vdim": int(right["vdim"]),
         "tau": float(right["tau"]), "rank": int(right.get("rank", 0) or 0) or -1, "eps": cfg.norm_eps})
    names = {"shift": f"l{i}.shift"}
    for x in ("q", "k", "v", "g", "o"):
        names["0." + x] = p + "left." + x
        names["1." + x] = p + "right." + x
    if left.get("bias_max") is not None:
        names["0.rel"] = p + "left.rel"
    names.update({"1.norm": p + "right.norm", "1.a1": p + "right.a1", "1.a2": p + "right.a2", "1.a2_bias": p + "right.a2.b"})
    return PartSpec("side_by_side", {"hidden_size": H, "mixers": (soft, gla),
                                     "scales": (float(m["left_scale"]), float(m["right_scale"])), "shift": True}, names)


def _feed_forward(cfg: TilivikConfig, i: int) -> PartSpec:
    mlp, p = cfg.layers[i].get("mlp"), f"l{i}.mlp."
    if mlp is None:
        return PartSpec("none")
    E = int(mlp["router"]["experts"])
    names = {"table": p + "table"}
    for e in range(E):
        names.update({f"gate_{e}": f"{p}e{e}.gate", f"up_{e}": f"{p}e{e}.up", f"down_{e}": f"{p}e{e}.down"})
    return PartSpec("table_experts", {"hidden_size": cfg.hidden_size, "vocab_size": cfg.vocab_size, "experts": E,
                                      "top": int(mlp["router"]["top"]), "ff": int(mlp["expert"]["ff"]), "activation": "silu"},
                    names)


def _norm(cfg: TilivikConfig, name: str, wide: bool = False) -> PartSpec:
    """An RMS norm whose gain is one number; ``wide``: its rows leave in float32 (the token shift reads them)."""
    return PartSpec("rmsnorm", {"dim": cfg.hidden_size, "eps": cfg.norm_eps, "scalar": True,
                                "out_dtype": "float32" if wide else None}, {"weight": name})


def tilivik_forward_config(cfg: TilivikConfig) -> ModelForwardConfig:
    H = cfg.hidden_size
    layers = []
    for i, layer in enumerate(cfg.layers):
        has_ff = layer.get("mlp") is not None
        layers.append(LayerSpec("prenorm", _mixer(cfg, i), _feed_forward(cfg, i),
                                {"input": _norm(cfg, f"l{i}.norm1", wide=True),
                                 "post_mixer": _norm(cfg, f"l{i}.norm2") if has_ff else PartSpec("none")}))
    schedule = []
    times = int(cfg.loop["times"]) if cfg.loop is not None else 0
    for run, (i, t) in enumerate(cfg.run_order()):
        enter = None
        if t is not None and i == int(cfg.loop["start"]):
            # the start of a pass: the embedding output again (but for the first pass), and the pass's learned row
            enter = PartSpec("reenter", {"hidden_size": H, "add_embedded": t > 0, "count": times, "row": t},
                             {"rows": "loop.step"})
        schedule.append(ScheduleStep(layer=i, cache=run, enter=enter))      # every run has a cache and state of its own
    emb = {"vocab_size": cfg.vocab_size, "hidden_size": H, "sinusoid": SINUSOID_BASE,
           "pair": dict(cfg.bigram) if cfg.bigram is not None else None}
    names = {"weight": "embed"}
    if cfg.bigram is not None:
        names["pair"] = "bigram"
    fc = ModelForwardConfig(
        architecture="Tilivik", hidden_size=H, vocab_size=cfg.vocab_size, embedding=PartSpec("token", emb, names),
        layers=tuple(layers), schedule=tuple(schedule), final_norm=_norm(cfg, "final.norm"),
        lm_head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": H, "tied_to": None}, {"weight": "head"}),
        eos_token_ids=cfg.eos_token_ids, max_position_embeddings=0,
        # a layer without a feed-forward may still carry the gain of the norm that would stand before it
        ignorable_tensors=tuple(f"l{i}.norm2" for i, layer in enumerate(cfg.layers) if layer.get("mlp") is None),
        family={"mixers": [cfg.layers[i]["type"] for i, _ in cfg.run_order()], "norm_eps": cfg.norm_eps})
    fc.validate()
    return fc


register_architecture("Tilivik", TilivikConfig, tilivik_forward_config, aliases=("tilivik",))
