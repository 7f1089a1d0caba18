"""Kegozen: the description of the design in parts.

A decoder whose layers are listed one by one in config.json.  A layer has a norm before and a norm after each
sublayer, x <- x + n1b(mixer(n1(x))), x <- x + n2b(ff(n2(x))), all RMS norms whose gain is stored around zero
(1 + w).  The mixer is a selective state-space mixer ("mamba2"), grouped-query attention with normed queries and
keys, a rotation of neighbouring pairs whose long wavelengths may be stretched, values turned by their own positions,
and a sliding window before which whole blocks of positions are seen as their means ("attention"), or causal attention
whose queries come through one latent and whose keys and values through another ("latent_attention"; the rotated part
pairs dim i with i + rot_dim / 2).  The feed-forward is a dense gated one (SiLU), or a mixture of such experts scored
by a sigmoid router (the score multiplies the expert's input) with a gated shared expert, or none.

Tensor names: ``embed``, ``l<i>.norm1`` / ``.norm1b`` / ``.norm2`` / ``.norm2b``, ``l<i>.mix.in`` / ``.conv`` /
``.conv.b`` / ``.dt_bias`` / ``.A_log`` / ``.D`` / ``.norm`` / ``.o`` (mamba2), ``l<i>.mix.q`` / ``.k`` / ``.v`` /
``.q.norm`` / ``.k.norm`` / ``.o`` (attention), ``l<i>.mix.dq`` / ``.dq.norm`` / ``.uq`` / ``.dkv`` / ``.dkv.norm`` /
``.uk`` / ``.uv`` / ``.o`` (latent attention), ``l<i>.mlp.gate`` / ``.up`` / ``.down`` (dense), ``l<i>.mlp.router``,
``l<i>.mlp.e<j>.gate`` / ``.up`` / ``.down``, ``l<i>.mlp.shared.gate`` / ``.up`` / ``.down`` / ``.sg`` (experts),
``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config.forward_config import LayerSpec, ModelForwardConfig, PartSpec, default_schedule
from ..config.model_config import KegozenConfig
from ..config.registry import register_architecture


def _mixer(cfg: KegozenConfig, i: int) -> PartSpec:
    layer, p, H = cfg.layers[i], f"l{i}.mix.", cfg.hidden_size
    m, kind = layer["mixer"], layer["type"]
    if kind == "mamba2":
        return PartSpec(
            "state_space",
            {"hidden_size": H, "heads": int(m["heads"]), "vdim": int(m["vdim"]), "state": int(m["state"]),
             "groups": int(m["groups"]), "conv": int(m["conv"]), "norm_groups": int(m["norm_groups"]), "eps": cfg.norm_eps},
            {"in": p + "in", "conv": p + "conv", "conv_bias": p + "conv.b", "dt_bias": p + "dt_bias", "A_log": p + "A_log",
             "D": p + "D", "norm": p + "norm", "o": p + "o"})
    rot = m.get("rot")
    if kind == "attention":
        mask = m.get("mask") or {}
        return PartSpec(
            "pooled_window_attention",
            {"hidden_size": H, "heads": int(m["heads"]), "kv_heads": int(m["kv_heads"]), "dim": int(m["dim"]),
             "vdim": int(m["vdim"]), "scale": float(m["scale"]), "window": int(mask.get("size", 0) or 0),
             "pool": int(mask.get("pool", 0) or 0), "qk_norm": True, "eps": cfg.norm_eps,
             "rotary_dim": int(rot["dims"]) if rot else 0, "theta": float(rot["base"]) if rot else 0.0,
             "scaling": dict(rot["scaling"]) if rot and rot.get("scaling") else None,
             "rotate_values": rot is not None, "pairing": "interleaved"},
            {"q": p + "q", "k": p + "k", "v": p + "v", "q_norm": p + "q.norm", "k_norm": p + "k.norm", "o": p + "o"})
    r = int(m["rot_dim"])
    position = PartSpec("rope_pairs", {"head_dim": r, "rotary_dim": int(rot["dims"]), "theta": float(rot["base"])})
    q_rank = int(m.get("q_rank", 0) or 0)
    names = {"dkv": p + "dkv", "dkv_norm": p + "dkv.norm", "uk": p + "uk", "uv": p + "uv", "o": p + "o"}
    names.update({"dq": p + "dq", "dq_norm": p + "dq.norm", "uq": p + "uq"} if q_rank else {"q": p + "q"})
    return PartSpec(
        "latent_attention",
        {"hidden_size": H, "heads": int(m["heads"]), "dim": int(m["dim"]), "rot_dim": r, "vdim": int(m["vdim"]),
         "kv_rank": int(m["kv_rank"]), "scale": float(m["scale"]), "window": 0, "eps": cfg.norm_eps, "shares_cache": False,
         "q_rank": q_rank, "pairing": "halves", "position": position},
        names)


def _feed_forward(cfg: KegozenConfig, i: int) -> PartSpec:
    mlp, p, H = cfg.layers[i].get("mlp"), f"l{i}.mlp.", cfg.hidden_size
    if mlp is None:
        return PartSpec("none")
    if mlp["kind"] == "dense":
        return PartSpec("swiglu", {"hidden_size": H, "intermediate_size": int(mlp["ff"])},
                        {"gate": p + "gate", "up": p + "up", "down": p + "down"})
    E = int(mlp["router"]["experts"])
    shared = mlp.get("shared")
    names = {"router": p + "router"}
    for e in range(E):
        names.update({f"gate_{e}": f"{p}e{e}.gate", f"up_{e}": f"{p}e{e}.up", f"down_{e}": f"{p}e{e}.down"})
    if shared:
        names.update({"shared_gate": p + "shared.gate", "shared_up": p + "shared.up", "shared_down": p + "shared.down",
                      "shared_sg": p + "shared.sg"})
    return PartSpec("scored_experts", {"hidden_size": H, "experts": E, "top": int(mlp["router"]["top"]),
                                       "ff": int(mlp["expert"]["ff"]), "shared_ff": int(shared["ff"]) if shared else 0,
                                       "shared_gate": bool(shared)}, names)


def _norm(cfg: KegozenConfig, name: str) -> PartSpec:
    return PartSpec("rmsnorm", {"dim": cfg.hidden_size, "eps": cfg.norm_eps, "add_one": True}, {"weight": name})


def kegozen_forward_config(cfg: KegozenConfig) -> ModelForwardConfig:
    H = cfg.hidden_size
    layers = []
    for i, layer in enumerate(cfg.layers):
        has_ff = layer.get("mlp") is not None
        none = PartSpec("none")
        layers.append(LayerSpec("sandwich", _mixer(cfg, i), _feed_forward(cfg, i),
                                {"input": _norm(cfg, f"l{i}.norm1"), "mixer_out": _norm(cfg, f"l{i}.norm1b"),
                                 "ff_in": _norm(cfg, f"l{i}.norm2") if has_ff else none,
                                 "ff_out": _norm(cfg, f"l{i}.norm2b") if has_ff else none}))
    fc = ModelForwardConfig(
        architecture="Kegozen", hidden_size=H, vocab_size=cfg.vocab_size,
        embedding=PartSpec("token", {"vocab_size": cfg.vocab_size, "hidden_size": H}, {"weight": "embed"}),
        layers=tuple(layers), schedule=default_schedule(len(layers)), final_norm=_norm(cfg, "final.norm"),
        lm_head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": H, "tied_to": None}, {"weight": "head"}),
        eos_token_ids=cfg.eos_token_ids, max_position_embeddings=0,
        # a layer without a feed-forward may still carry the gains of the norms that would stand around it
        ignorable_tensors=tuple(f"l{i}.{n}" for i, layer in enumerate(cfg.layers) if layer.get("mlp") is None
                                for n in ("norm2", "norm2b")),
        family={"mixers": [layer["type"] for layer in cfg.layers], "norm_eps": cfg.norm_eps})
    fc.validate()
    return fc


register_architecture("Kegozen", KegozenConfig, kegozen_forward_config, aliases=("kegozen",))
