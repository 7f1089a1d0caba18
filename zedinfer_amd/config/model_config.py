"""Typed views of a model folder's ``config.json``.

Every size and constant of a model comes from here; no layer size is written
in code.  The keys, their defaults and which of them are required follow the
reference's parser (reference: src/frontend/models/base.cpp:683-720 for the
shared keys, :807-813 for the Qwen2 extras).
"""
from __future__ import annotations

import json
import os
import sys
from dataclasses import dataclass, asdict
from typing import Any, Dict, Mapping, Tuple


class ConfigError(ValueError):
    """A config.json that cannot describe a runnable model."""


_REQUIRED = (
    "hidden_size",
    "intermediate_size",
    "vocab_size",
    "max_position_embeddings",
    "num_hidden_layers",
    "num_attention_heads",
)


def _as_int(d: Mapping[str, Any], key: str) -> int:
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, (int, float)) or int(v) != v:
        raise ConfigError(f"config.json: '{key}' must be an integer, got {v!r}")
    return int(v)


@dataclass(frozen=True)
class ModelConfig:
    """Keys shared by every decoder family the reference parses
    (reference: include/frontend/models/base.hpp:91-137)."""

    architectures: Tuple[str, ...] = ()
    model_type: str = "unknown"
    hidden_act: str = "silu"
    torch_dtype: str = "bfloat16"
    bos_token_id: int = 151643
    eos_token_ids: Tuple[int, ...] = (151643,)
    hidden_size: int = 0
    intermediate_size: int = 0
    vocab_size: int = 0
    max_position_embeddings: int = 0
    num_hidden_layers: int = 0
    num_attention_heads: int = 0
    num_key_value_heads: int = 0
    head_dim: int = 0
    rms_norm_eps: float = 1e-6
    rope_theta: float = 10000.0
    tie_word_embeddings: bool = False

    @property
    def eos_token_id(self) -> int:
        return self.eos_token_ids[0] if self.eos_token_ids else 151643

    # ---- parsing -------------------------------------------------------
    @classmethod
    def _base_kwargs(cls, d: Mapping[str, Any]) -> Dict[str, Any]:
        missing = [k for k in _REQUIRED if k not in d]
        if missing:
            raise ConfigError("config.json lacks required key(s): " + ", ".join(missing))
        eos = d.get("eos_token_id", 151643)
        eos_ids = tuple(int(e) for e in eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        nh = _as_int(d, "num_attention_heads")
        hidden = _as_int(d, "hidden_size")
        # The reference reads hidden_act (base.cpp:686) and computes SiLU whatever it says
        # (transformer_forward.cpp:128-137); a checkpoint trained with another activation would run and be
        # silently something else, so it is refused here.
        act = str(d.get("hidden_act") or "silu")
        if act != "silu":
            raise ConfigError(f"config.json: hidden_act '{act}' is not supported: the feed-forward computes 'silu'")
        # rope_scaling is not among the keys the reference parses (base.cpp:683-720): positions rotate by
        # rope_theta alone.  Said once, so that a long-context variant is not taken for what its config says.
        if d.get("rope_scaling") is not None:
            print("zedinfer_amd: config.json has 'rope_scaling'; it is ignored, as the reference ignores it "
                  "(src/frontend/models/base.cpp:683-720 does not parse it): angles come from rope_theta alone",
                  file=sys.stderr, flush=True)
        head_dim = int(d.get("head_dim") or 0)
        if head_dim == 0:
            if nh <= 0 or hidden % nh:
                raise ConfigError(
                    f"config.json: hidden_size {hidden} is not divisible by num_attention_heads {nh} "
                    "and no head_dim is given")
            head_dim = hidden // nh
        return dict(
            architectures=tuple(d.get("architectures") or ()),
            model_type=str(d.get("model_type") or "unknown"),
            hidden_act=act,
            torch_dtype=str(d.get("torch_dtype") or "bfloat16"),
            bos_token_id=int(d.get("bos_token_id", 151643)),
            eos_token_ids=eos_ids,
            hidden_size=hidden,
            intermediate_size=_as_int(d, "intermediate_size"),
            vocab_size=_as_int(d, "vocab_size"),
            max_position_embeddings=_as_int(d, "max_position_embeddings"),
            num_hidden_layers=_as_int(d, "num_hidden_layers"),
            num_attention_heads=nh,
            num_key_value_heads=int(d.get("num_key_value_heads", nh)),
            head_dim=head_dim,
            rms_norm_eps=float(d.get("rms_norm_eps", 1e-6)),
            rope_theta=float(d.get("rope_theta", 10000.0)),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
        )

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "ModelConfig":
        cfg = cls(**cls._base_kwargs(d))
        cfg.validate()
        return cfg

    @classmethod
    def from_json_file(cls, path: str) -> "ModelConfig":
        return cls.from_dict(read_config_json(path))

    # ---- checks --------------------------------------------------------
    def validate(self) -> None:
        pos = ("hidden_size", "intermediate_size", "vocab_size", "num_hidden_layers",
               "num_attention_heads", "num_key_value_heads", "head_dim", "max_position_embeddings")
        for k in pos:
            if getattr(self, k) <= 0:
                raise ConfigError(f"config.json: '{k}' must be positive, got {getattr(self, k)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"config.json: num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"config.json: head_dim {self.head_dim} must be even for rotary encoding")
        if not (self.rms_norm_eps > 0):
            raise ConfigError(f"config.json: rms_norm_eps must be positive, got {self.rms_norm_eps}")
        if not (self.rope_theta > 0):
            raise ConfigError(f"config.json: rope_theta must be positive, got {self.rope_theta}")

    # ---- writing -------------------------------------------------------
    def to_dict(self) -> Dict[str, Any]:
        d = asdict(self)
        d["architectures"] = list(self.architectures)
        eos = list(d.pop("eos_token_ids"))
        d["eos_token_id"] = eos[0] if len(eos) == 1 else eos
        return d

    def save(self, folder: str) -> None:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(self.to_dict(), f, indent=2)


@dataclass(frozen=True)
class Qwen2Config(ModelConfig):
    """Qwen2 adds the three sliding-window keys
    (reference: include/frontend/models/qwen2.hpp:10-15, base.cpp:807-813)."""

    sliding_window: int = 4096
    max_window_layers: int = 21
    use_sliding_window: bool = False

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "Qwen2Config":
        kw = cls._base_kwargs(d)
        sw = d.get("sliding_window")
        kw["sliding_window"] = int(sw) if isinstance(sw, (int, float)) and not isinstance(sw, bool) else 4096
        kw["max_window_layers"] = int(d.get("max_window_layers", 21))
        kw["use_sliding_window"] = bool(d.get("use_sliding_window", False))
        cfg = cls(**kw)
        cfg.validate()
        return cfg

    def validate(self) -> None:
        super().validate()
        if self.use_sliding_window:
            if self.sliding_window <= 0:
                raise ConfigError(f"config.json: sliding_window must be positive, got {self.sliding_window}")
            if self.max_window_layers < 0:
                raise ConfigError(
                    f"config.json: max_window_layers must be non-negative, got {self.max_window_layers}")


def read_config_json(path: str) -> Dict[str, Any]:
    """Read ``config.json`` from a model folder or a file path."""
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json at {path}")
    with open(path) as f:
        try:
            return json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path} is not valid JSON: {e}") from e


@dataclass(frozen=True)
class DedelornConfig(ModelConfig):
    """The Dedelorn design's config.json: ``width``, ``vocab``, ``norm.eps`` and a list ``layers`` whose entries
    each name a mixer by ``type`` ("delta": a gated delta rule; "latent_attention": windowed attention over cached
    latents) with its sizes under ``mixer`` and a feed-forward under ``mlp`` (``kind`` "dense" or "moe", or null for
    none).  Every size and constant of a model is read from here; the shared keys of ``ModelConfig`` that the
    format does not have keep their neutral values (no end-of-sequence token, no position limit)."""

    layers: Tuple[Any, ...] = ()
    norm_eps: float = 1e-6

    MIXER_KEYS = {"delta": ("heads", "kv_heads", "dim", "vdim", "conv"),
                  "latent_attention": ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot")}

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "DedelornConfig":
        missing = [k for k in ("width", "vocab", "layers", "norm") if k not in d]
        if missing:
            raise ConfigError("config.json lacks required key(s): " + ", ".join(missing))
        if not isinstance(d["layers"], (list, tuple)) or not d["layers"]:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        if not isinstance(d["norm"], Mapping) or "eps" not in d["norm"]:
            raise ConfigError("config.json: 'norm' must give 'eps'")
        eos = d.get("eos_token_id")
        cfg = cls(architectures=(str(d.get("architecture", "Dedelorn")),), model_type="dedelorn",
                  torch_dtype=str(d.get("torch_dtype") or "bfloat16"), hidden_size=_as_int(d, "width"),
                  vocab_size=_as_int(d, "vocab"), num_hidden_layers=len(d["layers"]),
                  eos_token_ids=() if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos])),
                  layers=tuple(json.loads(json.dumps(layer)) for layer in d["layers"]), norm_eps=float(d["norm"]["eps"]))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.hidden_size <= 0 or self.vocab_size <= 0:
            raise ConfigError("config.json: 'width' and 'vocab' must be positive")
        if not (self.norm_eps > 0):
            raise ConfigError(f"config.json: norm.eps must be positive, got {self.norm_eps}")
        for i, layer in enumerate(self.layers):
            kind = layer.get("type") if isinstance(layer, Mapping) else None
            if kind not in self.MIXER_KEYS:
                raise ConfigError(f"config.json: layer {i} has type {kind!r}; known: {', '.join(sorted(self.MIXER_KEYS))}")
            m = layer.get("mixer")
            lacking = [k for k in self.MIXER_KEYS[kind] if not isinstance(m, Mapping) or k not in m]
            if lacking:
                raise ConfigError(f"config.json: layer {i} ({kind}) lacks mixer key(s): " + ", ".join(lacking))
            if kind == "delta":
                if m["heads"] % m["kv_heads"]:
                    raise ConfigError(f"config.json: layer {i}: heads {m['heads']} is not a multiple of kv_heads {m['kv_heads']}")
            else:
                if m["rot"].get("dims") != m["rot_dim"] or m["rot_dim"] % 2 or not m["rot"].get("base", 0) > 0:
                    raise ConfigError(f"config.json: layer {i}: rot.dims must equal rot_dim and be even, rot.base positive")
                if m.get("mask") is not None and not int(m["mask"].get("size", 0)) > 0:
                    raise ConfigError(f"config.json: layer {i}: mask.size must be positive")
                src = m.get("kv_from")
                if src is not None:
                    ok = isinstance(src, int) and 0 <= src < i and self.layers[src].get("type") == "latent_attention" \
                        and self.layers[src]["mixer"].get("kv_from") is None
                    if ok:
                        o = self.layers[src]["mixer"]
                        ok = (o["kv_rank"], o["rot_dim"], o["rot"]) == (m["kv_rank"], m["rot_dim"], m["rot"])
                    if not ok:
                        raise ConfigError(f"config.json: layer {i}: kv_from must name an earlier latent_attention layer with "
                                          "a projection of its own and the same kv_rank, rot_dim and rot")
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            if mlp.get("kind") == "dense":
                if not int(mlp.get("ff", 0)) > 0:
                    raise ConfigError(f"config.json: layer {i}: a dense mlp needs a positive 'ff'")
            elif mlp.get("kind") == "moe":
                r = mlp.get("router") or {}
                if not int((mlp.get("expert") or {}).get("ff", 0)) > 0 or not (0 < int(r.get("top", 0)) <= int(r.get("experts", 0))):
                    raise ConfigError(f"config.json: layer {i}: a moe mlp needs expert.ff, router.experts and router.top "
                                      "(at most the experts)")
            else:
                raise ConfigError(f"config.json: layer {i}: mlp.kind {mlp.get('kind')!r} is neither 'dense' nor 'moe'")

    def to_dict(self) -> Dict[str, Any]:
        d = {"architecture": self.architectures[0] if self.architectures else "Dedelorn",
             "layers": json.loads(json.dumps(list(self.layers))), "norm": {"eps": self.norm_eps},
             "vocab": self.vocab_size, "width": self.hidden_size}
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d


@dataclass(frozen=True)
class TosisunConfig(ModelConfig):
    """The Tosisun design's config.json: ``width``, ``vocab``, ``norm.eps``, ``logit_softcap`` (optional) and a list
    ``layers`` whose entries each name a mixer by ``type`` ("attention": grouped-query attention whose projections
    pass a short convolution, with a sink in the softmax) with its sizes under ``mixer`` and a feed-forward under
    ``mlp`` (``kind`` "dense" or "moe", or null for none).  An entry with ``weights_of``: j runs with layer j's
    tensors and a cache and state of its own.  Every size and constant of a model is read from here; the shared keys
    of ``ModelConfig`` that the format does not have keep their neutral values."""

    layers: Tuple[Any, ...] = ()
    norm_eps: float = 1e-5
    logit_softcap: float = 0.0

    MIXER_KEYS = {"attention": ("heads", "kv_heads", "dim", "vdim", "conv", "scale", "rot")}

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "TosisunConfig":
        missing = [k for k in ("width", "vocab", "layers", "norm") if k not in d]
        if missing:
            raise ConfigError("config.json lacks required key(s): " + ", ".join(missing))
        if not isinstance(d["layers"], (list, tuple)) or not d["layers"]:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        if not isinstance(d["norm"], Mapping) or "eps" not in d["norm"]:
            raise ConfigError("config.json: 'norm' must give 'eps'")
        eos = d.get("eos_token_id")
        cap = d.get("logit_softcap")
        cfg = cls(architectures=(str(d.get("architecture", "Tosisun")),), model_type="tosisun",
                  torch_dtype=str(d.get("torch_dtype") or "bfloat16"), hidden_size=_as_int(d, "width"),
                  vocab_size=_as_int(d, "vocab"), num_hidden_layers=len(d["layers"]),
                  eos_token_ids=() if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos])),
                  layers=tuple(json.loads(json.dumps(layer)) for layer in d["layers"]), norm_eps=float(d["norm"]["eps"]),
                  logit_softcap=float(cap) if cap else 0.0)
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.hidden_size <= 0 or self.vocab_size <= 0:
            raise ConfigError("config.json: 'width' and 'vocab' must be positive")
        if not (self.norm_eps > 0):
            raise ConfigError(f"config.json: norm.eps must be positive, got {self.norm_eps}")
        if self.logit_softcap < 0:
            raise ConfigError(f"config.json: logit_softcap must be positive, got {self.logit_softcap}")
        for i, layer in enumerate(self.layers):
            if isinstance(layer, Mapping) and layer.get("weights_of") is not None:
                # such a layer is its owner's parts once more: what else its entry says repeats the owner's entry and
                # is not read
                self.owner_of(i)
                continue
            kind = layer.get("type") if isinstance(layer, Mapping) else None
            if kind not in self.MIXER_KEYS:
                raise ConfigError(f"config.json: layer {i} has type {kind!r}; known: {', '.join(sorted(self.MIXER_KEYS))}")
            m = layer.get("mixer")
            lacking = [k for k in self.MIXER_KEYS[kind] if not isinstance(m, Mapping) or k not in m]
            if lacking:
                raise ConfigError(f"config.json: layer {i} ({kind}) lacks mixer key(s): " + ", ".join(lacking))
            if any(int(m[k]) <= 0 for k in ("heads", "kv_heads", "dim", "vdim", "conv")) or int(m["heads"]) % int(m["kv_heads"]):
                raise ConfigError(f"config.json: layer {i}: heads, kv_heads, dim, vdim and conv must be positive, heads a "
                                  "multiple of kv_heads")
            if not float(m["scale"]) > 0:
                raise ConfigError(f"config.json: layer {i}: scale must be positive")
            rot = m["rot"]
            if not isinstance(rot, Mapping) or int(rot.get("dims", -1)) < 0 or int(rot.get("dims", -1)) % 2 \
                    or int(rot["dims"]) > int(m["dim"]) or (int(rot["dims"]) > 0 and not float(rot.get("base", 0)) > 0):
                raise ConfigError(f"config.json: layer {i}: rot.dims must be even and within dim, rot.base positive")
            sc = rot.get("scaling")
            if sc is not None and (not isinstance(sc, Mapping) or any(k not in sc for k in ("factor", "low", "high", "original"))):
                raise ConfigError(f"config.json: layer {i}: rot.scaling needs factor, low, high and original")
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            if mlp.get("kind") == "dense":
                if not int(mlp.get("ff", 0)) > 0:
                    raise ConfigError(f"config.json: layer {i}: a dense mlp needs a positive 'ff'")
            elif mlp.get("kind") == "moe":
                r, ex = mlp.get("router") or {}, mlp.get("expert") or {}
                if not int(ex.get("ff", 0)) > 0 or not float(ex.get("limit", 0)) > 0 \
                        or not (0 < int(r.get("top", 0)) <= int(r.get("experts", 0))):
                    raise ConfigError(f"config.json: layer {i}: a moe mlp needs expert.ff, expert.limit, router.experts and "
                                      "router.top (at most the experts)")
                sh = mlp.get("shared")
                if sh is not None and (not int(sh.get("ff", 0)) > 0 or not float(sh.get("limit", 0)) > 0):
                    raise ConfigError(f"config.json: layer {i}: a shared expert needs ff and limit")
            else:
                raise ConfigError(f"config.json: layer {i}: mlp.kind {mlp.get('kind')!r} is neither 'dense' nor 'moe'")

    def owner_of(self, i: int) -> int:
        """The layer whose tensors layer ``i`` runs with: itself, or what its ``weights_of`` names (followed to a
        layer that has tensors of its own; it may stand before or after)."""
        seen = set()
        while isinstance(self.layers[i], Mapping) and self.layers[i].get("weights_of") is not None:
            src = self.layers[i]["weights_of"]
            if isinstance(src, bool) or not isinstance(src, int) or not (0 <= src < len(self.layers)) or src == i or src in seen:
                raise ConfigError(f"config.json: layer {i}: weights_of must name another layer of the model, and lead to one "
                                  "with tensors of its own")
            seen.add(i)
            i = src
        return i

    def to_dict(self) -> Dict[str, Any]:
        d = {"architecture": self.architectures[0] if self.architectures else "Tosisun",
             "layers": json.loads(json.dumps(list(self.layers))), "norm": {"eps": self.norm_eps},
             "vocab": self.vocab_size, "width": self.hidden_size}
        if self.logit_softcap:
            d["logit_softcap"] = self.logit_softcap
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d


@dataclass(frozen=True)
class TilivikConfig(ModelConfig):
    """The Tilivik design's config.json: ``width``, ``vocab``, ``norm.eps``, ``embedding.bigram`` (``buckets``,
    ``mul_prev``, ``mul_cur``; optional), ``loop`` (``start``, ``stop``, ``times``: layers start .. stop-1 run
    ``times`` times in a row; optional) and a list ``layers`` whose entries each name a mixer by ``type``
    ("lightning": linear attention with a fixed decay per head; "parallel": windowed softmax attention with a bias
    by distance beside gated linear attention) with its sizes under ``mixer`` and a feed-forward under ``mlp``
    (``kind`` "moe": experts named by a table of token ids; or null for none).  Every size and constant of a model is
    read from here (the rows of a layer's bias table are the tensor's own unless ``mixer.left.bias_rows`` names
    them); the shared keys of ``ModelConfig`` that the format does not have keep their neutral values."""

    layers: Tuple[Any, ...] = ()
    norm_eps: float = 1e-6
    bigram: Any = None          # {"buckets", "mul_prev", "mul_cur"} or None
    loop: Any = None            # {"start", "stop", "times"} or None

    MIXER_KEYS = {"lightning": ("heads", "dim", "vdim", "decay"),
                  "parallel": ("left", "right", "left_scale", "right_scale")}
    LEFT_KEYS = ("heads", "kv_heads", "dim", "vdim", "scale")
    RIGHT_KEYS = ("heads", "dim", "vdim", "tau")

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "TilivikConfig":
        missing = [k for k in ("width", "vocab", "layers", "norm") if k not in d]
        if missing:
            raise ConfigError("config.json lacks required key(s): " + ", ".join(missing))
        if not isinstance(d["layers"], (list, tuple)) or not d["layers"]:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        if not isinstance(d["norm"], Mapping) or "eps" not in d["norm"]:
            raise ConfigError("config.json: 'norm' must give 'eps'")
        eos = d.get("eos_token_id")
        bigram = (d.get("embedding") or {}).get("bigram")
        loop = d.get("loop")
        cfg = cls(architectures=(str(d.get("architecture", "Tilivik")),), model_type="tilivik",
                  torch_dtype=str(d.get("torch_dtype") or "bfloat16"), hidden_size=_as_int(d, "width"),
                  vocab_size=_as_int(d, "vocab"), num_hidden_layers=len(d["layers"]),
                  eos_token_ids=() if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos])),
                  layers=tuple(json.loads(json.dumps(layer)) for layer in d["layers"]), norm_eps=float(d["norm"]["eps"]),
                  bigram=json.loads(json.dumps(bigram)) if bigram else None,
                  loop=json.loads(json.dumps(loop)) if loop else None)
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.hidden_size <= 0 or self.vocab_size <= 0:
            raise ConfigError("config.json: 'width' and 'vocab' must be positive")
        if not (self.norm_eps > 0):
            raise ConfigError(f"config.json: norm.eps must be positive, got {self.norm_eps}")
        if self.bigram is not None:
            lacking = [k for k in ("buckets", "mul_prev", "mul_cur") if not isinstance(self.bigram, Mapping) or k not in self.bigram]
            if lacking or int(self.bigram["buckets"]) <= 0:
                raise ConfigError("config.json: embedding.bigram needs a positive 'buckets', 'mul_prev' and 'mul_cur'")
        if self.loop is not None:
            lp = self.loop
            if not isinstance(lp, Mapping) or any(k not in lp for k in ("start", "stop", "times")) \
                    or not (0 <= int(lp["start"]) < int(lp["stop"]) <= len(self.layers)) or int(lp["times"]) < 1:
                raise ConfigError("config.json: loop needs 0 <= start < stop <= the number of layers and times >= 1")
        for i, layer in enumerate(self.layers):
            kind = layer.get("type") if isinstance(layer, Mapping) else None
            if kind not in self.MIXER_KEYS:
                raise ConfigError(f"config.json: layer {i} has type {kind!r}; known: {', '.join(sorted(self.MIXER_KEYS))}")
            m = layer.get("mixer")
            lacking = [k for k in self.MIXER_KEYS[kind] if not isinstance(m, Mapping) or k not in m]
            if lacking:
                raise ConfigError(f"config.json: layer {i} ({kind}) lacks mixer key(s): " + ", ".join(lacking))
            if kind == "lightning":
                if any(int(m[k]) <= 0 for k in ("heads", "dim", "vdim")) or len(m["decay"]) != int(m["heads"]):
                    raise ConfigError(f"config.json: layer {i}: heads, dim and vdim must be positive, one decay a head")
            else:
                for side, keys in (("left", self.LEFT_KEYS), ("right", self.RIGHT_KEYS)):
                    lacking = [k for k in keys if not isinstance(m[side], Mapping) or k not in m[side]]
                    if lacking:
                        raise ConfigError(f"config.json: layer {i}: mixer.{side} lacks key(s): " + ", ".join(lacking))
                left, right = m["left"], m["right"]
                if any(int(left[k]) <= 0 for k in ("heads", "kv_heads", "dim", "vdim")) or int(left["heads"]) % int(left["kv_heads"]):
                    raise ConfigError(f"config.json: layer {i}: mixer.left: sizes must be positive, heads a multiple of kv_heads")
                if not float(left["scale"]) > 0 or float(left.get("softcap") or 0) < 0:
                    raise ConfigError(f"config.json: layer {i}: mixer.left: scale must be positive, softcap not negative")
                mask = left.get("mask")
                if mask is not None and (not int(mask.get("size", 0)) > 0 or int(mask.get("keep_first", 0)) < 0):
                    raise ConfigError(f"config.json: layer {i}: mask.size must be positive, mask.keep_first not negative")
                if any(int(right[k]) <= 0 for k in ("heads", "dim", "vdim")) or not float(right["tau"]) > 0:
                    raise ConfigError(f"config.json: layer {i}: mixer.right: sizes and tau must be positive")
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            if mlp.get("kind") != "moe":
                raise ConfigError(f"config.json: layer {i}: mlp.kind {mlp.get('kind')!r} is not 'moe'")
            r = mlp.get("router") or {}
            if not int((mlp.get("expert") or {}).get("ff", 0)) > 0 or not (0 < int(r.get("top", 0)) <= int(r.get("experts", 0))):
                raise ConfigError(f"config.json: layer {i}: a moe mlp needs expert.ff, router.experts and router.top "
                                  "(at most the experts)")

    def run_order(self):
        """(layer, pass) in the order the layers run; pass is None outside the repeated run."""
        L = len(self.layers)
        if self.loop is None:
            return [(i, None) for i in range(L)]
        a, b, times = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        order = [(i, None) for i in range(a)]
        for t in range(times):
            order += [(i, t) for i in range(a, b)]
        return order + [(i, None) for i in range(b, L)]

    def to_dict(self) -> Dict[str, Any]:
        d = {"architecture": self.architectures[0] if self.architectures else "Tilivik",
             "layers": json.loads(json.dumps(list(self.layers))), "norm": {"eps": self.norm_eps},
             "vocab": self.vocab_size, "width": self.hidden_size}
        if self.bigram is not None:
            d["embedding"] = {"bigram": dict(self.bigram)}
        if self.loop is not None:
            d["loop"] = dict(self.loop)
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d


@dataclass(frozen=True)
class KegozenConfig(ModelConfig):
    """The Kegozen design's config.json: ``width``, ``vocab``, ``norm.eps`` and a list ``layers`` whose entries each
    name a mixer by ``type`` ("mamba2": a selective state-space mixer; "attention": grouped-query attention under a
    sliding window that sees older positions as means of blocks; "latent_attention": causal attention whose queries,
    keys and values come through latents) with its sizes and constants under ``mixer``, and a feed-forward under
    ``mlp`` (``kind`` "dense" with ``ff``; ``kind`` "moe" with ``router.experts`` / ``router.top``, ``expert.ff`` and
    optionally ``shared.ff``; or null for none).  Every size and constant of a model is read from here; the shared keys
    of ``ModelConfig`` that the format does not have keep their neutral values."""

    layers: Tuple[Any, ...] = ()
    norm_eps: float = 1e-6

    MIXER_KEYS = {"mamba2": ("heads", "vdim", "state", "groups", "conv", "norm_groups"),
                  "attention": ("heads", "kv_heads", "dim", "vdim", "scale"),
                  "latent_attention": ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale")}

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "KegozenConfig":
        missing = [k for k in ("width", "vocab", "layers", "norm") if k not in d]
        if missing:
            raise ConfigError("config.json lacks required key(s): " + ", ".join(missing))
        if not isinstance(d["layers"], (list, tuple)) or not d["layers"]:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        if not isinstance(d["norm"], Mapping) or "eps" not in d["norm"]:
            raise ConfigError("config.json: 'norm' must give 'eps'")
        eos = d.get("eos_token_id")
        cfg = cls(architectures=(str(d.get("architecture", "Kegozen")),), model_type="kegozen",
                  torch_dtype=str(d.get("torch_dtype") or "bfloat16"), hidden_size=_as_int(d, "width"),
                  vocab_size=_as_int(d, "vocab"), num_hidden_layers=len(d["layers"]),
                  eos_token_ids=() if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos])),
                  layers=tuple(json.loads(json.dumps(layer)) for layer in d["layers"]), norm_eps=float(d["norm"]["eps"]))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.hidden_size <= 0 or self.vocab_size <= 0:
            raise ConfigError("config.json: 'width' and 'vocab' must be positive")
        if not (self.norm_eps > 0):
            raise ConfigError(f"config.json: norm.eps must be positive, got {self.norm_eps}")
        for i, layer in enumerate(self.layers):
            kind = layer.get("type") if isinstance(layer, Mapping) else None
            if kind not in self.MIXER_KEYS:
                raise ConfigError(f"config.json: layer {i} has type {kind!r}; known: {', '.join(sorted(self.MIXER_KEYS))}")
            m = layer.get("mixer")
            lacking = [k for k in self.MIXER_KEYS[kind] if not isinstance(m, Mapping) or k not in m]
            if lacking:
                raise ConfigError(f"config.json: layer {i} ({kind}) lacks mixer key(s): " + ", ".join(lacking))
            if any(int(m[k]) <= 0 for k in self.MIXER_KEYS[kind] if k != "scale") or ("scale" in m and not float(m["scale"]) > 0):
                raise ConfigError(f"config.json: layer {i} ({kind}): sizes and the scale must be positive")
            if kind == "mamba2":
                if int(m["heads"]) % int(m["groups"]) or (int(m["heads"]) * int(m["vdim"])) % int(m["norm_groups"]):
                    raise ConfigError(f"config.json: layer {i}: heads must be a multiple of groups, heads * vdim of norm_groups")
            else:
                rot = m.get("rot")
                if rot is not None and (not isinstance(rot, Mapping) or "base" not in rot or "dims" not in rot
                                        or int(rot["dims"]) % 2 or int(rot["dims"]) <= 0 or not float(rot["base"]) > 1):
                    raise ConfigError(f"config.json: layer {i}: rot needs a base above 1 and an even, positive dims")
            if kind == "attention":
                if int(m["heads"]) % int(m["kv_heads"]):
                    raise ConfigError(f"config.json: layer {i}: heads must be a multiple of kv_heads")
                if m.get("rot") is not None and (int(m["rot"]["dims"]) > int(m["dim"]) or int(m["vdim"]) % 2):
                    raise ConfigError(f"config.json: layer {i}: rot.dims within dim, and an even vdim")
                mask = m.get("mask")
                if mask is not None and (not int(mask.get("size", 0)) > 0 or int(mask.get("pool", 0) or 0) < 0):
                    raise ConfigError(f"config.json: layer {i}: mask.size must be positive, mask.pool not negative")
            if kind == "latent_attention":
                if m.get("rot") is None or int(m["rot"]["dims"]) != int(m["rot_dim"]):
                    raise ConfigError(f"config.json: layer {i}: rot.dims must be rot_dim")
                if int(m.get("q_rank", 0) or 0) < 0:
                    raise ConfigError(f"config.json: layer {i}: q_rank must not be negative")
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            if mlp.get("kind") == "dense":
                if not int(mlp.get("ff", 0)) > 0:
                    raise ConfigError(f"config.json: layer {i}: a dense mlp needs a positive ff")
            elif mlp.get("kind") == "moe":
                r = mlp.get("router") or {}
                if not int((mlp.get("expert") or {}).get("ff", 0)) > 0 or not (0 < int(r.get("top", 0)) <= int(r.get("experts", 0))):
                    raise ConfigError(f"config.json: layer {i}: a moe mlp needs expert.ff, router.experts and router.top "
                                      "(at most the experts)")
                if mlp.get("shared") is not None and not int(mlp["shared"].get("ff", 0)) > 0:
                    raise ConfigError(f"config.json: layer {i}: a shared expert needs a positive ff")
            else:
                raise ConfigError(f"config.json: layer {i}: mlp.kind {mlp.get('kind')!r} is neither 'dense' nor 'moe'")

    def to_dict(self) -> Dict[str, Any]:
        d = {"architecture": self.architectures[0] if self.architectures else "Kegozen",
             "layers": json.loads(json.dumps(list(self.layers))), "norm": {"eps": self.norm_eps},
             "vocab": self.vocab_size, "width": self.hidden_size}
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d
