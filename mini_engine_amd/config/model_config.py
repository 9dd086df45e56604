"""Typed model configurations read from a model folder's ``config.json``.

The reference hands the untyped ``transformers`` config object straight to the
model (reference ``config.py:25``, ``models/qwen3.py:15-23,81-84,107-108``).
Here every architecture has a frozen dataclass whose fields are exactly the
``config.json`` keys it uses; no size or constant of the model lives anywhere
else in the code.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, fields
from typing import Any, Callable


class ConfigError(ValueError):
    """A ``config.json`` that the engine cannot run, with the reason."""


_CONFIG_CLASSES: dict[str, type] = {}


def register_config(architecture: str) -> Callable[[type], type]:
    """Class decorator: ``architecture`` (as spelled in ``architectures[0]``) -> config class."""

    def deco(cls: type) -> type:
        _CONFIG_CLASSES[architecture] = cls
        cls.architecture_name = architecture
        return cls

    return deco


def config_class_for(architecture: str) -> type:
    try:
        return _CONFIG_CLASSES[architecture]
    except KeyError:
        known = ", ".join(sorted(_CONFIG_CLASSES)) or "<none>"
        raise ConfigError(
            f"unknown architecture {architecture!r}; registered architectures: {known}"
        ) from None


def read_config_json(model_dir: str) -> dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{model_dir!r} has no config.json")
    with open(path) as f:
        raw = json.load(f)
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return raw


def architecture_of(raw: dict[str, Any]) -> str:
    archs = raw.get("architectures")
    if not archs and isinstance(raw.get("architecture"), str):
        return raw["architecture"]              # the one-name spelling some designs use
    if not archs or not isinstance(archs, (list, tuple)) or not isinstance(archs[0], str):
        raise ConfigError("config.json must name the model class in 'architectures': [\"...\"] (or 'architecture': \"...\")")
    return archs[0]


def load_model_config(model_dir: str):
    """Read ``config.json`` and build the typed config of the architecture it names."""
    raw = read_config_json(model_dir)
    return config_class_for(architecture_of(raw)).from_dict(raw)


def _need(raw: dict, key: str, kind, where: str = "config.json"):
    if key not in raw or raw[key] is None:
        raise ConfigError(f"{where} lacks the required key {key!r}")
    v = raw[key]
    if kind is int:
        if isinstance(v, bool) or not isinstance(v, int):
            raise ConfigError(f"{where}: {key!r} must be an integer, got {v!r}")
    elif kind is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{where}: {key!r} must be a number, got {v!r}")
        v = float(v)
    return v


@register_config("Qwen3ForCausalLM")
@dataclass(frozen=True)
class Qwen3Config:
    """The ``config.json`` keys of a Qwen3 dense decoder.

    Keys the reference reads: ``models/qwen3.py:15-23`` (heads, head_dim, eps),
    ``:60-62`` (hidden/intermediate), ``:81-84`` (rope theta, positions, vocab,
    layers), ``:107-108`` (tying). ``head_dim`` is read directly, so the query
    width ``num_attention_heads * head_dim`` need not equal ``hidden_size``.

    Beyond the reference: ``sliding_window`` / ``layer_types`` are honoured when
    ``use_sliding_window`` is true (a query at position i then sees keys j with
    ``0 <= i - j < sliding_window`` in layers of type ``"sliding_attention"``);
    the reference ignores those keys and always attends to every earlier key.
    """

    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool | None  # None: decided by whether the checkpoint stores lm_head.weight
    max_position_embeddings: int | None
    sliding_window: int | None
    layer_types: tuple[str, ...]
    eos_token_id: int | None = None

    LAYER_TYPES = ("full_attention", "sliding_attention")

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "Qwen3Config":
        hidden = _need(raw, "hidden_size", int)
        heads = _need(raw, "num_attention_heads", int)
        kv_heads = raw.get("num_key_value_heads")
        if kv_heads is None:
            kv_heads = heads
        head_dim = raw.get("head_dim")
        if head_dim is None:
            if hidden % heads:
                raise ConfigError("config.json has no 'head_dim' and hidden_size is not a multiple "
                                  "of num_attention_heads")
            head_dim = hidden // heads
        layers = _need(raw, "num_hidden_layers", int)

        # rope theta: transformers 5 nests it in rope_parameters (reference models/qwen3.py:81);
        # older config.json files carry it at the top level.
        rope = raw.get("rope_parameters") or {}
        scaling = raw.get("rope_scaling") or {}
        theta = rope.get("rope_theta", raw.get("rope_theta", scaling.get("rope_theta")))
        if theta is None:
            raise ConfigError("config.json lacks 'rope_theta' (top level or in 'rope_parameters')")
        for src in (rope, scaling):
            kind = src.get("rope_type", src.get("type", "default"))
            if kind not in (None, "default"):
                raise ConfigError(f"rope scaling of type {kind!r} is not supported (only plain rotary)")
        if raw.get("attention_bias"):
            raise ConfigError("attention_bias=true is not supported: Qwen3 dense has no biases")
        act = raw.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"hidden_act={act!r} is not supported (the feed-forward is SiLU-gated)")

        window = raw.get("sliding_window") if raw.get("use_sliding_window") else None
        if window is not None:
            if isinstance(window, bool) or not isinstance(window, int) or window < 1:
                raise ConfigError(f"sliding_window must be a positive integer, got {window!r}")
            types = raw.get("layer_types")
            if types is None:
                first = raw.get("max_window_layers", layers)
                types = ["sliding_attention" if i >= first else "full_attention" for i in range(layers)]
        else:
            types = ["full_attention"] * layers
        types = tuple(types)
        if len(types) != layers or any(t not in cls.LAYER_TYPES for t in types):
            raise ConfigError(f"layer_types must hold {layers} entries from {cls.LAYER_TYPES}, got {types!r}")
        if "sliding_attention" not in types:
            window = None

        tie = raw.get("tie_word_embeddings")
        if tie is not None and not isinstance(tie, bool):
            raise ConfigError(f"tie_word_embeddings must be true or false, got {tie!r}")
        eos = raw.get("eos_token_id")
        if isinstance(eos, (list, tuple)):
            eos = eos[0] if eos else None
        cfg = cls(
            vocab_size=_need(raw, "vocab_size", int),
            hidden_size=hidden,
            intermediate_size=_need(raw, "intermediate_size", int),
            num_hidden_layers=layers,
            num_attention_heads=heads,
            num_key_value_heads=int(kv_heads),
            head_dim=int(head_dim),
            rms_norm_eps=_need(raw, "rms_norm_eps", float),
            rope_theta=float(theta),
            tie_word_embeddings=tie,
            max_position_embeddings=raw.get("max_position_embeddings"),
            sliding_window=window,
            layer_types=types,
            eos_token_id=eos,
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for f in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                  "num_attention_heads", "num_key_value_heads", "head_dim"):
            v = getattr(self, f)
            if not isinstance(v, int) or isinstance(v, bool) or v < 1:
                raise ConfigError(f"{f} must be a positive integer, got {v!r}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads={self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads={self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim={self.head_dim} must be even for rotary pairs")
        if not self.rms_norm_eps > 0:
            raise ConfigError(f"rms_norm_eps must be positive, got {self.rms_norm_eps!r}")
        if not self.rope_theta > 0:
            raise ConfigError(f"rope_theta must be positive, got {self.rope_theta!r}")

    def to_dict(self) -> dict[str, Any]:
        """A ``config.json`` that reads back to an equal config."""
        d: dict[str, Any] = {
            "architectures": [self.architecture_name],
            "model_type": "qwen3",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "hidden_act": "silu",
            "attention_bias": False,
        }
        if self.tie_word_embeddings is not None:
            d["tie_word_embeddings"] = self.tie_word_embeddings
        if self.max_position_embeddings is not None:
            d["max_position_embeddings"] = self.max_position_embeddings
        if self.sliding_window is not None:
            d["use_sliding_window"] = True
            d["sliding_window"] = self.sliding_window
            d["layer_types"] = list(self.layer_types)
        else:
            d["use_sliding_window"] = False
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        return d

    def flat(self) -> dict[str, Any]:
        """Sizes as a flat dict (for benchmark records)."""
        return {f.name: getattr(self, f.name) for f in fields(self)
                if f.name not in ("layer_types",)}


# ------------------------------------------------------------------------------------ Sigosun

@dataclass(frozen=True)
class SigosunLayer:
    """One entry of a Sigosun config's `layers`: which mixer, the mixer's sizes and constants as the file
    gives them (validated, with the optional keys resolved), and the feed-forward width (None: no feed-forward)."""

    kind: str                  # "attention", "mamba2" or "lightning"
    mixer: dict
    ff: int | None


@register_config("Sigosun")
@dataclass(frozen=True)
class SigosunConfig:
    """The ``config.json`` keys of the Sigosun design: a list of layers, each with its own mixer (softmax
    attention under a block mask, a selective state-space recurrence, or linear attention with fixed decays),
    sizes and constants, and an optional dense feed-forward; one norm eps; vocabulary and width. Every size
    and constant comes from the file: nothing of a particular model is assumed."""

    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: tuple
    eos_token_id: int | None = None
    max_position_embeddings: int | None = None

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    MIXER_KEYS = {
        "attention": (("heads", int), ("kv_heads", int), ("dim", int), ("vdim", int), ("scale", float)),
        "mamba2": (("heads", int), ("vdim", int), ("state", int), ("groups", int), ("conv", int), ("norm_groups", int)),
        "lightning": (("heads", int), ("dim", int), ("vdim", int)),
    }

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "SigosunConfig":
        norm = raw.get("norm")
        if not isinstance(norm, dict):
            raise ConfigError("config.json lacks the object 'norm'")
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json lacks the list 'layers'")
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]"
            kind = entry.get("type") if isinstance(entry, dict) else None
            if kind not in cls.MIXER_KEYS:
                raise ConfigError(f"{where}: 'type' must be one of {sorted(cls.MIXER_KEYS)}, got {kind!r}")
            m = entry.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"{where} lacks the object 'mixer'")
            mixer = {key: _need(m, key, typ, where + ".mixer") for key, typ in cls.MIXER_KEYS[kind]}
            if kind == "attention":
                rot, mask = m.get("rot"), m.get("mask")
                mixer["rot_dims"] = _need(rot, "dims", int, where + ".mixer.rot") if rot else 0
                mixer["rot_base"] = _need(rot, "base", float, where + ".mixer.rot") if rot else 1.0
                mixer["mask_size"] = _need(mask, "size", int, where + ".mixer.mask") if mask else None
                mixer["kv_from"] = m.get("kv_from")
            elif kind == "lightning":
                decay = m.get("decay")
                if not isinstance(decay, list) or len(decay) != mixer["heads"]:
                    raise ConfigError(f"{where}.mixer: 'decay' must list one number per head")
                mixer["decay"] = tuple(float(d) for d in decay)
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"{where}.mlp: only kind 'dense' is known, got {mlp.get('kind')!r}")
                ff = _need(mlp, "ff", int, where + ".mlp")
            layers.append(SigosunLayer(kind, mixer, ff))
        cfg = cls(vocab_size=_need(raw, "vocab", int), hidden_size=_need(raw, "width", int),
                  norm_eps=_need(norm, "eps", float, "config.json norm"), layers=tuple(layers),
                  eos_token_id=raw.get("eos_token_id"), max_position_embeddings=raw.get("max_position_embeddings"))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab_size < 1 or self.hidden_size < 1 or not self.norm_eps > 0:
            raise ConfigError("vocab and width must be positive and norm.eps above zero")
        for i, layer in enumerate(self.layers):
            m, where = layer.mixer, f"layers[{i}]"
            if any(isinstance(v, int) and not isinstance(v, bool) and v < 1 for k, v in m.items()
                   if k not in ("rot_dims", "kv_from", "mask_size")):
                raise ConfigError(f"{where}: sizes must be positive")
            if layer.kind == "attention":
                if m["heads"] % m["kv_heads"]:
                    raise ConfigError(f"{where}: {m['heads']} heads are not a multiple of {m['kv_heads']} kv_heads")
                if m["rot_dims"] % 2 or not 0 <= m["rot_dims"] <= m["dim"]:
                    raise ConfigError(f"{where}: rot.dims must be even and at most dim")
                if m["mask_size"] is not None and m["mask_size"] < 1:
                    raise ConfigError(f"{where}: mask.size must be positive")
                src = m["kv_from"]
                if src is not None:
                    if not (isinstance(src, int) and 0 <= src < i and self.layers[src].kind == "attention"
                            and self.layers[src].mixer["kv_from"] is None):
                        raise ConfigError(f"{where}: kv_from must name an earlier attention layer that has keys of its own")
                    o = self.layers[src].mixer
                    if any(o[k] != m[k] for k in ("kv_heads", "dim", "vdim")):
                        raise ConfigError(f"{where}: kv_from names a layer with other key/value sizes")
            elif layer.kind == "mamba2":
                if m["heads"] % m["groups"] or (m["heads"] * m["vdim"]) % m["norm_groups"]:
                    raise ConfigError(f"{where}: heads must be a multiple of groups, and heads * vdim of norm_groups")
            if layer.ff is not None and layer.ff < 1:
                raise ConfigError(f"{where}.mlp: ff must be positive")

    def to_dict(self) -> dict[str, Any]:
        """A ``config.json`` that reads back to an equal config."""
        out = []
        for layer in self.layers:
            m = dict(layer.mixer)
            if layer.kind == "attention":
                dims, base, size, src = m.pop("rot_dims"), m.pop("rot_base"), m.pop("mask_size"), m.pop("kv_from")
                if dims:
                    m["rot"] = {"dims": dims, "base": base}
                if size is not None:
                    m["mask"] = {"size": size}
                if src is not None:
                    m["kv_from"] = src
            elif layer.kind == "lightning":
                m["decay"] = list(m["decay"])
            out.append({"type": layer.kind, "mixer": m, "mlp": None if layer.ff is None else {"kind": "dense", "ff": layer.ff}})
        d = {"architecture": self.architecture_name, "vocab": self.vocab_size, "width": self.hidden_size,
             "norm": {"eps": self.norm_eps}, "layers": out}
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        if self.max_position_embeddings is not None:
            d["max_position_embeddings"] = self.max_position_embeddings
        return d

    def flat(self) -> dict[str, Any]:
        return {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size, "num_hidden_layers": len(self.layers),
                "layer_kinds": [layer.kind for layer in self.layers]}


# ------------------------------------------------------------------------------------ Negosun

@dataclass(frozen=True)
class NegosunLayer:
    """One entry of a Negosun config's `layers`: the mixer's sizes and constants (validated, optional keys resolved)
    and the feed-forward's (None: the layer has no feed-forward)."""

    kind: str                  # "attention"
    mixer: dict
    mlp: dict | None


@register_config("Negosun")
@dataclass(frozen=True)
class NegosunConfig:
    """The ``config.json`` keys of the Negosun design: layers whose mixer and feed-forward read the same stream side by
    side, each through a norm of its own, their outputs scaled element by element and added under one multiplier
    (`residual_mult`); attention with biases, q and k normed over the whole projection, a query temperature that grows
    with the logarithm of the position, and values blended with those of the first such layer (`v_mix`); a
    feed-forward of routed experts with an optional limit to the best groups and an optional shared expert; tied
    output weights and an optional soft cap on the logits. Every size and constant comes from the file."""

    vocab_size: int
    hidden_size: int
    norm_eps: float
    residual_mult: float
    logit_softcap: float | None
    layers: tuple
    eos_token_id: int | None = None
    max_position_embeddings: int | None = None

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "NegosunConfig":
        norm = raw.get("norm")
        if not isinstance(norm, dict):
            raise ConfigError("config.json lacks the object 'norm'")
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json lacks the list 'layers'")
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]"
            kind = entry.get("type") if isinstance(entry, dict) else None
            if kind != "attention":
                raise ConfigError(f"{where}: 'type' must be 'attention', got {kind!r}")
            m = entry.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"{where} lacks the object 'mixer'")
            mixer = {key: _need(m, key, typ, where + ".mixer")
                     for key, typ in (("heads", int), ("kv_heads", int), ("dim", int), ("vdim", int), ("scale", float))}
            temp = m.get("q_temp")
            mixer["temp_coef"] = _need(temp, "coef", float, where + ".mixer.q_temp") if temp else None
            mixer["temp_every"] = _need(temp, "every", int, where + ".mixer.q_temp") if temp else None
            mixer["v_mix"] = bool(m.get("v_mix", False))
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                if mlp.get("kind", "moe") != "moe":
                    raise ConfigError(f"{where}.mlp: only kind 'moe' is known, got {mlp.get('kind')!r}")
                router = mlp.get("router")
                if not isinstance(router, dict) or not isinstance(mlp.get("expert"), dict):
                    raise ConfigError(f"{where}.mlp lacks the objects 'router' and 'expert'")
                groups, shared = router.get("groups"), mlp.get("shared")
                ff = {"ff": _need(mlp["expert"], "ff", int, where + ".mlp.expert"),
                      "experts": _need(router, "experts", int, where + ".mlp.router"),
                      "top": _need(router, "top", int, where + ".mlp.router"),
                      "group_count": _need(groups, "count", int, where + ".mlp.router.groups") if groups else 1,
                      "group_keep": _need(groups, "keep", int, where + ".mlp.router.groups") if groups else 1,
                      "shared_ff": _need(shared, "ff", int, where + ".mlp.shared") if shared else None}
            layers.append(NegosunLayer(kind, mixer, ff))
        cap = raw.get("logit_softcap")
        cfg = cls(vocab_size=_need(raw, "vocab", int), hidden_size=_need(raw, "width", int),
                  norm_eps=_need(norm, "eps", float, "config.json norm"),
                  residual_mult=float(raw["residual_mult"]) if raw.get("residual_mult") is not None else 1.0,
                  logit_softcap=None if cap is None else float(cap), layers=tuple(layers),
                  eos_token_id=raw.get("eos_token_id"), max_position_embeddings=raw.get("max_position_embeddings"))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab_size < 1 or self.hidden_size < 1 or not self.norm_eps > 0:
            raise ConfigError("vocab and width must be positive and norm.eps above zero")
        if self.logit_softcap is not None and not self.logit_softcap > 0:
            raise ConfigError("logit_softcap must be positive")
        mixed = None
        for i, layer in enumerate(self.layers):
            m, where = layer.mixer, f"layers[{i}]"
            if any(m[k] < 1 for k in ("heads", "kv_heads", "dim", "vdim")):
                raise ConfigError(f"{where}: sizes must be positive")
            if m["heads"] % m["kv_heads"]:
                raise ConfigError(f"{where}: {m['heads']} heads are not a multiple of {m['kv_heads']} kv_heads")
            if m["temp_every"] is not None and m["temp_every"] < 1:
                raise ConfigError(f"{where}: q_temp.every must be positive")
            if m["v_mix"]:
                width = m["kv_heads"] * m["vdim"]
                if mixed is not None and width != mixed:
                    raise ConfigError(f"{where}: layers with v_mix must have equally many value dimensions ({width} against {mixed})")
                mixed = width
            f = layer.mlp
            if f is not None:
                if f["ff"] < 1 or f["experts"] < 1 or not 1 <= f["top"] <= f["experts"]:
                    raise ConfigError(f"{where}.mlp: sizes must be positive and top at most experts")
                if f["group_count"] < 1 or f["experts"] % f["group_count"] or not 1 <= f["group_keep"] <= f["group_count"]:
                    raise ConfigError(f"{where}.mlp: {f['experts']} experts do not form {f['group_count']} equal groups "
                                      f"of which {f['group_keep']} are kept")
                if f["group_keep"] * (f["experts"] // f["group_count"]) < f["top"]:
                    raise ConfigError(f"{where}.mlp: the kept groups hold fewer experts than a token uses")
                if f["shared_ff"] is not None and f["shared_ff"] < 1:
                    raise ConfigError(f"{where}.mlp.shared: ff must be positive")

    def to_dict(self) -> dict[str, Any]:
        """A ``config.json`` that reads back to an equal config."""
        out = []
        for layer in self.layers:
            m = {k: layer.mixer[k] for k in ("heads", "kv_heads", "dim", "vdim", "scale", "v_mix")}
            if layer.mixer["temp_every"] is not None:
                m["q_temp"] = {"coef": layer.mixer["temp_coef"], "every": layer.mixer["temp_every"]}
            f = layer.mlp
            mlp = None
            if f is not None:
                mlp = {"kind": "moe", "expert": {"ff": f["ff"]},
                       "router": {"experts": f["experts"], "top": f["top"], "groups": {"count": f["group_count"], "keep": f["group_keep"]}}}
                if f["shared_ff"] is not None:
                    mlp["shared"] = {"ff": f["shared_ff"]}
            out.append({"type": layer.kind, "mixer": m, "mlp": mlp})
        d = {"architecture": self.architecture_name, "vocab": self.vocab_size, "width": self.hidden_size,
             "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult, "layers": out}
        if self.logit_softcap is not None:
            d["logit_softcap"] = self.logit_softcap
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        if self.max_position_embeddings is not None:
            d["max_position_embeddings"] = self.max_position_embeddings
        return d

    def flat(self) -> dict[str, Any]:
        return {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size, "num_hidden_layers": len(self.layers),
                "experts": [None if layer.mlp is None else layer.mlp["experts"] for layer in self.layers]}


# ------------------------------------------------------------------------------------ Tavevik

@dataclass(frozen=True)
class TavevikLayer:
    """One entry of a Tavevik config's `layers`: the kind of its two-sided mixer, the sizes and constants of the left
    (attention) and the right (recurrent) side with the optional keys resolved, the two output scales, and the
    feed-forward's width and limit (None: the layer has no feed-forward)."""

    kind: str                  # "parallel" or "parallel_2"
    left: dict
    right: dict
    left_scale: float
    right_scale: float
    mlp: dict | None


@register_config("Tavevik")
@dataclass(frozen=True)
class TavevikConfig:
    """The ``config.json`` keys of the Tavevik design: layers whose mixer is softmax attention under a trailing window
    beside a recurrence over a matrix per head, their outputs added under two scales; the norms sit on the sublayers'
    outputs. Kind `parallel`: the attention keeps its first positions visible, bends its scores under a cap and gates
    its heads element by element; the recurrence mixes each token's input with the previous token's and has a bonus for
    the token itself. Kind `parallel_2`: the attention has biases and a sink per head; the recurrence is a delta rule
    behind short convolutions. A feed-forward with a clamped gated activation; tied output weights. Every size and
    constant comes from the file; the inner widths of the thin matrix pairs (`decay_rank`, `gate_rank`) come from the
    checkpoint's tensors when the file does not name them."""

    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: tuple
    eos_token_id: int | None = None
    max_position_embeddings: int | None = None

    KINDS = ("parallel", "parallel_2")

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "TavevikConfig":
        norm = raw.get("norm")
        if not isinstance(norm, dict):
            raise ConfigError("config.json lacks the object 'norm'")
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json lacks the list 'layers'")
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]"
            kind = entry.get("type") if isinstance(entry, dict) else None
            if kind not in cls.KINDS:
                raise ConfigError(f"{where}: 'type' must be one of {list(cls.KINDS)}, got {kind!r}")
            m = entry.get("mixer")
            if not isinstance(m, dict) or not isinstance(m.get("left"), dict) or not isinstance(m.get("right"), dict):
                raise ConfigError(f"{where} lacks the object 'mixer' with 'left' and 'right'")
            l, r = m["left"], m["right"]
            left = {key: _need(l, key, typ, where + ".mixer.left")
                    for key, typ in (("heads", int), ("kv_heads", int), ("dim", int), ("vdim", int), ("scale", float))}
            rot, mask = l.get("rot"), l.get("mask")
            left["rot_dims"] = _need(rot, "dims", int, where + ".mixer.left.rot") if rot else 0
            left["rot_base"] = _need(rot, "base", float, where + ".mixer.left.rot") if rot else 1.0
            left["window"] = _need(mask, "size", int, where + ".mixer.left.mask") if mask else None
            keep = mask.get("keep_first") if mask else None
            left["keep_first"] = int(keep) if (keep and kind == "parallel") else 0
            cap = l.get("softcap")
            left["softcap"] = float(cap) if (cap and kind == "parallel") else None
            right = {key: _need(r, key, int, where + ".mixer.right") for key in ("heads", "dim")}
            right["decay_rank"] = r.get("decay_rank")
            if kind == "parallel_2":
                for key in ("kv_heads", "vdim", "conv"):
                    right[key] = _need(r, key, int, where + ".mixer.right")
                right["gate_rank"] = r.get("gate_rank")
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"{where}.mlp: only kind 'dense' is known, got {mlp.get('kind')!r}")
                ff = {"ff": _need(mlp, "ff", int, where + ".mlp"), "limit": _need(mlp, "limit", float, where + ".mlp")}
            layers.append(TavevikLayer(kind, left, right, float(m.get("left_scale", 1.0)), float(m.get("right_scale", 1.0)), ff))
        cfg = cls(vocab_size=_need(raw, "vocab", int), hidden_size=_need(raw, "width", int),
                  norm_eps=_need(norm, "eps", float, "config.json norm"), layers=tuple(layers),
                  eos_token_id=raw.get("eos_token_id"), max_position_embeddings=raw.get("max_position_embeddings"))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab_size < 1 or self.hidden_size < 1 or not self.norm_eps > 0:
            raise ConfigError("vocab and width must be positive and norm.eps above zero")
        for i, layer in enumerate(self.layers):
            l, r, where = layer.left, layer.right, f"layers[{i}]"
            if any(l[k] < 1 for k in ("heads", "kv_heads", "dim", "vdim")) or any(r[k] < 1 for k in r if isinstance(r[k], int)):
                raise ConfigError(f"{where}: sizes must be positive")
            if l["heads"] % l["kv_heads"]:
                raise ConfigError(f"{where}: {l['heads']} heads are not a multiple of {l['kv_heads']} kv_heads")
            if l["rot_dims"] % 2 or not 0 <= l["rot_dims"] <= l["dim"]:
                raise ConfigError(f"{where}: rot.dims must be even and at most dim")
            if l["window"] is not None and l["window"] < 1:
                raise ConfigError(f"{where}: mask.size must be positive")
            if l["keep_first"] < 0 or (l["keep_first"] and l["window"] is None):
                raise ConfigError(f"{where}: mask.keep_first needs mask.size and must not be negative")
            if l["softcap"] is not None and not l["softcap"] > 0:
                raise ConfigError(f"{where}: softcap must be positive")
            if layer.kind == "parallel_2" and r["heads"] % r["kv_heads"]:
                raise ConfigError(f"{where}: the right side's {r['heads']} heads are not a multiple of its {r['kv_heads']} kv_heads")
            if layer.mlp is not None and (layer.mlp["ff"] < 1 or not layer.mlp["limit"] > 0):
                raise ConfigError(f"{where}.mlp: ff and limit must be positive")

    def to_dict(self) -> dict[str, Any]:
        """A ``config.json`` that reads back to an equal config."""
        out = []
        for layer in self.layers:
            l = {k: layer.left[k] for k in ("heads", "kv_heads", "dim", "vdim", "scale")}
            if layer.left["rot_dims"]:
                l["rot"] = {"dims": layer.left["rot_dims"], "base": layer.left["rot_base"]}
            if layer.left["window"] is not None:
                l["mask"] = {"size": layer.left["window"]}
                if layer.left["keep_first"]:
                    l["mask"]["keep_first"] = layer.left["keep_first"]
            if layer.left["softcap"] is not None:
                l["softcap"] = layer.left["softcap"]
            r = {k: v for k, v in layer.right.items() if v is not None}
            mlp = None if layer.mlp is None else {"kind": "dense", "ff": layer.mlp["ff"], "limit": layer.mlp["limit"]}
            out.append({"type": layer.kind, "mixer": {"left": l, "right": r, "left_scale": layer.left_scale,
                                                      "right_scale": layer.right_scale}, "mlp": mlp})
        d = {"architecture": self.architecture_name, "vocab": self.vocab_size, "width": self.hidden_size,
             "norm": {"eps": self.norm_eps}, "layers": out}
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        if self.max_position_embeddings is not None:
            d["max_position_embeddings"] = self.max_position_embeddings
        return d

    def flat(self) -> dict[str, Any]:
        return {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size, "num_hidden_layers": len(self.layers),
                "layer_kinds": [layer.kind for layer in self.layers]}


# ------------------------------------------------------------------------------------ Goluzen
@dataclass(frozen=True)
class GoluzenLayer:
    """One entry of a Goluzen config's `layers`: which mixer it has, the mixer's sizes and constants with the optional
    keys resolved, and the feed-forward's (None: the layer has no feed-forward)."""

    kind: str                  # "attention", "latent_attention" or "gla"
    mixer: dict
    mlp: dict | None


def _scaling(rot: dict | None, kind: str, where: str) -> dict | None:
    """`rot.scaling` as the rotary encoding takes it: {"kind": "linear" | "yarn", ...} or None."""
    sc = rot.get("scaling") if rot else None
    if not sc:
        return None
    out = {"kind": kind, "factor": _need(sc, "factor", float, where)}
    if kind == "yarn":
        out["original"] = _need(sc, "original", float, where)
        out["fast"] = _need(sc, "fast", float, where)
        out["slow"] = _need(sc, "slow", float, where)
    return out


@register_config("Goluzen")
@dataclass(frozen=True)
class GoluzenConfig:
    """The ``config.json`` keys of the Goluzen design: pre-norm layers (norm weights stored around zero) that each name
    their mixer. `attention`: grouped heads with biases on q, k and v, a rotation of the first dimensions of each head
    (pairs half the rotating width apart) whose rates are divided by a factor, q and k at unit root mean square, scores
    bent under a cap, a trailing window that keeps the first positions visible, a sink per head. `latent_attention`:
    keys and values made head by head from a cached latent and one shared rotated key part (adjacent pairs, YaRN
    scaling), a trailing window, a gate on the heads' outputs; with `kv_from` the latent of an earlier layer. `gla`:
    linear attention with a decay per key channel from a thin matrix pair (`decay_rank` comes from the checkpoint's
    tensors when the file does not name it). Feed-forwards: dense with the tanh form of gelu, or routed experts without
    gates (sigmoid scores, a correction for the choice, groups scored by their two best, weights times a constant)
    beside an optional shared expert under a gate per token. The embedding's rows are multiplied by `embedding.scale`;
    the head has weights of its own. Every size and constant comes from the file."""

    vocab_size: int
    hidden_size: int
    norm_eps: float
    embedding_scale: float
    layers: tuple
    eos_token_id: int | None = None
    max_position_embeddings: int | None = None

    KINDS = ("attention", "latent_attention", "gla")

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "GoluzenConfig":
        norm = raw.get("norm")
        if not isinstance(norm, dict):
            raise ConfigError("config.json lacks the object 'norm'")
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json lacks the list 'layers'")
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]"
            kind = entry.get("type") if isinstance(entry, dict) else None
            if kind not in cls.KINDS:
                raise ConfigError(f"{where}: 'type' must be one of {list(cls.KINDS)}, got {kind!r}")
            m = entry.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"{where} lacks the object 'mixer'")
            at = where + ".mixer"
            rot, mask = m.get("rot"), m.get("mask")
            if kind == "attention":
                mixer = {key: _need(m, key, typ, at) for key, typ in (("heads", int), ("dim", int), ("vdim", int), ("scale", float))}
                mixer["kv_heads"] = _need(m, "kv_heads", int, at) if m.get("kv_heads") is not None else mixer["heads"]
                mixer["rot_dims"] = _need(rot, "dims", int, at + ".rot") if rot else 0
                mixer["rot_base"] = _need(rot, "base", float, at + ".rot") if rot else 1.0
                mixer["rot_scaling"] = _scaling(rot, "linear", at + ".rot.scaling")
                mixer["window"] = _need(mask, "size", int, at + ".mask") if mask else None
                mixer["keep_first"] = int(mask.get("keep_first") or 0) if mask else 0
                mixer["softcap"] = float(m["softcap"]) if m.get("softcap") else None
            elif kind == "latent_attention":
                mixer = {key: _need(m, key, typ, at) for key, typ in (("heads", int), ("dim", int), ("rot_dim", int), ("vdim", int),
                                                                       ("kv_rank", int), ("scale", float))}
                mixer["rot_base"] = _need(rot, "base", float, at + ".rot") if rot else 1.0
                if rot and rot.get("dims") is not None and int(rot["dims"]) != mixer["rot_dim"]:
                    raise ConfigError(f"{at}: rot.dims must equal rot_dim")
                mixer["rot_scaling"] = _scaling(rot, "yarn", at + ".rot.scaling")
                mixer["window"] = _need(mask, "size", int, at + ".mask") if mask else None
                mixer["kv_from"] = _need(m, "kv_from", int, at) if m.get("kv_from") is not None else None
            else:
                mixer = {key: _need(m, key, typ, at) for key, typ in (("heads", int), ("dim", int), ("vdim", int), ("tau", float))}
                mixer["decay_rank"] = m.get("decay_rank")
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                fkind = mlp.get("kind")
                if fkind == "dense":
                    ff = {"kind": "dense", "ff": _need(mlp, "ff", int, where + ".mlp")}
                elif fkind == "moe":
                    router = mlp.get("router")
                    if not isinstance(router, dict) or not isinstance(mlp.get("expert"), dict):
                        raise ConfigError(f"{where}.mlp lacks the objects 'router' and 'expert'")
                    groups, shared = router.get("groups"), mlp.get("shared")
                    ff = {"kind": "moe", "ff": _need(mlp["expert"], "ff", int, where + ".mlp.expert"),
                          "experts": _need(router, "experts", int, where + ".mlp.router"),
                          "top": _need(router, "top", int, where + ".mlp.router"),
                          "scale": float(router["scale"]) if router.get("scale") is not None else 1.0,
                          "group_count": _need(groups, "count", int, where + ".mlp.router.groups") if groups else 1,
                          "group_keep": _need(groups, "keep", int, where + ".mlp.router.groups") if groups else 1,
                          "shared_ff": _need(shared, "ff", int, where + ".mlp.shared") if shared else None}
                else:
                    raise ConfigError(f"{where}.mlp: 'kind' must be 'dense' or 'moe', got {fkind!r}")
            layers.append(GoluzenLayer(kind, mixer, ff))
        emb = raw.get("embedding") or {}
        cfg = cls(vocab_size=_need(raw, "vocab", int), hidden_size=_need(raw, "width", int),
                  norm_eps=_need(norm, "eps", float, "config.json norm"),
                  embedding_scale=float(emb["scale"]) if emb.get("scale") is not None else 1.0, layers=tuple(layers),
                  eos_token_id=raw.get("eos_token_id"), max_position_embeddings=raw.get("max_position_embeddings"))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab_size < 1 or self.hidden_size < 1 or not self.norm_eps > 0:
            raise ConfigError("vocab and width must be positive and norm.eps above zero")
        for i, layer in enumerate(self.layers):
            m, where = layer.mixer, f"layers[{i}]"
            if any(v < 1 for k, v in m.items() if k in ("heads", "kv_heads", "dim", "vdim", "kv_rank")) or not m.get("scale", 1.0) > 0:
                raise ConfigError(f"{where}: sizes and the score scale must be positive")
            if m.get("window") is not None and m["window"] < 1:
                raise ConfigError(f"{where}: mask.size must be positive")
            if layer.kind == "attention":
                if m["heads"] % m["kv_heads"]:
                    raise ConfigError(f"{where}: {m['heads']} heads are not a multiple of {m['kv_heads']} kv_heads")
                if m["rot_dims"] % 2 or not 0 <= m["rot_dims"] <= m["dim"]:
                    raise ConfigError(f"{where}: rot.dims must be even and at most dim")
                if m["keep_first"] < 0 or (m["keep_first"] and m["window"] is None):
                    raise ConfigError(f"{where}: mask.keep_first needs mask.size and must not be negative")
                if m["softcap"] is not None and not m["softcap"] > 0:
                    raise ConfigError(f"{where}: softcap must be positive")
            elif layer.kind == "latent_attention":
                if m["rot_dim"] < 0 or m["rot_dim"] % 2:
                    raise ConfigError(f"{where}: rot_dim must be even")
                src = m["kv_from"]
                if src is not None:
                    if not 0 <= src < i or self.layers[src].kind != "latent_attention" or self.layers[src].mixer["kv_from"] is not None:
                        raise ConfigError(f"{where}: kv_from must name an earlier latent_attention layer that makes its own latent")
                    theirs = self.layers[src].mixer
                    if any(theirs[k] != m[k] for k in ("kv_rank", "rot_dim", "rot_base", "rot_scaling")):
                        raise ConfigError(f"{where}: the layer named by kv_from has another latent size or rotation")
            else:
                if not m["tau"] > 0 or (m["decay_rank"] is not None and int(m["decay_rank"]) < 1):
                    raise ConfigError(f"{where}: tau and decay_rank must be positive")
            for sc in (m.get("rot_scaling"),):
                if sc is not None and (not sc["factor"] > 0 or (sc["kind"] == "yarn" and not (sc["original"] > 0 and sc["fast"] > 0 and sc["slow"] > 0))):
                    raise ConfigError(f"{where}: rot.scaling's numbers must be positive")
            f = layer.mlp
            if f is not None and f["ff"] < 1:
                raise ConfigError(f"{where}.mlp: ff must be positive")
            if f is not None and f["kind"] == "moe":
                if f["experts"] < 1 or not 1 <= f["top"] <= f["experts"]:
                    raise ConfigError(f"{where}.mlp: experts must be positive and top at most experts")
                if f["group_count"] < 1 or f["experts"] % f["group_count"] or not 1 <= f["group_keep"] <= f["group_count"]:
                    raise ConfigError(f"{where}.mlp: {f['experts']} experts do not form {f['group_count']} equal groups "
                                      f"of which {f['group_keep']} are kept")
                if f["group_keep"] * (f["experts"] // f["group_count"]) < f["top"]:
                    raise ConfigError(f"{where}.mlp: the kept groups hold fewer experts than a token uses")
                if f["shared_ff"] is not None and f["shared_ff"] < 1:
                    raise ConfigError(f"{where}.mlp.shared: ff must be positive")

    def to_dict(self) -> dict[str, Any]:
        """A ``config.json`` that reads back to an equal config."""
        def scaling(sc):
            return {k: v for k, v in sc.items() if k != "kind"}

        out = []
        for layer in self.layers:
            x = layer.mixer
            if layer.kind == "attention":
                m = {k: x[k] for k in ("heads", "kv_heads", "dim", "vdim", "scale")}
                if x["rot_dims"]:
                    m["rot"] = {"dims": x["rot_dims"], "base": x["rot_base"]}
                    if x["rot_scaling"]:
                        m["rot"]["scaling"] = scaling(x["rot_scaling"])
                if x["window"] is not None:
                    m["mask"] = {"size": x["window"]}
                    if x["keep_first"]:
                        m["mask"]["keep_first"] = x["keep_first"]
                if x["softcap"] is not None:
                    m["softcap"] = x["softcap"]
            elif layer.kind == "latent_attention":
                m = {k: x[k] for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale")}
                m["rot"] = {"dims": x["rot_dim"], "base": x["rot_base"]}
                if x["rot_scaling"]:
                    m["rot"]["scaling"] = scaling(x["rot_scaling"])
                if x["window"] is not None:
                    m["mask"] = {"size": x["window"]}
                if x["kv_from"] is not None:
                    m["kv_from"] = x["kv_from"]
            else:
                m = {k: x[k] for k in ("heads", "dim", "vdim", "tau")}
                if x["decay_rank"] is not None:
                    m["decay_rank"] = x["decay_rank"]
            f = layer.mlp
            mlp = None
            if f is not None and f["kind"] == "dense":
                mlp = {"kind": "dense", "ff": f["ff"]}
            elif f is not None:
                mlp = {"kind": "moe", "expert": {"ff": f["ff"]},
                       "router": {"experts": f["experts"], "top": f["top"], "scale": f["scale"],
                                  "groups": {"count": f["group_count"], "keep": f["group_keep"]}}}
                if f["shared_ff"] is not None:
                    mlp["shared"] = {"ff": f["shared_ff"]}
            out.append({"type": layer.kind, "mixer": m, "mlp": mlp})
        d = {"architecture": self.architecture_name, "vocab": self.vocab_size, "width": self.hidden_size,
             "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale}, "layers": out}
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        if self.max_position_embeddings is not None:
            d["max_position_embeddings"] = self.max_position_embeddings
        return d

    def flat(self) -> dict[str, Any]:
        return {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size, "num_hidden_layers": len(self.layers),
                "layer_kinds": [layer.kind for layer in self.layers]}
