"""Typed model configurations read from an architecture's own config.json keys.

The Qwen3 fields, their defaults and their types follow the reference's
``ModelConfig`` (src/models/model_config.hpp:7-47).  Unlike the reference,
which never consults ``model_type``/``hidden_act`` and wires the model class in
code (src/engine/model_runner.hpp:21), every value is validated here and the
model class is looked up by ``architectures[0]``.
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Any, ClassVar, Dict, List, Optional


class ConfigError(ValueError):
    """A config.json that this engine cannot run, with the reason."""


@dataclasses.dataclass
class ModelConfig:
    """Base of all architecture configurations.

    A subclass lists its config.json keys as dataclass fields (the field name is
    the key), gives defaults where the architecture defines them, and checks
    consistency in ``validate``.
    """

    architectures: List[str] = dataclasses.field(default_factory=list)

    #: keys that must be present in config.json
    required: ClassVar[tuple] = ()

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "ModelConfig":
        missing = [k for k in cls.required if k not in raw]
        if missing:
            raise ConfigError("config.json lacks required key(s): " + ", ".join(missing))
        known = {f.name: f for f in dataclasses.fields(cls)}
        kwargs = {}
        for name, field in known.items():
            if name not in raw or raw[name] is None:
                continue
            kwargs[name] = _coerce(name, raw[name], field.type)
        cfg = cls(**kwargs)
        cfg._raw = dict(raw)
        cfg.fill_defaults()
        cfg.validate()
        return cfg

    @classmethod
    def from_json(cls, path: str) -> "ModelConfig":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        with open(path) as f:
            return cls.from_dict(json.load(f))

    def to_dict(self) -> Dict[str, Any]:
        return {f.name: getattr(self, f.name) for f in dataclasses.fields(self)}

    def fill_defaults(self) -> None:
        pass

    def validate(self) -> None:
        pass

    # What the engine itself asks of any architecture's configuration, whatever its config.json keys are called.
    @property
    def position_limit(self) -> Optional[int]:
        """Most tokens a request may reach (the architecture's positions end there); None = no limit."""
        return None

    @property
    def end_token_id(self) -> Optional[int]:
        """The token at which generation ends; None = the architecture names none."""
        return None


def _coerce(name, value, type_name):
    t = str(type_name)
    try:
        if t in ("int", "<class 'int'>"):
            if isinstance(value, bool) or (isinstance(value, float) and value != int(value)):
                raise TypeError
            if isinstance(value, (list, dict, str)):
                raise TypeError
            return int(value)
        if t in ("float", "<class 'float'>"):
            if isinstance(value, (bool, list, dict, str)):
                raise TypeError
            return float(value)
        if t in ("bool", "<class 'bool'>"):
            if not isinstance(value, bool):
                raise TypeError
            return value
        if t in ("str", "<class 'str'>"):
            if not isinstance(value, str):
                raise TypeError
            return value
    except (TypeError, ValueError):
        raise ConfigError("config.json key %r has value %r, expected %s" % (name, value, t)) from None
    return value


@dataclasses.dataclass
class Qwen3Config(ModelConfig):
    """Qwen3 dense decoder.  Keys and defaults: src/models/model_config.hpp:32-46."""

    model_type: str = ""
    hidden_act: str = ""
    hidden_size: int = -1
    intermediate_size: int = -1
    num_key_value_heads: int = -1
    num_hidden_layers: int = -1
    num_attention_heads: int = -1
    tie_word_embeddings: bool = False
    rope_theta: float = 1000000.0
    rms_norm_eps: float = 1e-6
    head_dim: int = -1  # falls back to hidden_size / num_attention_heads (model_config.hpp:42)
    bos_token_id: int = -1
    eos_token_id: int = -1
    max_position_embeddings: int = 16384
    vocab_size: int = -1

    required: ClassVar[tuple] = ("model_type", "hidden_act")

    @property
    def position_limit(self):
        return self.max_position_embeddings

    @property
    def end_token_id(self):
        return self.eos_token_id if self.eos_token_id >= 0 else None

    def fill_defaults(self) -> None:
        if self.head_dim == -1 and self.num_attention_heads > 0:
            self.head_dim = self.hidden_size // self.num_attention_heads

    def validate(self) -> None:
        raw = getattr(self, "_raw", {})
        for name in ("hidden_size", "intermediate_size", "num_key_value_heads", "num_hidden_layers",
                     "num_attention_heads", "head_dim", "max_position_embeddings", "vocab_size"):
            if getattr(self, name) <= 0:
                raise ConfigError("config.json: %s must be a positive integer, got %r" % (name, getattr(self, name)))
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError("config.json: num_attention_heads (%d) is not a multiple of num_key_value_heads (%d)"
                              % (self.num_attention_heads, self.num_key_value_heads))
        if self.head_dim % 2 != 0:
            raise ConfigError("config.json: head_dim (%d) must be even for rotary pairs" % self.head_dim)
        # The reference fixes SiLU in code (src/backends/cpu/x64/kernels.cpp:224-247) and never reads hidden_act.
        if self.hidden_act != "silu":
            raise ConfigError("config.json: hidden_act %r is not supported (the architecture uses 'silu')" % self.hidden_act)
        if not (self.rms_norm_eps > 0.0):
            raise ConfigError("config.json: rms_norm_eps must be positive")
        if not (self.rope_theta > 0.0):
            raise ConfigError("config.json: rope_theta must be positive")
        # Options that the reference does not implement are refused rather than silently ignored.
        if raw.get("attention_bias"):
            raise ConfigError("config.json: attention_bias is set, but this architecture has no projection biases "
                              "(src/models/qwen3.hpp:39)")
        if raw.get("rope_scaling") not in (None, {}):
            raise ConfigError("config.json: rope_scaling is not supported (src/utils/constant_table.hpp:28-41 has no scaling)")
        if raw.get("use_sliding_window"):
            raise ConfigError("config.json: use_sliding_window is set, but this architecture attends to all keys "
                              "(src/backends/cpu/cpu_attention.cpp:98-111)")


def _need(raw: Dict[str, Any], path: str, kinds, where: str = "config.json"):
    """raw[a][b][c] for path "a.b.c", checked for presence and type."""
    node = raw
    for key in path.split("."):
        if not isinstance(node, dict) or key not in node or node[key] is None:
            raise ConfigError("%s lacks %r" % (where, path))
        node = node[key]
    if isinstance(node, bool) or not isinstance(node, kinds):
        raise ConfigError("%s: %r has value %r of the wrong type" % (where, path, node))
    return node


@dataclasses.dataclass
class SefevikConfig(ModelConfig):
    """Sefevik: layers that add the norm of a sublayer's output to the stream and hand on a learned mix of all layer
    results so far; token mixers 'mingru' (a gated recurrence) and 'latent_attention' (keys and values expanded from a
    low-rank vector per token, rotated shared key part, window, sink); an embedding with a hashed pair table.  The
    configuration is nested; ``layers`` lists every layer's type and sizes, and nothing is assumed equal between
    layers."""

    architecture: str = ""
    vocab: int = -1
    width: int = -1
    norm_eps: float = 0.0
    #: pair table of the embedding: rows (without the first-token row), multipliers of the previous and the current id;
    #: buckets == 0: the model has none
    bigram_buckets: int = 0
    bigram_mul_prev: int = 0
    bigram_mul_cur: int = 0
    #: one dict per layer: type, mixer (sizes and constants of that mixer), mlp (None or {kind, ff})
    layers: List[Dict[str, Any]] = dataclasses.field(default_factory=list)

    MIXERS: ClassVar[tuple] = ("mingru", "latent_attention")

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "SefevikConfig":
        cfg = cls(architecture=str(raw.get("architecture") or (raw.get("architectures") or [""])[0]),
                  vocab=_need(raw, "vocab", int), width=_need(raw, "width", int), norm_eps=float(_need(raw, "norm.eps", (int, float))))
        pair = (raw.get("embedding") or {}).get("bigram")
        if pair:
            cfg.bigram_buckets = _need(pair, "buckets", int, "config.json embedding.bigram")
            cfg.bigram_mul_prev = _need(pair, "mul_prev", int, "config.json embedding.bigram")
            cfg.bigram_mul_cur = _need(pair, "mul_cur", int, "config.json embedding.bigram")
        layers = _need(raw, "layers", list)
        cfg.layers = [cls._layer(i, l) for i, l in enumerate(layers)]
        cfg._raw = dict(raw)
        cfg.validate()
        return cfg

    @classmethod
    def _layer(cls, i: int, raw: Dict[str, Any]) -> Dict[str, Any]:
        where = "config.json layers[%d]" % i
        if not isinstance(raw, dict):
            raise ConfigError("%s is no object" % where)
        kind = _need(raw, "type", str, where)
        if kind not in cls.MIXERS:
            raise ConfigError("%s: mixer type %r is not known (%s)" % (where, kind, ", ".join(cls.MIXERS)))
        m = _need(raw, "mixer", dict, where)
        out = {"type": kind, "mlp": None}
        if kind == "mingru":
            out["mixer"] = {"width": _need(m, "width", int, where + ".mixer")}
        else:
            mix = {k: _need(m, k, int, where + ".mixer") for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank")}
            mix["scale"] = float(_need(m, "scale", (int, float), where + ".mixer"))
            mix["kv_from"] = _need(m, "kv_from", int, where + ".mixer") if m.get("kv_from") is not None else None
            mix["window"] = _need(m, "mask.size", int, where + ".mixer") if m.get("mask") else None
            rot = m.get("rot")
            if rot:
                mix["rot"] = {"base": float(_need(rot, "base", (int, float), where + ".mixer.rot")),
                              "dims": _need(rot, "dims", int, where + ".mixer.rot") if rot.get("dims") is not None else mix["rot_dim"],
                              "scaling": None}
                sc = rot.get("scaling")
                if sc:
                    mix["rot"]["scaling"] = {k: float(_need(sc, k, (int, float), where + ".mixer.rot.scaling"))
                                             for k in ("factor", "original", "fast", "slow")}
            else:
                mix["rot"] = None
            out["mixer"] = mix
        mlp = raw.get("mlp")
        if mlp is not None:
            kind = _need(mlp, "kind", str, where + ".mlp")
            if kind != "dense":
                raise ConfigError("%s.mlp: kind %r is not known (dense)" % (where, kind))
            out["mlp"] = {"kind": kind, "ff": _need(mlp, "ff", int, where + ".mlp")}
        return out

    def to_dict(self) -> Dict[str, Any]:
        return dict(getattr(self, "_raw", {}))

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("config.json: vocab and width must be positive")
        if not (self.norm_eps > 0.0):
            raise ConfigError("config.json: norm.eps must be positive")
        if self.bigram_buckets < 0:
            raise ConfigError("config.json: embedding.bigram.buckets must be positive")
        if not self.layers:
            raise ConfigError("config.json: no layers")
        for i, layer in enumerate(self.layers):
            m = layer["mixer"]
            if any(isinstance(v, int) and not isinstance(v, bool) and v <= 0 for k, v in m.items() if k not in ("kv_from", "dim")):
                raise ConfigError("config.json layers[%d].mixer: sizes must be positive" % i)
            if layer["mlp"] and layer["mlp"]["ff"] <= 0:
                raise ConfigError("config.json layers[%d].mlp.ff must be positive" % i)
            if layer["type"] != "latent_attention":
                continue
            if m["dim"] < 0:
                raise ConfigError("config.json layers[%d].mixer.dim must not be negative" % i)
            rot = m["rot"]
            if rot and (rot["dims"] % 2 or not (0 < rot["dims"] <= m["rot_dim"]) or not rot["base"] > 1.0):
                raise ConfigError("config.json layers[%d].mixer.rot: dims must be even and at most rot_dim, base above 1" % i)
            src = m["kv_from"]
            if src is not None:
                if not (0 <= src < i) or self.layers[src]["type"] != "latent_attention" or self.layers[src]["mixer"]["kv_from"] is not None:
                    raise ConfigError("config.json layers[%d].mixer.kv_from = %r must name an earlier latent_attention layer "
                                      "with a projection of its own" % (i, src))
                other = self.layers[src]["mixer"]
                if (other["kv_rank"], other["rot_dim"], other["rot"]) != (m["kv_rank"], m["rot_dim"], m["rot"]):
                    raise ConfigError("config.json layers[%d].mixer: kv_rank, rot_dim and rot must equal those of layer %d, "
                                      "whose cache it reads" % (i, src))


@dataclasses.dataclass
class SodedraConfig(ModelConfig):
    """Sodedra: layers whose two sublayers read one norm of the stream (weights stored around zero) and are added
    together; token mixers 'mlstm' (a matrix memory with exponential gates), 'attention' (grouped queries, projection
    biases, heads rotated in part with frequencies rescaled by wavelength, a sliding window, a sigmoid gate on the
    result) and 'channel_delta' (a gated delta rule with short convolutions and a decay per key channel); feed-forwards
    'dense' (gated) or 'moe' (a mixture of gated experts chosen among the best groups); a scaled embedding whose table is
    also the output head.  The configuration is nested; ``layers`` lists every layer's type and sizes, and nothing is
    assumed equal between layers."""

    architecture: str = ""
    vocab: int = -1
    width: int = -1
    norm_eps: float = 0.0
    embedding_scale: float = 1.0
    #: one dict per layer: type, mixer (sizes and constants of that mixer), mlp (None, {kind: dense, ff} or
    #: {kind: moe, ff, experts, top, groups, keep, scale})
    layers: List[Dict[str, Any]] = dataclasses.field(default_factory=list)

    MIXERS: ClassVar[tuple] = ("mlstm", "attention", "channel_delta")

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "SodedraConfig":
        cfg = cls(architecture=str(raw.get("architecture") or (raw.get("architectures") or [""])[0]),
                  vocab=_need(raw, "vocab", int), width=_need(raw, "width", int), norm_eps=float(_need(raw, "norm.eps", (int, float))))
        if (raw.get("embedding") or {}).get("scale") is not None:
            cfg.embedding_scale = float(_need(raw, "embedding.scale", (int, float)))
        cfg.layers = [cls._layer(i, l) for i, l in enumerate(_need(raw, "layers", list))]
        cfg._raw = dict(raw)
        cfg.validate()
        return cfg

    @classmethod
    def _layer(cls, i: int, raw: Dict[str, Any]) -> Dict[str, Any]:
        where = "config.json layers[%d]" % i
        if not isinstance(raw, dict):
            raise ConfigError("%s is no object" % where)
        kind = _need(raw, "type", str, where)
        if kind not in cls.MIXERS:
            raise ConfigError("%s: mixer type %r is not known (%s)" % (where, kind, ", ".join(cls.MIXERS)))
        m = _need(raw, "mixer", dict, where)
        at = where + ".mixer"
        if kind == "mlstm":
            mix = {k: _need(m, k, int, at) for k in ("heads", "dim", "vdim")}
            mix["gate_cap"] = float(_need(m, "gate_cap", (int, float), at))
        elif kind == "attention":
            mix = {k: _need(m, k, int, at) for k in ("heads", "dim", "vdim")}
            mix["kv_heads"] = _need(m, "kv_heads", int, at) if m.get("kv_heads") is not None else mix["heads"]
            mix["scale"] = float(_need(m, "scale", (int, float), at))
            mix["window"] = _need(m, "mask.size", int, at) if m.get("mask") else None
            rot = m.get("rot")
            mix["rot"] = None
            if rot:
                mix["rot"] = {"base": float(_need(rot, "base", (int, float), at + ".rot")), "dims": _need(rot, "dims", int, at + ".rot"),
                              "scaling": None}
                sc = rot.get("scaling")
                if sc:
                    mix["rot"]["scaling"] = {k: float(_need(sc, k, (int, float), at + ".rot.scaling")) for k in ("factor", "low", "high", "original")}
        else:
            mix = {k: _need(m, k, int, at) for k in ("heads", "dim", "vdim", "conv")}
            mix["kv_heads"] = _need(m, "kv_heads", int, at) if m.get("kv_heads") is not None else mix["heads"]
            # inner sizes of the low-rank projections: no key of the design; the stored tensors decide unless these are given
            for k in ("decay_rank", "gate_rank"):
                mix[k] = _need(m, k, int, at) if m.get(k) is not None else None
        out = {"type": kind, "mixer": mix, "mlp": None}
        mlp = raw.get("mlp")
        if mlp is not None:
            at = where + ".mlp"
            fk = _need(mlp, "kind", str, at)
            if fk == "dense":
                out["mlp"] = {"kind": fk, "ff": _need(mlp, "ff", int, at)}
            elif fk == "moe":
                groups = (mlp.get("router") or {}).get("groups")
                out["mlp"] = {"kind": fk, "ff": _need(mlp, "expert.ff", int, at), "experts": _need(mlp, "router.experts", int, at),
                              "top": _need(mlp, "router.top", int, at),
                              "groups": _need(groups, "count", int, at + ".router.groups") if groups else 1,
                              "keep": _need(groups, "keep", int, at + ".router.groups") if groups else 1,
                              "scale": float(_need(mlp, "router.scale", (int, float), at)) if (mlp.get("router") or {}).get("scale") is not None else 1.0}
            else:
                raise ConfigError("%s: kind %r is not known (dense, moe)" % (at, fk))
        return out

    def to_dict(self) -> Dict[str, Any]:
        return dict(getattr(self, "_raw", {}))

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("config.json: vocab and width must be positive")
        if not (self.norm_eps > 0.0):
            raise ConfigError("config.json: norm.eps must be positive")
        if not self.layers:
            raise ConfigError("config.json: no layers")
        for i, layer in enumerate(self.layers):
            m, where = layer["mixer"], "config.json layers[%d]" % i
            if any(isinstance(v, int) and not isinstance(v, bool) and v <= 0 for v in m.values()):
                raise ConfigError("%s.mixer: sizes must be positive" % where)
            if "kv_heads" in m and m["heads"] % m["kv_heads"]:
                raise ConfigError("%s.mixer: heads (%d) is not a multiple of kv_heads (%d)" % (where, m["heads"], m["kv_heads"]))
            if layer["type"] == "mlstm" and not m["gate_cap"] > 0.0:
                raise ConfigError("%s.mixer.gate_cap must be positive" % where)
            if layer["type"] == "channel_delta" and m["conv"] > 8:
                raise ConfigError("%s.mixer.conv: at most 8 taps" % where)
            if layer["type"] == "attention" and m["rot"]:
                rot = m["rot"]
                if rot["dims"] % 2 or not (0 < rot["dims"] <= m["dim"]) or not rot["base"] > 1.0:
                    raise ConfigError("%s.mixer.rot: dims must be even and at most dim, base above 1" % where)
                sc = rot["scaling"]
                if sc and not (sc["factor"] > 0.0 and sc["original"] > 0.0 and 0.0 < sc["low"] <= sc["high"]):
                    raise ConfigError("%s.mixer.rot.scaling: factor and original positive, 0 < low <= high" % where)
            f = layer["mlp"]
            if f and f["ff"] <= 0:
                raise ConfigError("%s.mlp: the inner size must be positive" % where)
            if f and f["kind"] == "moe":
                E, G = f["experts"], f["groups"]
                if E <= 0 or G <= 0 or E % G or not 0 < f["keep"] <= G or not 0 < f["top"] <= f["keep"] * (E // G):
                    raise ConfigError("%s.mlp.router: %d choices among %d of %d groups of %d experts cannot be made"
                                      % (where, f["top"], f["keep"], G, E))


@dataclasses.dataclass
class MeronexConfig(ModelConfig):
    """Meronex: pre-norm layers whose sublayers' results are multiplied by a sigmoid gate of the sublayer's input and by a
    constant before they meet the stream; norms over consecutive groups of the vector; token mixers 'mlstm' (a matrix
    memory with exponential gates), 'delta' (a gated delta rule with short convolutions and one decay per head) and
    'parallel' (an attention with rescaled rotation, normed values and capped scores beside a time mix with token shift
    and a decay per key channel, their normed results averaged); feed-forwards 'moe' (experts with a clamped activation
    whose sigmoid scores multiply the experts' input) or none.  The configuration is nested; ``layers`` lists every
    layer's type and sizes, and nothing is assumed equal between layers."""

    architecture: str = ""
    vocab: int = -1
    width: int = -1
    norm_eps: float = 0.0
    norm_groups: int = 1
    residual_mult: float = 1.0
    #: one dict per layer: type, mixer (sizes and constants of that mixer), mlp (None or {kind: moe, ff, limit, experts, top})
    layers: List[Dict[str, Any]] = dataclasses.field(default_factory=list)

    MIXERS: ClassVar[tuple] = ("mlstm", "delta", "parallel")

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "MeronexConfig":
        cfg = cls(architecture=str(raw.get("architecture") or (raw.get("architectures") or [""])[0]),
                  vocab=_need(raw, "vocab", int), width=_need(raw, "width", int), norm_eps=float(_need(raw, "norm.eps", (int, float))))
        if (raw.get("norm") or {}).get("groups") is not None:
            cfg.norm_groups = _need(raw, "norm.groups", int)
        if raw.get("residual_mult") is not None:
            cfg.residual_mult = float(_need(raw, "residual_mult", (int, float)))
        cfg.layers = [cls._layer(i, l) for i, l in enumerate(_need(raw, "layers", list))]
        cfg._raw = dict(raw)
        cfg.validate()
        return cfg

    @staticmethod
    def _attention(m: Dict[str, Any], at: str) -> Dict[str, Any]:
        mix = {k: _need(m, k, int, at) for k in ("heads", "dim", "vdim")}
        mix["kv_heads"] = _need(m, "kv_heads", int, at) if m.get("kv_heads") is not None else mix["heads"]
        mix["scale"] = float(_need(m, "scale", (int, float), at))
        mix["softcap"] = float(_need(m, "softcap", (int, float), at)) if m.get("softcap") is not None else 0.0
        rot = m.get("rot")
        mix["rot"] = None
        if rot:
            mix["rot"] = {"base": float(_need(rot, "base", (int, float), at + ".rot")), "dims": _need(rot, "dims", int, at + ".rot"),
                          "scaling": None}
            sc = rot.get("scaling")
            if sc:
                mix["rot"]["scaling"] = {k: float(_need(sc, k, (int, float), at + ".rot.scaling")) for k in ("factor", "original", "fast", "slow")}
        return mix

    @classmethod
    def _layer(cls, i: int, raw: Dict[str, Any]) -> Dict[str, Any]:
        where = "config.json layers[%d]" % i
        if not isinstance(raw, dict):
            raise ConfigError("%s is no object" % where)
        kind = _need(raw, "type", str, where)
        if kind not in cls.MIXERS:
            raise ConfigError("%s: mixer type %r is not known (%s)" % (where, kind, ", ".join(cls.MIXERS)))
        m = _need(raw, "mixer", dict, where)
        at = where + ".mixer"
        if kind == "mlstm":
            mix = {k: _need(m, k, int, at) for k in ("heads", "dim", "vdim")}
            mix["gate_cap"] = float(_need(m, "gate_cap", (int, float), at))
        elif kind == "delta":
            mix = {k: _need(m, k, int, at) for k in ("heads", "dim", "vdim", "conv")}
            mix["kv_heads"] = _need(m, "kv_heads", int, at) if m.get("kv_heads") is not None else mix["heads"]
        else:
            right = _need(m, "right", dict, at)
            mix = {"left": cls._attention(_need(m, "left", dict, at), at + ".left"),
                   "right": {k: _need(right, k, int, at + ".right") for k in ("heads", "dim")}}
            # the inner size of the decay's two projections: no key of the design; the stored tensors decide unless it is given
            mix["right"]["decay_rank"] = _need(right, "decay_rank", int, at + ".right") if right.get("decay_rank") is not None else None
        out = {"type": kind, "mixer": mix, "mlp": None}
        mlp = raw.get("mlp")
        if mlp is not None:
            at = where + ".mlp"
            fk = _need(mlp, "kind", str, at)
            if fk != "moe":
                raise ConfigError("%s: kind %r is not known (moe)" % (at, fk))
            out["mlp"] = {"kind": fk, "ff": _need(mlp, "expert.ff", int, at), "limit": float(_need(mlp, "expert.limit", (int, float), at)),
                          "experts": _need(mlp, "router.experts", int, at), "top": _need(mlp, "router.top", int, at)}
        return out

    def to_dict(self) -> Dict[str, Any]:
        return dict(getattr(self, "_raw", {}))

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("config.json: vocab and width must be positive")
        if not (self.norm_eps > 0.0):
            raise ConfigError("config.json: norm.eps must be positive")
        if self.norm_groups <= 0 or self.width % self.norm_groups:
            raise ConfigError("config.json: norm.groups (%d) must divide the width (%d)" % (self.norm_groups, self.width))
        if not self.layers:
            raise ConfigError("config.json: no layers")
        for i, layer in enumerate(self.layers):
            where = "config.json layers[%d]" % i
            sides = [("", layer["mixer"])] if layer["type"] != "parallel" else [(".left", layer["mixer"]["left"]), (".right", layer["mixer"]["right"])]
            for side, m in sides:
                if any(isinstance(v, int) and not isinstance(v, bool) and v <= 0 for v in m.values()):
                    raise ConfigError("%s.mixer%s: sizes must be positive" % (where, side))
                if "kv_heads" in m and m["heads"] % m["kv_heads"]:
                    raise ConfigError("%s.mixer%s: heads (%d) is not a multiple of kv_heads (%d)" % (where, side, m["heads"], m["kv_heads"]))
            if layer["type"] == "mlstm" and not layer["mixer"]["gate_cap"] > 0.0:
                raise ConfigError("%s.mixer.gate_cap must be positive" % where)
            if layer["type"] == "delta" and layer["mixer"]["conv"] > 8:
                raise ConfigError("%s.mixer.conv: at most 8 taps" % where)
            if layer["type"] == "parallel":
                left = layer["mixer"]["left"]
                if left["softcap"] < 0.0:
                    raise ConfigError("%s.mixer.left.softcap must not be negative" % where)
                rot = left["rot"]
                if rot and (rot["dims"] % 2 or not (0 < rot["dims"] <= left["dim"]) or not rot["base"] > 1.0):
                    raise ConfigError("%s.mixer.left.rot: dims must be even and at most dim, base above 1" % where)
                sc = rot["scaling"] if rot else None
                if sc and not (sc["factor"] > 0.0 and sc["original"] > 0.0 and sc["fast"] > 0.0 and sc["slow"] > 0.0):
                    raise ConfigError("%s.mixer.left.rot.scaling: factor, original, fast and slow must be positive" % where)
            f = layer["mlp"]
            if f and (f["ff"] <= 0 or not f["limit"] > 0.0 or f["experts"] <= 0 or not 0 < f["top"] <= f["experts"]):
                raise ConfigError("%s.mlp: inner size and limit positive, 1 to %d choices" % (where, max(f["experts"], 1)))


@dataclasses.dataclass
class TarunexConfig(ModelConfig):
    """Tarunex: layers whose mixer and feed-forward read the stream through a norm each (a norm's weight is one number)
    and are added together; a run of consecutive layers may be walked several times with the same weights (``loop``),
    every walk with caches of its own, the embedding output added back before every walk but the first and a learned
    vector before each; token mixers 'attention' (grouped queries with biases and no rotation, a temperature on the
    queries that grows with the logarithm of the position, capped scores lowered by a logarithmic penalty on the
    distance, a softmax with a one in its denominator, one gate number per head) and 'latent_attention' (queries through
    a normed low-rank vector, keys and values expanded from a cached one, interleaved rotary pairs on a part that all
    heads share, one gate number per head); the feed-forward a mixture of gated experts (a router with a bias, the
    weights a softmax over the chosen logits) plus an expert that every token uses; scaled and capped logits.  The
    configuration is nested; ``layers`` lists every layer's type and sizes, and nothing is assumed equal between layers."""

    architecture: str = ""
    vocab: int = -1
    width: int = -1
    norm_eps: float = 0.0
    embedding_scale: float = 1.0
    logit_scale: float = 1.0
    logit_softcap: float = 0.0
    #: None, or {start, stop, times}: layers start .. stop - 1 are walked ``times`` times in a row
    loop: Optional[Dict[str, int]] = None
    #: one dict per layer: type, mixer (sizes and constants of that mixer), mlp (None or {kind: moe, ff, experts, top, shared_ff})
    layers: List[Dict[str, Any]] = dataclasses.field(default_factory=list)

    MIXERS: ClassVar[tuple] = ("attention", "latent_attention")

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "TarunexConfig":
        cfg = cls(architecture=str(raw.get("architecture") or (raw.get("architectures") or [""])[0]),
                  vocab=_need(raw, "vocab", int), width=_need(raw, "width", int), norm_eps=float(_need(raw, "norm.eps", (int, float))))
        if (raw.get("embedding") or {}).get("scale") is not None:
            cfg.embedding_scale = float(_need(raw, "embedding.scale", (int, float)))
        if raw.get("logit_scale") is not None:
            cfg.logit_scale = float(_need(raw, "logit_scale", (int, float)))
        if raw.get("logit_softcap") is not None:
            cfg.logit_softcap = float(_need(raw, "logit_softcap", (int, float)))
        if raw.get("loop"):
            cfg.loop = {k: _need(raw, "loop." + k, int) for k in ("start", "stop", "times")}
        cfg.layers = [cls._layer(i, l) for i, l in enumerate(_need(raw, "layers", list))]
        cfg._raw = dict(raw)
        cfg.validate()
        return cfg

    @classmethod
    def _layer(cls, i: int, raw: Dict[str, Any]) -> Dict[str, Any]:
        where = "config.json layers[%d]" % i
        if not isinstance(raw, dict):
            raise ConfigError("%s is no object" % where)
        kind = _need(raw, "type", str, where)
        if kind not in cls.MIXERS:
            raise ConfigError("%s: mixer type %r is not known (%s)" % (where, kind, ", ".join(cls.MIXERS)))
        m = _need(raw, "mixer", dict, where)
        at = where + ".mixer"
        if kind == "attention":
            mix = {k: _need(m, k, int, at) for k in ("heads", "dim", "vdim")}
            mix["kv_heads"] = _need(m, "kv_heads", int, at) if m.get("kv_heads") is not None else mix["heads"]
            mix["scale"] = float(_need(m, "scale", (int, float), at))
            mix["softcap"] = float(_need(m, "softcap", (int, float), at)) if m.get("softcap") is not None else 0.0
            mix["q_temp"] = None
            if m.get("q_temp"):
                mix["q_temp"] = {"coef": float(_need(m, "q_temp.coef", (int, float), at)), "every": _need(m, "q_temp.every", int, at)}
        else:
            mix = {k: _need(m, k, int, at) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank")}
            mix["scale"] = float(_need(m, "scale", (int, float), at))
            rot = m.get("rot")
            mix["rot"] = None
            if rot:
                mix["rot"] = {"base": float(_need(rot, "base", (int, float), at + ".rot")), "dims": _need(rot, "dims", int, at + ".rot")}
        out = {"type": kind, "mixer": mix, "mlp": None}
        mlp = raw.get("mlp")
        if mlp is not None:
            at = where + ".mlp"
            fk = _need(mlp, "kind", str, at)
            if fk != "moe":
                raise ConfigError("%s: kind %r is not known (moe)" % (at, fk))
            out["mlp"] = {"kind": fk, "ff": _need(mlp, "expert.ff", int, at), "experts": _need(mlp, "router.experts", int, at),
                          "top": _need(mlp, "router.top", int, at),
                          "shared_ff": _need(mlp, "shared.ff", int, at) if mlp.get("shared") else None}
        return out

    def to_dict(self) -> Dict[str, Any]:
        return dict(getattr(self, "_raw", {}))

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("config.json: vocab and width must be positive")
        if not (self.norm_eps > 0.0):
            raise ConfigError("config.json: norm.eps must be positive")
        if self.logit_softcap < 0.0:
            raise ConfigError("config.json: logit_softcap must not be negative")
        if not self.layers:
            raise ConfigError("config.json: no layers")
        if self.loop is not None:
            lp = self.loop
            if not (0 <= lp["start"] < lp["stop"] <= len(self.layers)) or lp["times"] < 1:
                raise ConfigError("config.json loop: layers %d .. %d of %d, %d times" % (lp["start"], lp["stop"] - 1, len(self.layers), lp["times"]))
        for i, layer in enumerate(self.layers):
            where = "config.json layers[%d]" % i
            m = layer["mixer"]
            if any(isinstance(v, int) and not isinstance(v, bool) and v <= 0 for k, v in m.items() if k != "dim"):
                raise ConfigError("%s.mixer: sizes must be positive" % where)
            if layer["type"] == "attention":
                if m["dim"] <= 0 or m["heads"] % m["kv_heads"]:
                    raise ConfigError("%s.mixer: heads (%d) is not a multiple of kv_heads (%d)" % (where, m["heads"], m["kv_heads"]))
                if m["softcap"] < 0.0:
                    raise ConfigError("%s.mixer.softcap must not be negative" % where)
                if m["q_temp"] and m["q_temp"]["every"] <= 0:
                    raise ConfigError("%s.mixer.q_temp.every must be positive" % where)
            else:
                rot = m["rot"]
                if m["dim"] < 0 or (rot and (rot["dims"] % 2 or not (0 < rot["dims"] <= m["rot_dim"]) or not rot["base"] > 1.0)):
                    raise ConfigError("%s.mixer.rot: dims must be even and at most rot_dim, base above 1" % where)
            f = layer["mlp"]
            if f and (f["ff"] <= 0 or f["experts"] <= 0 or not 0 < f["top"] <= f["experts"] or (f["shared_ff"] is not None and f["shared_ff"] <= 0)):
                raise ConfigError("%s.mlp: inner sizes positive, 1 to %d choices" % (where, max(f["experts"], 1)))
