"""Mukutar configuration, read from the design's own ``config.json`` keys.

A decoder whose layers are listed one by one (``layers``): each has one mixer, named by ``type``
(``attention``: windowed grouped-query attention with a logarithmic distance bias and a sink;
``retention``: linear attention with a fixed decay per head; ``general_delta``: a generalized delta rule),
the mixer's sizes (``mixer``) and a dense feed-forward with a PolyNorm activation (``mlp``, or null).
Layers are pre-norm, the norms' weights are stored around zero, and every branch is scaled feature by
feature before it is added to the stream.  ``width``, ``vocab`` and ``norm.eps`` are the model's.

Tensors are stored without ``.weight``: ``l<i>.mix.q``, its bias ``l<i>.mix.q.b``, ``l<i>.norm1``, ``embed``,
``final.norm``, ``head``.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Tuple

from .spec import (AttentionSpec, ConfigError, GeneralDeltaSpec, LayerSpec, LogDistanceBiasSpec, MixerSlot,
                   ModelSpec, NoPositionSpec, PolyNormFFNSpec, RetentionSpec, RmsNormSpec, RopeSpec,
                   ScheduleEntry, _require)

# a tensor's name in the model -> the name it is stored under
STORED_NAME_RULES = ((r"_proj\.", "."), (r"\.weight$", ""), (r"\.bias$", ".b"))

FIELD_NAMES = (("attention.head_dim", "layers[].mixer.dim"), ("attention.num_heads", "layers[].mixer.heads"),
               ("retention.key_dim", "layers[].mixer.dim"), ("retention.value_dim", "layers[].mixer.vdim"),
               ("general_delta.head_dim", "layers[].mixer.dim"), ("rmsnorm.hidden_size", "width"))

DEFAULT_MAX_CONTEXT = 1 << 20       # the design names no limit: the longest the engine's tables index


def _table(value, where: str) -> dict:
    if not isinstance(value, dict):
        raise ConfigError(f"config.json: '{where}' must be a table, got {value!r}")
    return value


def _integer(table: dict, key: str, where: str, default=None) -> int:
    value = table.get(key, default)
    if value is None:
        raise ConfigError(f"config.json: required key '{where}.{key}' is missing")
    if isinstance(value, bool) or not isinstance(value, int):
        raise ConfigError(f"config.json: '{where}.{key}' must be an integer, got {value!r}")
    return value


def _number(table: dict, key: str, where: str, default=None) -> float:
    value = table.get(key, default)
    if value is None:
        raise ConfigError(f"config.json: required key '{where}.{key}' is missing")
    if isinstance(value, bool) or not isinstance(value, (int, float)) or not math.isfinite(value):
        raise ConfigError(f"config.json: '{where}.{key}' must be a finite number, got {value!r}")
    return float(value)


@dataclass(frozen=True)
class MukutarLayer:
    type: str
    mixer: object                       # the mixer's spec
    ff: Optional[int]                   # the feed-forward's inner width, None for a layer without one
    raw: dict                           # the layer's own table, for ``to_dict``


@dataclass(frozen=True)
class MukutarConfig:
    width: int
    vocab: int
    norm_eps: float
    layers: Tuple[MukutarLayer, ...]
    max_context: int = DEFAULT_MAX_CONTEXT
    eos_token_id: Optional[int] = None

    architecture_names = ("Mukutar", "mukutar")

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, raw: dict) -> "MukutarConfig":
        width = _integer(raw, "width", "")
        vocab = _integer(raw, "vocab", "")
        eps = _number(_table(raw.get("norm", {}), "norm"), "eps", "norm")
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for index, entry in enumerate(listed):
            where = f"layers[{index}]"
            entry = _table(entry, where)
            kind = entry.get("type")
            mixer = _table(entry.get("mixer"), f"{where}.mixer")
            reader = _MIXERS.get(kind)
            if reader is None:
                raise ConfigError(f"config.json: '{where}.type' is {kind!r}; known: {sorted(_MIXERS)}")
            spec = reader(mixer, f"{where}.mixer", eps)
            ff = None
            if entry.get("mlp") is not None:
                mlp = _table(entry["mlp"], f"{where}.mlp")
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"config.json: '{where}.mlp.kind' is {mlp.get('kind')!r}; known: ['dense']")
                ff = _integer(mlp, "ff", f"{where}.mlp")
            layers.append(MukutarLayer(kind, spec, ff, entry))
        eos = raw.get("eos_token_id")
        config = cls(width=width, vocab=vocab, norm_eps=eps, layers=tuple(layers),
                     max_context=_integer(raw, "max_context", "", DEFAULT_MAX_CONTEXT),
                     eos_token_id=eos if isinstance(eos, int) and not isinstance(eos, bool) else None)
        config.validate()
        return config

    def to_dict(self) -> dict:
        out = {"architecture": "Mukutar", "layers": [layer.raw for layer in self.layers],
               "norm": {"eps": self.norm_eps}, "vocab": self.vocab, "width": self.width}
        if self.max_context != DEFAULT_MAX_CONTEXT:
            out["max_context"] = self.max_context
        return out

    def validate(self) -> None:
        _require(self.width > 0 and self.vocab > 0, "config.json: 'width' and 'vocab' must be positive")
        self.to_model_spec().validate()

    # ------------------------------------------------------------------ lowering
    def to_model_spec(self) -> ModelSpec:
        norm = RmsNormSpec(eps=self.norm_eps, weight_offset=1.0)
        layers = tuple(
            LayerSpec(prefix=f"l{index}", mixers=(MixerSlot("mix", layer.mixer),),
                      ffn=None if layer.ff is None else PolyNormFFNSpec(intermediate_size=layer.ff, eps=self.norm_eps),
                      mixer_norm=norm, ffn_norm=norm, mixer_norm_name="norm1", ffn_norm_name="norm2", ffn_name="mlp",
                      mixer_scale_name="ls1", ffn_scale_name="ls2")
            for index, layer in enumerate(self.layers))
        return ModelSpec(
            architecture="Mukutar", hidden_size=self.width, vocab_size=self.vocab, max_context=self.max_context,
            layers=layers, schedule=tuple(ScheduleEntry(layer=index) for index in range(len(layers))),
            final_norm=norm, embedding_name="embed", final_norm_name="final.norm", lm_head_name="head",
            root_namespace="", stored_name_rules=STORED_NAME_RULES, field_names=FIELD_NAMES)

    # ------------------------------------------------------------------ reports
    def kv_bytes_per_token(self, bytes_per_element: int) -> int:
        """Keys and values of every attention layer for one token (until its window has passed)."""
        return sum(layer.mixer.num_kv_heads * (layer.mixer.head_dim + layer.mixer.value_width) * bytes_per_element
                   for layer in self.layers if layer.type == "attention")

    def fixed_state_bytes(self, bytes_per_element: int) -> int:
        """The float32 states of every recurrent layer for one request."""
        total = 0
        for layer in self.layers:
            if layer.type == "retention":
                total += layer.mixer.num_heads * layer.mixer.key_dim * layer.mixer.value_dim * 4
            elif layer.type == "general_delta":
                total += layer.mixer.num_heads * layer.mixer.head_dim ** 2 * 4
        return total


def _attention(mixer: dict, where: str, eps: float) -> AttentionSpec:
    heads = _integer(mixer, "heads", where)
    dim = _integer(mixer, "dim", where)
    mask = mixer.get("mask")
    window = None if mask is None else _integer(_table(mask, f"{where}.mask"), "size", f"{where}.mask")
    return AttentionSpec(num_heads=heads, num_kv_heads=_integer(mixer, "kv_heads", where, heads), head_dim=dim,
                         scale=_number(mixer, "scale", where), position=LogDistanceBiasSpec(num_heads=heads),
                         window=window, qkv_bias=True, out_bias=False, value_dim=_integer(mixer, "vdim", where, dim),
                         sink=True)


def _retention(mixer: dict, where: str, eps: float) -> RetentionSpec:
    heads = _integer(mixer, "heads", where)
    dim = _integer(mixer, "dim", where)
    decay = mixer.get("decay")
    if (not isinstance(decay, list) or len(decay) != heads
            or any(isinstance(d, bool) or not isinstance(d, (int, float)) for d in decay)):
        raise ConfigError(f"config.json: '{where}.decay' must list one number for each of the {heads} heads")
    position = NoPositionSpec()
    if mixer.get("rot") is not None:
        rot = _table(mixer["rot"], f"{where}.rot")
        position = RopeSpec(theta=_number(rot, "base", f"{where}.rot"), rotary_dim=_integer(rot, "dims", f"{where}.rot"))
    return RetentionSpec(num_heads=heads, key_dim=dim, value_dim=_integer(mixer, "vdim", where, dim),
                         decay=tuple(float(d) for d in decay), key_scale=dim ** -0.5, norm_eps=eps, position=position)


def _general_delta(mixer: dict, where: str, eps: float) -> GeneralDeltaSpec:
    rank = mixer.get("decay_rank")
    return GeneralDeltaSpec(num_heads=_integer(mixer, "heads", where), head_dim=_integer(mixer, "dim", where),
                            norm_eps=eps, decay_rank=None if rank is None else _integer(mixer, "decay_rank", where))


_MIXERS = {"attention": _attention, "retention": _retention, "general_delta": _general_delta}
