"""Lutosun configuration, read from the design's own ``config.json`` keys.

A decoder whose layers are listed one by one (``layers``): each has a latent attention mixer (``type``
``latent_attention``, its sizes in ``mixer``) and a mixture-of-experts feed-forward (``mlp`` with ``kind`` ``moe``,
or null for a layer without one).  Layers are pre-norm with a layer norm (weight and bias) and every branch is
multiplied by ``residual_mult`` where it joins the stream.  The embedding is scaled (``embedding.scale``) and a
hashed bigram row is added to it (``embedding.bigram``).  ``loop``: the layers ``start`` to ``stop`` - 1 run
``times`` times in a row with the same weights, each pass with a cache of its own; before every pass but the
first the embedding output is added to the stream again, and before every pass row t of ``loop.step``.  The logits
are capped (``logit_softcap``).

Tensors are stored without ``.weight``: ``l<i>.mix.dq``, ``l<i>.norm1`` and its bias ``l<i>.norm1.b``, ``embed``,
``bigram``, ``loop.step``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from .mukutar import _integer, _number, _table
from .spec import (ClampedGLUSpec, ConfigError, HashedBigramSpec, InterleavedRopeSpec, LatentAttentionSpec,
                   LayerNormSpec, LayerSpec, MixerSlot, ModelSpec, NoPositionSpec, RoutedExpertsSpec, ScheduleEntry,
                   StreamInjection, _require)

# a tensor's name in the model -> the name it is stored under
STORED_NAME_RULES = ((r"\.weight$", ""), (r"\.bias$", ".b"))

FIELD_NAMES = (("latent_attention.cached_key_dim", "layers[].mixer.kv_rank + rot_dim"),
               ("latent_attention.num_heads", "layers[].mixer.heads"),
               ("routed_experts.num_experts", "layers[].mlp.router.experts"),
               ("layernorm.hidden_size", "width"))

DEFAULT_MAX_CONTEXT = 1 << 20       # the design names no limit: the longest the engine's tables index
LOOP_VECTORS = "loop.step"


@dataclass(frozen=True)
class LutosunLayer:
    type: str
    mixer: object                       # the mixer's spec
    mlp: Optional[object]               # the feed-forward's spec, None for a layer without one
    raw: dict                           # the layer's own table, for ``to_dict``


@dataclass(frozen=True)
class LutosunLoop:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class LutosunConfig:
    width: int
    vocab: int
    norm_eps: float
    residual_mult: float
    embedding_scale: float
    layers: Tuple[LutosunLayer, ...]
    bigram: Optional[HashedBigramSpec] = None
    loop: Optional[LutosunLoop] = None
    logit_softcap: Optional[float] = None
    max_context: int = DEFAULT_MAX_CONTEXT
    eos_token_id: Optional[int] = None

    architecture_names = ("Lutosun", "lutosun")

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, raw: dict) -> "LutosunConfig":
        width = _integer(raw, "width", "")
        vocab = _integer(raw, "vocab", "")
        eps = _number(_table(raw.get("norm", {}), "norm"), "eps", "norm")
        embedding = _table(raw.get("embedding", {}), "embedding")
        bigram = None
        if embedding.get("bigram") is not None:
            hashed = _table(embedding["bigram"], "embedding.bigram")
            bigram = HashedBigramSpec(buckets=_integer(hashed, "buckets", "embedding.bigram"),
                                      mul_prev=_integer(hashed, "mul_prev", "embedding.bigram"),
                                      mul_cur=_integer(hashed, "mul_cur", "embedding.bigram"))
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for index, entry in enumerate(listed):
            where = f"layers[{index}]"
            entry = _table(entry, where)
            kind = entry.get("type")
            reader = _MIXERS.get(kind)
            if reader is None:
                raise ConfigError(f"config.json: '{where}.type' is {kind!r}; known: {sorted(_MIXERS)}")
            mixer = reader(_table(entry.get("mixer"), f"{where}.mixer"), f"{where}.mixer", eps)
            mlp = None
            if entry.get("mlp") is not None:
                table = _table(entry["mlp"], f"{where}.mlp")
                if table.get("kind") not in _FEED_FORWARDS:
                    raise ConfigError(f"config.json: '{where}.mlp.kind' is {table.get('kind')!r}; "
                                      f"known: {sorted(_FEED_FORWARDS)}")
                mlp = _FEED_FORWARDS[table["kind"]](table, f"{where}.mlp")
            layers.append(LutosunLayer(kind, mixer, mlp, entry))
        loop = None
        if raw.get("loop") is not None:
            table = _table(raw["loop"], "loop")
            loop = LutosunLoop(start=_integer(table, "start", "loop"), stop=_integer(table, "stop", "loop"),
                               times=_integer(table, "times", "loop"))
        cap = raw.get("logit_softcap")
        eos = raw.get("eos_token_id")
        config = cls(width=width, vocab=vocab, norm_eps=eps, residual_mult=_number(raw, "residual_mult", "", 1.0),
                     embedding_scale=_number(embedding, "scale", "embedding", 1.0), layers=tuple(layers),
                     bigram=bigram, loop=loop, logit_softcap=None if cap is None else _number(raw, "logit_softcap", ""),
                     max_context=_integer(raw, "max_context", "", DEFAULT_MAX_CONTEXT),
                     eos_token_id=eos if isinstance(eos, int) and not isinstance(eos, bool) else None)
        config.validate()
        return config

    def to_dict(self) -> dict:
        out = {"architecture": "Lutosun", "embedding": {"scale": self.embedding_scale},
               "layers": [layer.raw for layer in self.layers], "norm": {"eps": self.norm_eps},
               "residual_mult": self.residual_mult, "vocab": self.vocab, "width": self.width}
        if self.bigram is not None:
            out["embedding"]["bigram"] = {"buckets": self.bigram.buckets, "mul_cur": self.bigram.mul_cur,
                                          "mul_prev": self.bigram.mul_prev}
        if self.loop is not None:
            out["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
        if self.logit_softcap is not None:
            out["logit_softcap"] = self.logit_softcap
        if self.max_context != DEFAULT_MAX_CONTEXT:
            out["max_context"] = self.max_context
        return out

    def validate(self) -> None:
        _require(self.width > 0 and self.vocab > 0, "config.json: 'width' and 'vocab' must be positive")
        if self.loop is not None:
            _require(0 <= self.loop.start < self.loop.stop <= len(self.layers),
                     f"config.json: 'loop' runs layers {self.loop.start} to {self.loop.stop} - 1 of {len(self.layers)}")
            _require(self.loop.times >= 1, "config.json: 'loop.times' must be at least 1")
        self.to_model_spec().validate()

    # ------------------------------------------------------------------ lowering
    def run_order(self) -> Tuple[ScheduleEntry, ...]:
        """The layers in the order they run: the looped ones ``times`` times in a row, each run an entry (and so a
        cache) of its own; the first run of a pass carries what is added to the stream before it."""
        count = len(self.layers)
        if self.loop is None:
            return tuple(ScheduleEntry(layer=index) for index in range(count))
        loop = self.loop
        entries = [ScheduleEntry(layer=index) for index in range(loop.start)]
        for turn in range(loop.times):
            for index in range(loop.start, loop.stop):
                before = None
                if index == loop.start:
                    before = StreamInjection(embedding=turn > 0, vector_name=LOOP_VECTORS, row=turn)
                entries.append(ScheduleEntry(layer=index, before=before))
        entries += [ScheduleEntry(layer=index) for index in range(loop.stop, count)]
        return tuple(entries)

    def to_model_spec(self) -> ModelSpec:
        norm = LayerNormSpec(eps=self.norm_eps)
        layers = tuple(
            LayerSpec(prefix=f"l{index}", mixers=(MixerSlot("mix", layer.mixer),), ffn=layer.mlp,
                      mixer_norm=norm, ffn_norm=norm, mixer_norm_name="norm1", ffn_norm_name="norm2", ffn_name="mlp",
                      branch_multiplier=self.residual_mult)
            for index, layer in enumerate(self.layers))
        return ModelSpec(
            architecture="Lutosun", hidden_size=self.width, vocab_size=self.vocab, max_context=self.max_context,
            layers=layers, schedule=self.run_order(), final_norm=norm, embedding_multiplier=self.embedding_scale,
            logit_softcap=self.logit_softcap, bigram=self.bigram, bigram_name="bigram",
            injected_vectors=() if self.loop is None else ((LOOP_VECTORS, self.loop.times),),
            embedding_name="embed", final_norm_name="final.norm", lm_head_name="head",
            root_namespace="", stored_name_rules=STORED_NAME_RULES, field_names=FIELD_NAMES)

    # ------------------------------------------------------------------ reports
    def kv_bytes_per_token(self, bytes_per_element: int) -> int:
        """The latent and the turned key part of every run of every layer for one token."""
        return sum(self.layers[entry.layer].mixer.cached_key_dim * bytes_per_element for entry in self.run_order())

    def fixed_state_bytes(self, bytes_per_element: int) -> int:
        return 4 if self.bigram is not None else 0          # the previous token


def _latent_attention(mixer: dict, where: str, eps: float) -> LatentAttentionSpec:
    rope_dim = _integer(mixer, "rot_dim", where, 0)
    position = NoPositionSpec()
    if rope_dim and mixer.get("rot") is not None:
        rot = _table(mixer["rot"], f"{where}.rot")
        position = InterleavedRopeSpec(theta=_number(rot, "base", f"{where}.rot"),
                                       rotary_dim=_integer(rot, "dims", f"{where}.rot", rope_dim))
    dim = _integer(mixer, "dim", where)
    return LatentAttentionSpec(num_heads=_integer(mixer, "heads", where), head_dim=dim, rope_dim=rope_dim,
                               value_dim=_integer(mixer, "vdim", where, dim), q_rank=_integer(mixer, "q_rank", where),
                               kv_rank=_integer(mixer, "kv_rank", where), scale=_number(mixer, "scale", where),
                               norm_eps=eps, position=position)


def _moe(mlp: dict, where: str) -> RoutedExpertsSpec:
    expert = _table(mlp.get("expert"), f"{where}.expert")
    router = _table(mlp.get("router"), f"{where}.router")
    shared_size = shared_activation = None
    if mlp.get("shared") is not None:
        shared = _table(mlp["shared"], f"{where}.shared")
        shared_size = _integer(shared, "ff", f"{where}.shared")
        shared_activation = ClampedGLUSpec(limit=_number(shared, "limit", f"{where}.shared"))
    return RoutedExpertsSpec(num_experts=_integer(router, "experts", f"{where}.router"),
                             top_k=_integer(router, "top", f"{where}.router"),
                             expert_size=_integer(expert, "ff", f"{where}.expert"),
                             activation=ClampedGLUSpec(limit=_number(expert, "limit", f"{where}.expert")),
                             route_scale=_number(router, "scale", f"{where}.router", 1.0),
                             shared_size=shared_size, shared_activation=shared_activation)


_MIXERS = {"latent_attention": _latent_attention}
_FEED_FORWARDS = {"moe": _moe}
