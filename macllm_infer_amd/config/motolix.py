"""Motolix configuration, read from the design's own ``config.json`` keys.

A decoder whose layers are listed one by one (``layers``).  A layer normalizes (layer norm with weight and bias)
before and after each branch: x <- x + norm1b(mixer(norm1(x))), x <- x + norm2b(ff(norm2(x))).  Mixers (``type``):

``attention``  grouped-query attention with biases on q, k and the output, whose values are the keys as projected;
               rotation of the first ``rot.dims`` dims of q and k, frequencies optionally stretched by wavelength
               (``rot.scaling``); every head's scores times a learned number; a visible key weighs
               sigmoid(score + a learned number per head), nothing is normalized.
``parallel``   two mixers on the same rows, summed with ``left_scale`` and ``right_scale``: ``left`` is softmax
               attention with an RMS norm over the whole q and the whole k projection and values turned by their
               position (outputs turned back); ``right`` is gated linear attention (a decay per key channel).

The feed-forward (``mlp`` with ``kind`` ``dense``, or null) is gated with the tanh form of GELU.  ``loop``: layers
``start`` to ``stop`` - 1 run ``times`` times in a row with the same weights, each pass with a cache of its own;
before every pass the stream x becomes ``loop.in`` [x; x0] (x0 the embedding output) plus row t of ``loop.step``.
The embedding is scaled (``embedding.scale``), the logits too (``logit_scale``).

Tensors are stored without ``.weight``: ``l<i>.mix.q`` and its bias ``l<i>.mix.q.b``, ``l<i>.mix.left.q.norm``,
``l<i>.norm1`` and ``l<i>.norm1.b``, ``embed``, ``loop.in``, ``loop.step``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from .mukutar import _integer, _number, _table
from .spec import (AttentionSpec, ConfigError, GatedLinearAttentionSpec, LayerNormSpec, LayerSpec, MixerSlot,
                   ModelSpec, NoPositionSpec, RopeSpec, ScheduleEntry, StreamInjection, SwiGLUSpec,
                   WavelengthScalingSpec, _require)

# a tensor's name in the model -> the name it is stored under
STORED_NAME_RULES = ((r"\.(q|k)_norm\.weight$", r".\1.norm"), (r"_proj\.", "."), (r"\.weight$", ""), (r"\.bias$", ".b"))

FIELD_NAMES = (("attention.head_dim", "layers[].mixer.dim"), ("attention.num_heads", "layers[].mixer.heads"),
               ("gated_linear_attention.key_dim", "layers[].mixer.right.dim"),
               ("gated_linear_attention.num_heads", "layers[].mixer.right.heads"), ("layernorm.hidden_size", "width"))

DEFAULT_MAX_CONTEXT = 1 << 20       # the design names no limit: the longest the engine's tables index
LOOP_VECTORS = "loop.step"
LOOP_MIX = "loop.in"


@dataclass(frozen=True)
class MotolixLayer:
    type: str
    mixers: Tuple[MixerSlot, ...]       # one mixer, or the two of a parallel layer
    ff: Optional[int]                   # the feed-forward's inner width, None for a layer without one
    raw: dict                           # the layer's own table, for ``to_dict``


@dataclass(frozen=True)
class MotolixLoop:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class MotolixConfig:
    width: int
    vocab: int
    norm_eps: float
    embedding_scale: float
    logit_scale: float
    layers: Tuple[MotolixLayer, ...]
    loop: Optional[MotolixLoop] = None
    max_context: int = DEFAULT_MAX_CONTEXT
    eos_token_id: Optional[int] = None

    architecture_names = ("Motolix", "motolix")

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, raw: dict) -> "MotolixConfig":
        width = _integer(raw, "width", "")
        vocab = _integer(raw, "vocab", "")
        eps = _number(_table(raw.get("norm", {}), "norm"), "eps", "norm")
        embedding = _table(raw.get("embedding", {}), "embedding")
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
            mixers = reader(_table(entry.get("mixer"), f"{where}.mixer"), f"{where}.mixer", eps)
            ff = None
            if entry.get("mlp") is not None:
                mlp = _table(entry["mlp"], f"{where}.mlp")
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"config.json: '{where}.mlp.kind' is {mlp.get('kind')!r}; known: ['dense']")
                ff = _integer(mlp, "ff", f"{where}.mlp")
            layers.append(MotolixLayer(kind, mixers, ff, entry))
        loop = None
        if raw.get("loop") is not None:
            table = _table(raw["loop"], "loop")
            loop = MotolixLoop(start=_integer(table, "start", "loop"), stop=_integer(table, "stop", "loop"),
                               times=_integer(table, "times", "loop"))
        eos = raw.get("eos_token_id")
        config = cls(width=width, vocab=vocab, norm_eps=eps, embedding_scale=_number(embedding, "scale", "embedding", 1.0),
                     logit_scale=_number(raw, "logit_scale", "", 1.0), layers=tuple(layers), loop=loop,
                     max_context=_integer(raw, "max_context", "", DEFAULT_MAX_CONTEXT),
                     eos_token_id=eos if isinstance(eos, int) and not isinstance(eos, bool) else None)
        config.validate()
        return config

    def to_dict(self) -> dict:
        out = {"architecture": "Motolix", "embedding": {"scale": self.embedding_scale},
               "layers": [layer.raw for layer in self.layers], "logit_scale": self.logit_scale,
               "norm": {"eps": self.norm_eps}, "vocab": self.vocab, "width": self.width}
        if self.loop is not None:
            out["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
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
        cache) of its own; the first run of every pass carries what happens to the stream before it."""
        count = len(self.layers)
        if self.loop is None:
            return tuple(ScheduleEntry(layer=index) for index in range(count))
        loop = self.loop
        entries = [ScheduleEntry(layer=index) for index in range(loop.start)]
        for turn in range(loop.times):
            for index in range(loop.start, loop.stop):
                before = None
                if index == loop.start:
                    before = StreamInjection(mix_name=LOOP_MIX, vector_name=LOOP_VECTORS, row=turn)
                entries.append(ScheduleEntry(layer=index, before=before))
        entries += [ScheduleEntry(layer=index) for index in range(loop.stop, count)]
        return tuple(entries)

    def to_model_spec(self) -> ModelSpec:
        norm = LayerNormSpec(eps=self.norm_eps)
        layers = tuple(
            LayerSpec(prefix=f"l{index}", mixers=layer.mixers,
                      ffn=None if layer.ff is None else SwiGLUSpec(intermediate_size=layer.ff, activation="gelu_tanh"),
                      mixer_norm=norm, ffn_norm=norm, mixer_norm_name="norm1", ffn_norm_name="norm2", ffn_name="mlp",
                      arrangement="sandwich", mixer_post_norm=norm, ffn_post_norm=norm,
                      mixer_post_norm_name="norm1b", ffn_post_norm_name="norm2b")
            for index, layer in enumerate(self.layers))
        return ModelSpec(
            architecture="Motolix", hidden_size=self.width, vocab_size=self.vocab, max_context=self.max_context,
            layers=layers, schedule=self.run_order(), final_norm=norm, embedding_multiplier=self.embedding_scale,
            logit_multiplier=self.logit_scale,
            injected_vectors=() if self.loop is None else ((LOOP_VECTORS, self.loop.times),),
            injected_mixes=() if self.loop is None else (LOOP_MIX,),
            embedding_name="embed", final_norm_name="final.norm", lm_head_name="head",
            root_namespace="", stored_name_rules=STORED_NAME_RULES, field_names=FIELD_NAMES)

    # ------------------------------------------------------------------ reports
    def kv_bytes_per_token(self, bytes_per_element: int) -> int:
        """Keys and values of every attention mixer of every run of every layer for one token."""
        total = 0
        for entry in self.run_order():
            for slot in self.layers[entry.layer].mixers:
                if isinstance(slot.spec, AttentionSpec):
                    total += slot.spec.num_kv_heads * (slot.spec.head_dim + slot.spec.value_width) * bytes_per_element
        return total

    def fixed_state_bytes(self, bytes_per_element: int) -> int:
        """The float32 states of every gated linear attention mixer of every run for one request."""
        total = 0
        for entry in self.run_order():
            for slot in self.layers[entry.layer].mixers:
                if isinstance(slot.spec, GatedLinearAttentionSpec):
                    total += slot.spec.num_heads * slot.spec.key_dim * slot.spec.value_dim * 4
        return total


def _rotation(mixer: dict, where: str):
    if mixer.get("rot") is None:
        return NoPositionSpec(), None
    rot = _table(mixer["rot"], f"{where}.rot")
    scaling = None
    if rot.get("scaling") is not None:
        table = _table(rot["scaling"], f"{where}.rot.scaling")
        scaling = WavelengthScalingSpec(factor=_number(table, "factor", f"{where}.rot.scaling"),
                                        low=_number(table, "low", f"{where}.rot.scaling"),
                                        high=_number(table, "high", f"{where}.rot.scaling"),
                                        original=_number(table, "original", f"{where}.rot.scaling"))
    base = _number(rot, "base", f"{where}.rot")
    return RopeSpec(theta=base, rotary_dim=_integer(rot, "dims", f"{where}.rot"), scaling=scaling), base


def _sigmoid_attention(mixer: dict, where: str, eps: float) -> AttentionSpec:
    heads = _integer(mixer, "heads", where)
    dim = _integer(mixer, "dim", where)
    position, _ = _rotation(mixer, where)
    if _integer(mixer, "vdim", where, dim) != dim:
        raise ConfigError(f"config.json: '{where}.vdim' must equal '{where}.dim': the values are the keys")
    return AttentionSpec(num_heads=heads, num_kv_heads=_integer(mixer, "kv_heads", where, heads), head_dim=dim,
                         scale=_number(mixer, "scale", where), position=position, qkv_bias=True, out_bias=True,
                         values_from_keys=True, head_temperature=True, weighting="sigmoid", score_bias=True)


def _softmax_attention(mixer: dict, where: str, eps: float) -> AttentionSpec:
    heads = _integer(mixer, "heads", where)
    dim = _integer(mixer, "dim", where)
    position, base = _rotation(mixer, where)
    if base is None:
        raise ConfigError(f"config.json: required key '{where}.rot' is missing (the values turn by its base)")
    return AttentionSpec(num_heads=heads, num_kv_heads=_integer(mixer, "kv_heads", where, heads), head_dim=dim,
                         scale=_number(mixer, "scale", where), position=position,
                         value_dim=_integer(mixer, "vdim", where, dim), projection_norm_eps=eps,
                         value_rotation_theta=base)


def _gated_linear(mixer: dict, where: str, eps: float) -> GatedLinearAttentionSpec:
    dim = _integer(mixer, "dim", where)
    return GatedLinearAttentionSpec(num_heads=_integer(mixer, "heads", where), key_dim=dim,
                                    value_dim=_integer(mixer, "vdim", where, dim),
                                    decay_temperature=_number(mixer, "tau", where), query_scale=dim ** -0.5, norm_eps=eps)


def _attention_layer(mixer: dict, where: str, eps: float) -> Tuple[MixerSlot, ...]:
    return (MixerSlot("mix", _sigmoid_attention(mixer, where, eps)),)


def _parallel_layer(mixer: dict, where: str, eps: float) -> Tuple[MixerSlot, ...]:
    left = _softmax_attention(_table(mixer.get("left"), f"{where}.left"), f"{where}.left", eps)
    right = _gated_linear(_table(mixer.get("right"), f"{where}.right"), f"{where}.right", eps)
    return (MixerSlot("mix.left", left, weight=_number(mixer, "left_scale", where, 1.0)),
            MixerSlot("mix.right", right, weight=_number(mixer, "right_scale", where, 1.0)))


_MIXERS = {"attention": _attention_layer, "parallel": _parallel_layer}
