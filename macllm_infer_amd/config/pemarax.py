"""Pemarax configuration, read from the design's own ``config.json`` keys.

A decoder whose layers are listed one by one (``layers``).  A layer is pre-norm with an RMS norm whose weight is
stored around zero, one mixer and (``mlp`` with ``kind`` ``moe``, or null) a mixture of experts; each branch is
multiplied by ``residual_mult`` where it joins the float32 stream.  Mixers (``type``):

``attention``         grouped-query attention with a short causal convolution behind the q, k and v projections
                      (``conv`` taps), neighbouring-pair rotation of the first ``rot.dims`` dims with ramp-blended
                      frequencies (``rot.scaling``: factor, original, fast, slow), q and k divided by their root mean
                      square head by head after the rotation, a window of ``mask.size`` keys that also keeps the
                      first ``mask.keep_first`` tokens of the sequence, and a softmax with one more in its denominator.
``latent_attention``  queries projected directly, keys and values through one latent of ``kv_rank`` numbers and one
                      shared turned key part of ``rot_dim`` (half-split pairs); a window of ``mask.size`` keys.
``parallel``          ``left``: windowed grouped-query attention without rotation whose q and k heads are RMS-normed
                      with one weight for all heads; ``right``: a Mamba-2 state-space mixer (``heads``, ``vdim``,
                      ``state``, ``groups``, ``conv``, ``norm_groups``).  Each output is RMS-normed over the model
                      width with a weight of its own; the layer takes half their sum.

The experts are down(max(up(x), 0)^2); the router's logits get a bias, the ``top`` largest are chosen and weighted
by the softmax over the chosen logits.

Tensors are stored without ``.weight``: ``l<i>.mix.q``, ``l<i>.mix.q.conv``, ``l<i>.mix.left.q.norm``,
``l<i>.mix.right.in``, ``l<i>.mix.right.conv.b``, ``l<i>.mix.left.out``, ``l<i>.mlp.router.b``, ``l<i>.mlp.e<k>.up``,
``l<i>.norm1``, ``embed``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from .mukutar import _integer, _number, _table
from .spec import (AttentionSpec, ConfigError, InterleavedRopeSpec, LatentAttentionSpec, LayerSpec, Mamba2Spec, MixerSlot,
                   ModelSpec, NoPositionSpec, PowerReluSpec, RampScalingSpec, RmsNormSpec, RopeSpec, RoutedExpertsSpec,
                   ScheduleEntry, _require)

# a tensor's name in the model -> the name it is stored under
STORED_NAME_RULES = ((r"\.(q|k)_norm\.weight$", r".\1.norm"), (r"\.in_proj\.", ".in."), (r"\.out_proj\.", ".o."),
                     (r"\.conv1d\.", ".conv."), (r"_proj\.", "."), (r"\.weight$", ""), (r"\.bias$", ".b"))

FIELD_NAMES = (("attention.head_dim", "layers[].mixer.dim"), ("attention.num_heads", "layers[].mixer.heads"),
               ("latent_attention.cached_key_dim", "layers[].mixer.kv_rank + rot_dim"),
               ("latent_attention.num_heads", "layers[].mixer.heads"),
               ("mamba2.state_size", "layers[].mixer.right.state"), ("mamba2.conv_kernel", "layers[].mixer.right.conv"),
               ("mamba2.num_heads", "layers[].mixer.right.heads"), ("mamba2.num_groups", "layers[].mixer.right.groups"),
               ("routed_experts.num_experts", "layers[].mlp.router.experts"), ("rmsnorm.hidden_size", "width"))

DEFAULT_MAX_CONTEXT = 1 << 20       # the design names no limit: the longest the engine's tables index
SCAN_CHUNK = 128                    # tokens of a chunk of the state-space scan over prompt portions (the result does not depend on it)


@dataclass(frozen=True)
class PemaraxLayer:
    type: str
    mixers: Tuple[MixerSlot, ...]       # one mixer, or the two of a parallel layer
    mlp: Optional[object]               # the feed-forward's spec, None for a layer without one
    raw: dict                           # the layer's own table, for ``to_dict``


@dataclass(frozen=True)
class PemaraxConfig:
    width: int
    vocab: int
    norm_eps: float
    residual_mult: float
    layers: Tuple[PemaraxLayer, ...]
    max_context: int = DEFAULT_MAX_CONTEXT
    eos_token_id: Optional[int] = None

    architecture_names = ("Pemarax", "pemarax")

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, raw: dict) -> "PemaraxConfig":
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
            reader = _MIXERS.get(kind)
            if reader is None:
                raise ConfigError(f"config.json: '{where}.type' is {kind!r}; known: {sorted(_MIXERS)}")
            mixers = reader(_table(entry.get("mixer"), f"{where}.mixer"), f"{where}.mixer", eps)
            mlp = None
            if entry.get("mlp") is not None:
                table = _table(entry["mlp"], f"{where}.mlp")
                if table.get("kind", "moe") not in _FEED_FORWARDS:
                    raise ConfigError(f"config.json: '{where}.mlp.kind' is {table.get('kind')!r}; "
                                      f"known: {sorted(_FEED_FORWARDS)}")
                mlp = _FEED_FORWARDS[table.get("kind", "moe")](table, f"{where}.mlp")
            layers.append(PemaraxLayer(kind, mixers, mlp, entry))
        eos = raw.get("eos_token_id")
        config = cls(width=width, vocab=vocab, norm_eps=eps, residual_mult=_number(raw, "residual_mult", "", 1.0),
                     layers=tuple(layers), max_context=_integer(raw, "max_context", "", DEFAULT_MAX_CONTEXT),
                     eos_token_id=eos if isinstance(eos, int) and not isinstance(eos, bool) else None)
        config.validate()
        return config

    def to_dict(self) -> dict:
        out = {"architecture": "Pemarax", "layers": [layer.raw for layer in self.layers], "norm": {"eps": self.norm_eps},
               "residual_mult": self.residual_mult, "vocab": self.vocab, "width": self.width}
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
            LayerSpec(prefix=f"l{index}", mixers=layer.mixers, ffn=layer.mlp, mixer_norm=norm, ffn_norm=norm,
                      mixer_norm_name="norm1", ffn_norm_name="norm2", ffn_name="mlp",
                      branch_multiplier=self.residual_mult)
            for index, layer in enumerate(self.layers))
        return ModelSpec(
            architecture="Pemarax", hidden_size=self.width, vocab_size=self.vocab, max_context=self.max_context,
            layers=layers, schedule=tuple(ScheduleEntry(layer=index) for index in range(len(layers))),
            final_norm=norm, embedding_name="embed", final_norm_name="final.norm", lm_head_name="head",
            root_namespace="", stored_name_rules=STORED_NAME_RULES, field_names=FIELD_NAMES)

    # ------------------------------------------------------------------ reports
    def _mixer_specs(self):
        return [slot.spec for layer in self.layers for slot in layer.mixers]

    def kv_bytes_per_token(self, bytes_per_element: int) -> int:
        """What every attention mixer caches for one token (windows bound how many tokens are kept, not this)."""
        total = 0
        for spec in self._mixer_specs():
            if isinstance(spec, AttentionSpec):
                total += spec.num_kv_heads * (spec.head_dim + spec.value_width) * bytes_per_element
            elif isinstance(spec, LatentAttentionSpec):
                total += (spec.cached_key_dim + spec.kv_rank) * bytes_per_element
        return total

    def fixed_state_bytes(self, bytes_per_element: int) -> int:
        """The convolutions' tails and the float32 state-space states of one request."""
        total = 0
        for spec in self._mixer_specs():
            if isinstance(spec, AttentionSpec) and spec.conv_kernel > 1:
                columns = spec.num_heads * spec.head_dim + spec.num_kv_heads * (spec.head_dim + spec.value_width)
                total += (spec.conv_kernel - 1) * columns * bytes_per_element
            elif isinstance(spec, Mamba2Spec):
                total += (spec.conv_kernel - 1) * spec.conv_width * bytes_per_element
                total += spec.num_heads * spec.head_dim * spec.state_size * 4
        return total


def _window(mixer: dict, where: str):
    """(window or None, first tokens kept) of ``mask``."""
    if mixer.get("mask") is None:
        return None, 0
    mask = _table(mixer["mask"], f"{where}.mask")
    size = mask.get("size")
    window = None if size is None else _integer(mask, "size", f"{where}.mask")
    return window, _integer(mask, "keep_first", f"{where}.mask", 0)


def _ramp_scaling(rot: dict, where: str) -> Optional[RampScalingSpec]:
    if rot.get("scaling") is None:
        return None
    table = _table(rot["scaling"], f"{where}.scaling")
    return RampScalingSpec(factor=_number(table, "factor", f"{where}.scaling"),
                           original=_number(table, "original", f"{where}.scaling"),
                           fast=_number(table, "fast", f"{where}.scaling"),
                           slow=_number(table, "slow", f"{where}.scaling"))


def _attention(mixer: dict, where: str, eps: float) -> Tuple[MixerSlot, ...]:
    heads = _integer(mixer, "heads", where)
    dim = _integer(mixer, "dim", where)
    position = NoPositionSpec()
    if mixer.get("rot") is not None:
        rot = _table(mixer["rot"], f"{where}.rot")
        position = InterleavedRopeSpec(theta=_number(rot, "base", f"{where}.rot"),
                                       rotary_dim=_integer(rot, "dims", f"{where}.rot", dim),
                                       scaling=_ramp_scaling(rot, f"{where}.rot"))
    window, keep_first = _window(mixer, where)
    spec = AttentionSpec(num_heads=heads, num_kv_heads=_integer(mixer, "kv_heads", where, heads), head_dim=dim,
                         scale=_number(mixer, "scale", where), position=position, window=window,
                         keep_first=keep_first if window is not None else 0,
                         value_dim=_integer(mixer, "vdim", where, dim), fixed_sink=0.0,
                         conv_kernel=_integer(mixer, "conv", where, 0), head_norm="after_rotation",
                         head_norm_weight=False, head_norm_eps=eps)
    return (MixerSlot("mix", spec),)


def _latent_attention(mixer: dict, where: str, eps: float) -> Tuple[MixerSlot, ...]:
    rope_dim = _integer(mixer, "rot_dim", where, 0)
    position = NoPositionSpec()
    if rope_dim and mixer.get("rot") is not None:
        rot = _table(mixer["rot"], f"{where}.rot")
        position = RopeSpec(theta=_number(rot, "base", f"{where}.rot"),
                            rotary_dim=_integer(rot, "dims", f"{where}.rot", rope_dim))
    dim = _integer(mixer, "dim", where)
    window, _ = _window(mixer, where)
    spec = LatentAttentionSpec(num_heads=_integer(mixer, "heads", where), head_dim=dim, rope_dim=rope_dim,
                               value_dim=_integer(mixer, "vdim", where, dim), q_rank=None,
                               kv_rank=_integer(mixer, "kv_rank", where), scale=_number(mixer, "scale", where),
                               norm_eps=eps, position=position, window=window)
    return (MixerSlot("mix", spec),)


def _normed_attention(mixer: dict, where: str, eps: float) -> AttentionSpec:
    heads = _integer(mixer, "heads", where)
    dim = _integer(mixer, "dim", where)
    window, keep_first = _window(mixer, where)
    return AttentionSpec(num_heads=heads, num_kv_heads=_integer(mixer, "kv_heads", where, heads), head_dim=dim,
                         scale=_number(mixer, "scale", where), window=window,
                         keep_first=keep_first if window is not None else 0,
                         value_dim=_integer(mixer, "vdim", where, dim), head_norm="before_rotation",
                         head_norm_weight=True, head_norm_eps=eps)


def _state_space(mixer: dict, where: str, eps: float) -> Mamba2Spec:
    groups = _integer(mixer, "groups", where, 1)
    return Mamba2Spec(num_heads=_integer(mixer, "heads", where), head_dim=_integer(mixer, "vdim", where),
                      state_size=_integer(mixer, "state", where), num_groups=groups,
                      conv_kernel=_integer(mixer, "conv", where), chunk_size=SCAN_CHUNK, norm_eps=eps, conv_bias=True,
                      gated_norm=True, norm_groups=_integer(mixer, "norm_groups", where, 1))


def _parallel(mixer: dict, where: str, eps: float) -> Tuple[MixerSlot, ...]:
    left = _normed_attention(_table(mixer.get("left"), f"{where}.left"), f"{where}.left", eps)
    right = _state_space(_table(mixer.get("right"), f"{where}.right"), f"{where}.right", eps)
    out_norm = RmsNormSpec(eps=eps)
    return (MixerSlot("mix.left", left, weight=0.5, post_norm=out_norm, post_norm_name="out"),
            MixerSlot("mix.right", right, weight=0.5, post_norm=out_norm, post_norm_name="out"))


def _moe(mlp: dict, where: str) -> RoutedExpertsSpec:
    expert = _table(mlp.get("expert"), f"{where}.expert")
    router = _table(mlp.get("router"), f"{where}.router")
    return RoutedExpertsSpec(num_experts=_integer(router, "experts", f"{where}.router"),
                             top_k=_integer(router, "top", f"{where}.router"),
                             expert_size=_integer(expert, "ff", f"{where}.expert"), activation=PowerReluSpec(),
                             routing="top_then_softmax")


_MIXERS = {"attention": _attention, "latent_attention": _latent_attention, "parallel": _parallel}
_FEED_FORWARDS = {"moe": _moe}
