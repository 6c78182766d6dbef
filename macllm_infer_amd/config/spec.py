"""Typed, format-neutral description of a decoder: which parts each layer is made of,
with every size and constant as a field, and the order in which layers run.

An architecture's config class (for example ``FalconH1Config``) lowers its own
``config.json`` keys to a ``ModelSpec``; the engine only ever sees the spec.  The
reference keeps the same split between a typed spec and family adapters
(src/architecture.rs:342-364 ``DecoderSpec``, :254-265 ``DecoderLayerSpec``,
:139-151 ``AttentionSpec``, :201-212 ``Mamba2Spec``, :51-62 ``RopeSpec``).

Every part spec carries a ``kind`` string; ``parts.registry`` maps kinds to the
classes that run them, so a new mixer, feed-forward, norm or position encoding is a
new spec dataclass plus a registered class, with no change here.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


class ConfigError(ValueError):
    """A configuration value is missing, malformed or unsupported; the message names the field."""


def _require(condition: bool, message: str) -> None:
    if not condition:
        raise ConfigError(message)


@dataclass(frozen=True)
class WavelengthScalingSpec:
    """Frequencies stretched by their wavelength l = 2 pi / f against a context of ``original`` tokens: kept where
    l < original / high, divided by ``factor`` where l > original / low, and between the two blended,
    (1 - s) f / factor + s f with s = (original / l - low) / (high - low)."""
    factor: float
    low: float
    high: float
    original: float

    def validate(self) -> None:
        _require(self.factor > 0 and self.original > 0, "rope scaling needs a positive factor and original context")
        _require(self.high != self.low, "rope scaling needs two different bounds (low, high)")


@dataclass(frozen=True)
class RampScalingSpec:
    """Frequencies blended with their ``factor``-th part by a ramp over the pair index i (YaRN): with
    where(t) = dims * ln(original / (2 pi t)) / (2 ln theta), lo = max(floor(where(fast)), 0),
    hi = min(ceil(where(slow)), dims - 1) and ramp_i = clamp((i - lo) / max(hi - lo, ``min_span``), 0, 1) the
    frequency is f_i / factor * ramp_i + f_i * (1 - ramp_i); cosines and sines are multiplied by
    ``magnitude_slope`` * ln(factor) + 1."""
    factor: float
    original: float
    fast: float
    slow: float
    magnitude_slope: float = 0.1
    min_span: float = 0.001

    def validate(self) -> None:
        _require(self.factor > 0 and self.original > 0, "rope scaling needs a positive factor and original context")
        _require(self.fast > 0 and self.slow > 0, "rope scaling needs positive numbers of turns (fast, slow)")

    @property
    def magnitude(self) -> float:
        import math
        return self.magnitude_slope * math.log(self.factor) + 1.0


@dataclass(frozen=True)
class RopeSpec:
    """Half-split rotary position encoding of the first ``rotary_dim`` dims of a head
    (src/architecture.rs:44-62).  ``scaling``: the frequencies are stretched by wavelength
    (``WavelengthScalingSpec``) or blended by a ramp (``RampScalingSpec``); None: as they are."""
    theta: float
    rotary_dim: int
    scaling: Optional[object] = None
    kind: str = "rope"

    def validate(self, head_dim: int) -> None:
        _require(self.theta > 0 and self.theta == self.theta and self.theta != float("inf"),
                 f"rope theta must be finite and positive, got {self.theta}")
        _require(0 < self.rotary_dim <= head_dim and self.rotary_dim % 2 == 0,
                 f"rotary_dim {self.rotary_dim} must be even and in 2..={head_dim}")
        if self.scaling is not None:
            self.scaling.validate()


@dataclass(frozen=True)
class NoPositionSpec:
    """No position encoding: q and k are used as projected."""
    kind: str = "none"

    def validate(self, head_dim: int) -> None:
        return None


@dataclass(frozen=True)
class RmsNormSpec:
    """``weight_offset``: what is added to the stored weight (1.0 for a weight stored around zero)."""
    eps: float
    weight_offset: float = 0.0
    kind: str = "rmsnorm"

    def validate(self) -> None:
        _require(self.eps > 0, f"norm eps must be positive, got {self.eps}")


@dataclass(frozen=True)
class InterleavedRopeSpec:
    """Rotary position encoding whose pairs are neighbours: dimension 2i turns with dimension 2i + 1, i below
    ``rotary_dim`` / 2, by the angle position * theta^(-2i / rotary_dim); dimensions from ``rotary_dim`` on pass
    unchanged.  ``scaling``: as for ``RopeSpec``."""
    theta: float
    rotary_dim: int
    scaling: Optional[object] = None
    kind: str = "rope_interleaved"

    def validate(self, head_dim: int) -> None:
        _require(self.theta > 0 and self.theta == self.theta and self.theta != float("inf"),
                 f"rope theta must be finite and positive, got {self.theta}")
        _require(0 < self.rotary_dim <= head_dim and self.rotary_dim % 2 == 0,
                 f"rotary_dim {self.rotary_dim} must be even and in 2..={head_dim}")
        if self.scaling is not None:
            self.scaling.validate()


@dataclass(frozen=True)
class LayerNormSpec:
    """y = (x - mean) / sqrt(variance + eps) * weight + bias, the variance the mean of the squared deviations."""
    eps: float
    kind: str = "layernorm"

    def validate(self) -> None:
        _require(self.eps > 0, f"norm eps must be positive, got {self.eps}")


@dataclass(frozen=True)
class LogDistanceBiasSpec:
    """No rotation; the score of a key at distance n behind the query loses r1 * ln(1 + r2 * n), with r1 and
    r2 learned numbers of each query head (tensors ``r1`` and ``r2`` of the mixer)."""
    num_heads: int
    kind: str = "log_distance"

    def validate(self, head_dim: int) -> None:
        _require(self.num_heads > 0, "a distance bias needs the number of query heads")


@dataclass(frozen=True)
class AttentionSpec:
    """Grouped-query causal attention (src/architecture.rs:139-151).

    ``window``: None = every earlier key; w = the w most recent keys, the query's own
    included (a key is masked when query - key >= w, src/decoder.rs:4521-4526).
    ``value_dim``: values may be narrower or wider than keys.  ``sink``: a learned number per query
    head that takes part in the softmax's denominator without a key or a value.
    Multipliers scale the normed input, the key projection's output and the output
    projection's output.
    """
    num_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float
    position: object = field(default_factory=NoPositionSpec)
    window: Optional[int] = None
    qkv_bias: bool = False
    out_bias: bool = False
    in_multiplier: float = 1.0
    key_multiplier: float = 1.0
    out_multiplier: float = 1.0
    value_dim: Optional[int] = None      # width of a value head (None: the keys' head_dim)
    sink: bool = False                   # one more term exp(sink[head]) in the softmax's denominator (tensor ``sink``)
    # the values are the keys as projected (before any norm's successor, rotation or scaling of the keys): no v_proj
    values_from_keys: bool = False
    # a learned number per query head that multiplies its scores (tensor ``temp``)
    head_temperature: bool = False
    # "softmax": weights normalized over the visible keys; "sigmoid": every visible key weighs
    # sigmoid(score + score_bias[head]) on its own, nothing is normalized (tensor ``pb`` when ``score_bias``)
    weighting: str = "softmax"
    score_bias: bool = False
    # RMS norm (plain weights ``q_norm`` / ``k_norm``, this eps) over ALL rows of the q projection at once, and of
    # the k projection, before the heads are split and before rotation; None: no such norm
    projection_norm_eps: Optional[float] = None
    # values are turned by their position over all their dims (half-split pairs, angle = position *
    # value_rotation_theta^(-2m / value width)) before they are cached, and every head's output is turned back by
    # its query's position; None: values as projected
    value_rotation_theta: Optional[float] = None
    # with a window: keys at positions below ``keep_first`` stay visible to every later query, at their true
    # positions, however far the window has moved on
    keep_first: int = 0
    # a sink whose score is this fixed number (no tensor): exp(fixed_sink) is one more term of the denominator
    fixed_sink: Optional[float] = None
    # a causal convolution over time on every channel of the q, k and v projections, right behind the products
    # (tensors ``q_proj.conv`` ... [channels, taps], no bias, no activation); the last taps - 1 projected rows of a
    # request are part of its state.  0: none
    conv_kernel: int = 0
    # an RMS norm of every q head and every k head over ``head_dim`` (``head_norm_eps`` inside the root):
    # "before_rotation" or "after_rotation"; with ``head_norm_weight`` times a weight of ``head_dim`` numbers that
    # all heads share (tensors ``q_norm`` / ``k_norm``), else the bare division.  None: no such norm
    head_norm: Optional[str] = None
    head_norm_weight: bool = False
    head_norm_eps: float = 1e-6
    kind: str = "attention"

    @property
    def value_width(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim

    def validate(self) -> None:
        _require(self.num_heads > 0 and self.num_kv_heads > 0,
                 "attention head counts must be positive")
        _require(self.value_width > 0, "the width of a value head must be positive")
        _require(self.num_heads % self.num_kv_heads == 0,
                 f"num_attention_heads {self.num_heads} is not a multiple of "
                 f"num_key_value_heads {self.num_kv_heads}")
        _require(self.head_dim > 0 and self.head_dim % 2 == 0,
                 f"head_dim {self.head_dim} must be positive and even")
        _require(self.scale > 0, "attention scale must be positive")
        _require(self.window is None or self.window > 0, "attention window must be positive")
        _require(self.weighting in ("softmax", "sigmoid"), f"attention weighting {self.weighting!r} is not known")
        _require(not self.score_bias or self.weighting == "sigmoid", "a bias per head is for sigmoid weights")
        _require(not (self.sink and self.weighting == "sigmoid"), "a sink belongs to a softmax")
        _require(not self.values_from_keys or self.value_width == self.head_dim,
                 "values that are the keys have the keys' width")
        _require(self.projection_norm_eps is None or self.projection_norm_eps > 0, "the projections' norm eps must be positive")
        if self.value_rotation_theta is not None:
            _require(self.value_rotation_theta > 0 and self.value_width % 2 == 0,
                     "turned values need a positive base and an even width")
        _require(self.keep_first >= 0, "the number of first tokens a window keeps cannot be negative")
        _require(self.fixed_sink is None or (not self.sink and self.weighting == "softmax"),
                 "a fixed sink stands in a softmax, in place of a learned one")
        _require(0 <= self.conv_kernel, "the taps of the projections' convolution cannot be negative")
        _require(self.head_norm in (None, "before_rotation", "after_rotation"),
                 f"the heads' norm {self.head_norm!r} is not known")
        _require(self.head_norm is None or self.projection_norm_eps is None,
                 "q and k are normed head by head or as whole projections, not both")
        _require(self.head_norm is None or self.head_norm_eps > 0, "the heads' norm eps must be positive")
        self.position.validate(self.head_dim)


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Causal softmax attention whose queries, keys and values come through low-rank latents.

    Queries: c_q = RMSNorm(W_dq h) [``q_rank``], q = W_uq c_q (``q_rank`` None: q = W_q h, no latent), per head
    ``head_dim`` plain dimensions followed by ``rope_dim`` turned ones.  Keys and values: W_dkv h gives ``kv_rank`` + ``rope_dim`` numbers; the first
    ``kv_rank``, RMS-normed, are the latent c, the rest is one turned key part shared by all heads.  A head's plain
    key is W_uk c, its value W_uv c (``value_dim`` wide); score = (q_plain . k_plain + q_turned . k_turned) *
    ``scale``.  The cache holds c and the turned key part of a token, nothing per head.  ``position`` turns the
    ``rope_dim`` part of q and k."""
    num_heads: int
    head_dim: int
    rope_dim: int
    value_dim: int
    q_rank: Optional[int]
    kv_rank: int
    scale: float
    norm_eps: float
    position: object = field(default_factory=NoPositionSpec)
    window: Optional[int] = None
    kind: str = "latent_attention"

    @property
    def cached_key_dim(self) -> int:
        """What a token's key is in the cache: its latent and the turned part."""
        return self.kv_rank + self.rope_dim

    def validate(self) -> None:
        for name in ("num_heads", "head_dim", "value_dim", "kv_rank"):
            _require(getattr(self, name) > 0, f"latent attention {name} must be positive")
        _require(self.q_rank is None or self.q_rank > 0, "latent attention q_rank must be positive")
        _require(self.rope_dim >= 0, "latent attention rope_dim cannot be negative")
        _require(self.scale > 0, "attention scale must be positive")
        _require(self.norm_eps > 0, "latent attention norm eps must be positive")
        _require(self.window is None or self.window > 0, "attention window must be positive")
        if self.rope_dim:
            self.position.validate(self.rope_dim)


@dataclass(frozen=True)
class ClampedGLUSpec:
    """The activation of a gated feed-forward with clamped branches: g = min(gate, limit),
    u = clamp(up, -limit, limit), y = g * sigmoid(alpha g) * (u + up_offset)."""
    limit: float
    alpha: float = 1.702
    up_offset: float = 1.0

    def validate(self) -> None:
        _require(self.limit > 0 and self.limit == self.limit, "the activation's limit must be positive")


@dataclass(frozen=True)
class PowerReluSpec:
    """The activation of a feed-forward without a gate: act(z) = max(z, 0)^2 (an expert is then
    down(act(up(x))), with no gate matrix)."""
    gated = False

    def validate(self) -> None:
        return None


@dataclass(frozen=True)
class RoutedExpertsSpec:
    """A mixture of ``num_experts`` small feed-forwards (``expert_size`` wide, no biases) of which a token
    uses ``top_k``, and optionally a shared one (``shared_size`` wide) that every token uses, times
    sigmoid(w_sg . x).  An expert is gated (``ClampedGLUSpec``: gate, up, down) or not (``PowerReluSpec``: up, down).
    Router, ``routing`` "softmax_then_top": s = softmax(W_router x) over all experts in float32; the ``top_k``
    largest of s + correction are chosen; their weights are their s divided by the sum of the chosen s
    (+ ``weight_eps``), times ``route_scale``.  ``routing`` "top_then_softmax": the ``top_k`` largest logits
    z = W_router x + bias (tensor ``router.bias``) are chosen and weighted by the softmax over the chosen logits
    alone, times ``route_scale``."""
    num_experts: int
    top_k: int
    expert_size: int
    activation: object
    route_scale: float = 1.0
    weight_eps: float = 1e-20
    shared_size: Optional[int] = None
    shared_activation: Optional[ClampedGLUSpec] = None
    routing: str = "softmax_then_top"
    kind: str = "routed_experts"

    def validate(self) -> None:
        _require(self.num_experts > 0 and self.expert_size > 0, "the experts' number and width must be positive")
        _require(0 < self.top_k <= self.num_experts,
                 f"a token uses {self.top_k} experts of {self.num_experts}")
        _require(self.routing in ("softmax_then_top", "top_then_softmax"), f"routing {self.routing!r} is not known")
        self.activation.validate()
        if self.shared_size is not None:
            _require(self.shared_size > 0 and self.shared_activation is not None,
                     "a shared expert needs a positive width and an activation")
            self.shared_activation.validate()


@dataclass(frozen=True)
class HashedBigramSpec:
    """A second embedding row for every token, picked by a hash of the token and the one before it: row
    (previous * mul_prev + token * mul_cur) mod ``buckets`` of a table of ``buckets`` + 1 rows; a sequence's
    first token takes the last row.  The previous token is part of a request's state."""
    buckets: int
    mul_prev: int
    mul_cur: int

    def validate(self) -> None:
        _require(self.buckets > 0, "the bigram table needs at least one bucket")


@dataclass(frozen=True)
class StreamInjection:
    """What happens to the residual stream right before a schedule entry runs: with ``mix_name`` the stream x
    becomes W [x; x0], W the tensor ``mix_name`` [hidden, 2 hidden] and x0 the embedding output; then the embedding
    output is added once more (``embedding``), and row ``row`` of the tensor ``vector_name`` [rows, hidden]
    (None: no vector)."""
    embedding: bool = False
    vector_name: Optional[str] = None
    row: int = 0
    mix_name: Optional[str] = None


@dataclass(frozen=True)
class Mamba2Spec:
    """Mamba2 state-space mixer (src/architecture.rs:201-212; checks :580-628).

    ``multipliers`` scale the five segments z, x, B, C, dt of the input projection.
    """
    num_heads: int
    head_dim: int
    state_size: int
    num_groups: int
    conv_kernel: int
    chunk_size: int
    norm_eps: float
    conv_bias: bool = True
    proj_bias: bool = False
    gated_norm: bool = False
    in_multiplier: float = 1.0
    out_multiplier: float = 1.0
    multipliers: Tuple[float, float, float, float, float] = (1.0, 1.0, 1.0, 1.0, 1.0)
    # equal parts of the gated rows that the gated norm divides by their own root mean square (None: ``num_groups``)
    norm_groups: Optional[int] = None
    kind: str = "mamba2"

    @property
    def norm_parts(self) -> int:
        return self.num_groups if self.norm_groups is None else self.norm_groups

    @property
    def inner_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def conv_width(self) -> int:
        return self.inner_size + 2 * self.num_groups * self.state_size

    @property
    def projection_width(self) -> int:
        return self.inner_size + self.conv_width + self.num_heads

    def validate(self) -> None:
        for name in ("num_heads", "head_dim", "state_size", "num_groups", "conv_kernel", "chunk_size"):
            _require(getattr(self, name) > 0, f"mamba {name} must be positive")
        _require(self.num_heads % self.num_groups == 0,
                 f"mamba_n_heads {self.num_heads} is not a multiple of mamba_n_groups {self.num_groups}")
        _require(self.inner_size % self.num_groups == 0, "mamba inner size must divide into its groups")
        _require(len(self.multipliers) == 5, "ssm_multipliers must have 5 entries (z, x, B, C, dt)")
        _require(self.norm_eps > 0, "mamba norm eps must be positive")
        _require(self.norm_parts > 0 and self.inner_size % self.norm_parts == 0,
                 "mamba inner size must divide into the parts of its gated norm")


@dataclass(frozen=True)
class RetentionSpec:
    """Linear attention with a fixed decay per head and no softmax: S <- decay[h] S + k v^T, o = S^T q, the
    state [key_dim, value_dim] per head carried in float32.  q and k are turned by ``position`` (a rotation of the
    first dims of a head, or none), k is then multiplied by ``key_scale``; each head's o is divided by its root
    mean square (``norm_eps``), gated by SiLU of a fourth projection and projected out."""
    num_heads: int
    key_dim: int
    value_dim: int
    decay: Tuple[float, ...]
    key_scale: float
    norm_eps: float
    position: object = field(default_factory=NoPositionSpec)
    kind: str = "retention"

    def validate(self) -> None:
        _require(self.num_heads > 0 and self.key_dim > 0 and self.value_dim > 0, "retention sizes must be positive")
        _require(len(self.decay) == self.num_heads,
                 f"retention needs one decay per head: {len(self.decay)} given for {self.num_heads} heads")
        _require(all(d == d and abs(d) != float("inf") for d in self.decay), "retention decays must be finite")
        _require(self.norm_eps > 0, "retention norm eps must be positive")
        self.position.validate(self.key_dim)


@dataclass(frozen=True)
class GeneralDeltaSpec:
    """Generalized delta rule: per head a state S [dim, dim] in float32 with
    S <- diag(w) S - (a * u)(u^T S) + k v^T (u the unit key, both products on the old state), o = S^T r.
    w = exp(-``decay_floor`` * sigmoid(w2 tanh(w1 h) + w0)) per head and key channel, a = sigmoid(a h + bias).
    ``decay_rank``: the inner width of the decay's two projections (None: whatever the stored tensors have)."""
    num_heads: int
    head_dim: int
    norm_eps: float
    decay_floor: float = 0.6065306597126334     # exp(-1/2)
    key_eps: float = 1e-6                        # inside the root of the unit key
    decay_rank: Optional[int] = None
    kind: str = "general_delta"

    def validate(self) -> None:
        _require(self.num_heads > 0 and self.head_dim > 0, "general_delta sizes must be positive")
        _require(self.decay_rank is None or self.decay_rank > 0, "general_delta decay_rank must be positive")
        _require(self.norm_eps > 0 and self.key_eps > 0, "general_delta eps must be positive")


@dataclass(frozen=True)
class GatedLinearAttentionSpec:
    """Linear attention whose state decays per key channel by a gate of the token: per head
    S <- diag(alpha) S + k v^T, o = S^T q, with q = (W_q h) * ``query_scale``, k = W_k h, v = W_v h and
    alpha = sigmoid(z)^(1 / ``decay_temperature``), z = W_a2 (W_a1 h) + bias, one number per head and key channel.
    Each head's o is divided by its root mean square (``norm_eps``) and multiplied by a weight of ``value_dim``
    numbers that all heads share, then by SiLU of a gate projection, and projected out.  ``decay_rank``: the inner
    width of the gate's two projections (None: whatever the stored tensors have)."""
    num_heads: int
    key_dim: int
    value_dim: int
    decay_temperature: float
    query_scale: float
    norm_eps: float
    decay_rank: Optional[int] = None
    kind: str = "gated_linear_attention"

    def validate(self) -> None:
        _require(self.num_heads > 0 and self.key_dim > 0 and self.value_dim > 0,
                 "gated linear attention sizes must be positive")
        _require(self.decay_temperature > 0, "the decay's temperature must be positive")
        _require(self.decay_rank is None or self.decay_rank > 0, "the decay's inner width must be positive")
        _require(self.norm_eps > 0, "the norm eps must be positive")


@dataclass(frozen=True)
class PolyNormFFNSpec:
    """down(act(up(x))) with act(z) = c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3, powers element by element, N the
    division of a token's row by its root mean square (``eps``); the four numbers are the tensor ``act``."""
    intermediate_size: int
    eps: float
    kind: str = "polynorm_ffn"

    def validate(self) -> None:
        _require(self.intermediate_size > 0, "the feed-forward width must be positive")
        _require(self.eps > 0, "the feed-forward's norm eps must be positive")


@dataclass(frozen=True)
class SwiGLUSpec:
    """down(act(gate(x) * gate_multiplier) * up(x)) * down_multiplier (src/decoder.rs:261-306), act = SiLU or,
    with ``activation`` "gelu_tanh", 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3)))."""
    intermediate_size: int
    bias: bool = False
    gate_multiplier: float = 1.0
    down_multiplier: float = 1.0
    activation: str = "silu"
    kind: str = "swiglu"

    def validate(self) -> None:
        _require(self.intermediate_size > 0, "intermediate_size must be positive")
        _require(self.activation in ("silu", "gelu_tanh"), f"the gate's activation {self.activation!r} is not known")


@dataclass(frozen=True)
class MixerSlot:
    """One mixer of a layer: the sub-path of its tensors and its spec.  ``weight``: the number its output is
    multiplied by (in float32) where the layer's mixers are summed."""
    name: str
    spec: object
    weight: float = 1.0
    # an RMS norm of the mixer's output over the model width (``RmsNormSpec``, tensor ``<name>.<post_norm_name>``)
    # before the weighted sum of the layer's mixers; None: the output as it is
    post_norm: object = None
    post_norm_name: str = "out"


@dataclass(frozen=True)
class LayerSpec:
    """One layer's parts and their arrangement.

    ``arrangement`` "parallel_prenorm": n = norm(h); h += sum of mixers(n);
    h += ffn(norm(h)) (src/decoder.rs:2658-2699).  One mixer gives the ordinary
    sequential pre-norm layer.  ``prefix`` is the tensor-name path of the layer;
    ``mixer_norm_name`` / ``ffn_norm_name`` / ``ffn_name`` the sub-paths below it
    (src/architecture.rs:1543-1567, :1639-1647).  ``ffn`` None: the layer is its mixers alone (a checkpoint may
    still hold the second norm and scale of such a layer; they are not used).
    """
    prefix: str
    mixers: Tuple[MixerSlot, ...]
    ffn: object
    mixer_norm: object
    ffn_norm: object
    mixer_norm_name: str = "attn_norm"
    ffn_norm_name: str = "ffn_norm"
    ffn_name: str = "mlp"
    arrangement: str = "parallel_prenorm"
    # tensors [hidden] that multiply the mixers' summed output / the feed-forward's output, feature by feature,
    # before it is added to the residual stream (None: no such scale)
    mixer_scale_name: Optional[str] = None
    ffn_scale_name: Optional[str] = None
    # one number that multiplies every branch where it joins the stream (x <- x + m * branch), applied in float32
    branch_multiplier: float = 1.0
    # arrangement "sandwich": a second norm on each branch before it joins the stream,
    # x <- x + mixer_post_norm(sum of mixers(mixer_norm(x))), x <- x + ffn_post_norm(ffn(ffn_norm(x)))
    mixer_post_norm: object = None
    ffn_post_norm: object = None
    mixer_post_norm_name: str = "norm1b"
    ffn_post_norm_name: str = "norm2b"


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.  ``layer`` indexes ``ModelSpec.layers`` (a layer may be named by
    several entries: its weights run again, with a cache of their own).  ``kv_from``
    names an earlier entry whose attention cache this run reads instead of writing one
    of its own (only mixers whose cache is token-proportional can do that)."""
    layer: int
    kv_from: Optional[int] = None
    before: Optional[StreamInjection] = None      # added to the stream right before this run


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_context: int
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: object
    tied_embeddings: bool = False
    embedding_multiplier: float = 1.0
    logit_multiplier: float = 1.0
    # logits <- cap * tanh(logits / cap) after their scaling (src/decoder.rs:3349-3355, 4791-4796); None: no cap
    logit_softcap: Optional[float] = None
    bigram: Optional[HashedBigramSpec] = None      # a hashed bigram row added to every token's embedding
    bigram_name: str = "bigram"
    # tensors [rows, hidden] that schedule entries name (``StreamInjection.vector_name``): (name, rows)
    injected_vectors: Tuple[Tuple[str, int], ...] = ()
    # tensors [hidden, 2 hidden] that schedule entries name (``StreamInjection.mix_name``)
    injected_mixes: Tuple[str, ...] = ()
    embedding_name: str = "model.embed_tokens"
    final_norm_name: str = "model.norm"
    lm_head_name: str = "lm_head"
    # other spellings under which checkpoints of this architecture store the same tensors:
    # (piece of a stored name, the piece it stands for here)
    tensor_aliases: Tuple[Tuple[str, str], ...] = ()
    # a checkpoint none of whose names starts with this gets it in front of all but the output head's
    root_namespace: str = "model."
    # (regular expression, replacement) pairs that turn a tensor's name in the model into the name the
    # architecture's checkpoints store it under, applied in order (``stored_name``)
    stored_name_rules: Tuple[Tuple[str, str], ...] = ()
    # ("part kind.spec field", the configuration file's key for it): for messages that name a field
    field_names: Tuple[Tuple[str, str], ...] = ()

    def stored_name(self, name: str) -> str:
        """The name under which the architecture's checkpoints hold the model's tensor ``name``."""
        import re
        for pattern, replacement in self.stored_name_rules:
            name = re.sub(pattern, replacement, name)
        return name

    def validate(self) -> None:
        """Positivity, divisibility and bounds, field by field (src/architecture.rs:367-452)."""
        _require(self.hidden_size > 0, "hidden_size must be positive")
        _require(self.vocab_size > 0, "vocab_size must be positive")
        _require(0 < self.max_context <= (1 << 20),
                 f"max_position_embeddings {self.max_context} must be in 1..=2^20")
        _require(0 < len(self.layers) <= 4096, "num_hidden_layers must be in 1..=4096")
        _require(len(self.schedule) > 0, "the schedule of layers is empty")
        _require(self.logit_softcap is None or (0 < self.logit_softcap < float("inf")),
                 f"the cap on the logits must be finite and positive, got {self.logit_softcap}")
        self.final_norm.validate()
        if self.bigram is not None:
            self.bigram.validate()
        vectors = dict(self.injected_vectors)
        for index, entry in enumerate(self.schedule):
            if entry.before is not None and entry.before.vector_name is not None:
                _require(entry.before.vector_name in vectors
                         and 0 <= entry.before.row < vectors[entry.before.vector_name],
                         f"schedule entry {index} adds a row of a vector table that the model does not have")
            if entry.before is not None and entry.before.mix_name is not None:
                _require(entry.before.mix_name in self.injected_mixes,
                         f"schedule entry {index} mixes the stream with a matrix that the model does not have")
        for layer in self.layers:
            _require(len(layer.mixers) > 0, f"layer {layer.prefix} has no mixer")
            names = [slot.name for slot in layer.mixers]
            _require(len(set(names)) == len(names), f"layer {layer.prefix} names a mixer twice")
            for slot in layer.mixers:
                slot.spec.validate()
                if slot.post_norm is not None:
                    slot.post_norm.validate()
            layer.mixer_norm.validate()
            if layer.mixer_post_norm is not None:
                layer.mixer_post_norm.validate()
            if layer.ffn is not None:
                layer.ffn.validate()
                layer.ffn_norm.validate()
                if layer.ffn_post_norm is not None:
                    layer.ffn_post_norm.validate()
        for index, entry in enumerate(self.schedule):
            _require(0 <= entry.layer < len(self.layers),
                     f"schedule entry {index} names layer {entry.layer}, which does not exist")
            if entry.kv_from is not None:
                _require(0 <= entry.kv_from < index,
                         f"schedule entry {index} reads the cache of entry {entry.kv_from}, "
                         "which does not run before it")
                _require(self.schedule[entry.kv_from].kv_from is None,
                         f"schedule entry {index} reads the cache of an entry that owns none")
