"""Position encodings: transforms of q and k before the cache write, and biases on the attention scores."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import Expect
from .base import BuildContext, Part, register_part


class PositionEncoding(Part):
    """Interface: ``rotate_and_store`` encodes the absolute positions ``step.positions`` into
    the q and k heads of ``qkv`` (q in place) and, if ``cache.owns_kv``, writes the encoded
    k and the raw v of every token into the cache cell ``step.slot_mappings[cache.group]``.
    A subclass may implement only ``rotate`` (in place on ``qkv``); the store is then done
    by the cache-write kernel without rotation.

    An encoding that (also) biases the scores by distance sets ``score_slopes``: a float32 tensor [query heads]
    on the device, with score(head, query at s, key at p) -= score_slopes[head] * (s - p).  The attention part
    then takes its general kernel, which knows the term; the matrix-core and fused decode kernels do not.
    A bias that grows with the logarithm of the distance sets ``score_log_bias`` instead: float32 [query heads, 2]
    = (r1, r2) with score -= r1 * ln(1 + r2 * (s - p)).  An encoding with tensors of its own sets ``learned``; it
    then declares them (``expected_tensors(spec, prefix, hidden_size)``, beside the mixer's) and is built with
    ``prefix`` and ``tensors``."""
    kernel_modules = ("attention",)
    score_slopes = None
    score_log_bias = None
    learned = False

    def fused_rotation(self):
        """What a kernel that rotates q and the new key itself has to apply in place of ``rotate_and_store``:
        ``(inv_freq, rotary_dim)`` of a half-split rotation by position * inv_freq[j] of the first ``rotary_dim``
        dimensions of every head (``(None, 0)``: nothing), or None when the encoding is no such rotation; the
        layer then runs this part's own ``rotate_and_store`` and the general kernels."""
        return None

    # what the cosines and sines of a rotation are multiplied by (a scaling of the frequencies may bring one)
    magnitude = 1.0

    def pair_rotation(self):
        """``(inv_freq or None, rotary_dim, interleaved)`` of an encoding that turns pairs of dimensions by
        position * inv_freq[i]: pair i is dimensions (i, i + rotary_dim / 2) (half-split) or (2i, 2i + 1)
        (``interleaved``); ``(None, 0, False)``: nothing is turned.  None: the encoding is no such rotation.  For
        mixers whose kernels turn a part of their rows themselves."""
        return None

    def rotate(self, qkv, num_heads, num_kv_heads, head_dim, step) -> None:
        return None

    def rotate_and_store(self, qkv, num_heads, num_kv_heads, head_dim, step, cache) -> None:
        self.rotate(qkv, num_heads, num_kv_heads, head_dim, step)
        if cache.owns_kv:
            ops.rope_kv_store(qkv, num_heads, num_kv_heads, head_dim, step.positions, None, 0,
                              step.slot_mappings[cache.group], cache.k_cache, cache.v_cache)


@register_part("none")
class NoPosition(PositionEncoding):
    graph_safe = True

    def __init__(self, spec, head_dim: int, build: BuildContext):
        pass

    def fused_rotation(self):
        return None, 0

    def pair_rotation(self):
        return None, 0, False


def rotary_frequencies(theta: float, rotary_dim: int, scaling=None) -> list:
    """f_j = theta^(-2j / rotary_dim), j below rotary_dim / 2, in float64; with ``scaling`` (factor, low, high,
    original) stretched by wavelength l = 2 pi / f: kept where l < original / high, f / factor where
    l > original / low, between the two (1 - s) f / factor + s f with s = (original / l - low) / (high - low).
    A ``scaling`` with ``fast`` and ``slow`` (``RampScalingSpec``) blends f_j with f_j / factor by a ramp over j."""
    import math
    frequencies = [1.0 / (theta ** (index / rotary_dim)) for index in range(0, rotary_dim, 2)]
    if scaling is None:
        return frequencies
    if hasattr(scaling, "fast"):
        # blended by a ramp over the pair index: where(t) = dims ln(original / (2 pi t)) / (2 ln theta) is the index
        # of the pair that makes t turns over the original context
        def where(turns: float) -> float:
            return rotary_dim * math.log(scaling.original / (2.0 * math.pi * turns)) / (2.0 * math.log(theta))
        low = max(math.floor(where(scaling.fast)), 0)
        high = min(math.ceil(where(scaling.slow)), rotary_dim - 1)
        out = []
        for index, frequency in enumerate(frequencies):
            ramp = min(max((index - low) / max(high - low, scaling.min_span), 0.0), 1.0)
            out.append(frequency / scaling.factor * ramp + frequency * (1.0 - ramp))
        return out
    out = []
    for frequency in frequencies:
        wavelength = 2.0 * math.pi / frequency
        if wavelength < scaling.original / scaling.high:
            out.append(frequency)
        elif wavelength > scaling.original / scaling.low:
            out.append(frequency / scaling.factor)
        else:
            blend = (scaling.original / wavelength - scaling.low) / (scaling.high - scaling.low)
            out.append((1.0 - blend) * frequency / scaling.factor + blend * frequency)
    return out


@register_part("rope")
class Rope(PositionEncoding):
    """Half-split rotary encoding: f_j = theta^(-2j/rotary_dim) formed in float64 (stretched by wavelength when the
    spec says so) and rounded to float32; angle = position * f_j, cos and sin in float32
    (reference: src/decoder.rs:136-144, 186-195, 226-229)."""
    graph_safe = True

    def __init__(self, spec, head_dim: int, build: BuildContext):
        self.rotary_dim = spec.rotary_dim
        scaling = getattr(spec, "scaling", None)
        frequencies = rotary_frequencies(spec.theta, spec.rotary_dim, scaling)
        self.inv_freq = torch.tensor(frequencies, dtype=torch.float64).to(torch.float32).to(build.device)
        self.magnitude = float(getattr(scaling, "magnitude", 1.0))

    def fused_rotation(self):
        if self.magnitude != 1.0:          # the kernels that turn q and k themselves know no magnitude
            return None
        return self.inv_freq, self.rotary_dim

    def pair_rotation(self):
        return self.inv_freq, self.rotary_dim, False

    def rotate_and_store(self, qkv, num_heads, num_kv_heads, head_dim, step, cache) -> None:
        owns = cache.owns_kv
        ops.rope_kv_store(qkv, num_heads, num_kv_heads, head_dim, step.positions, self.inv_freq,
                          self.rotary_dim, step.slot_mappings[cache.group] if owns else None,
                          cache.k_cache if owns else None, cache.v_cache if owns else None)


@register_part("log_distance")
class LogDistanceBias(PositionEncoding):
    """No rotation of q and k: a key n positions behind the query loses r1[head] * ln(1 + r2[head] * n) of its
    score, r1 and r2 learned numbers of each query head (tensors ``r1`` and ``r2`` beside the mixer's)."""
    graph_safe = True
    learned = True

    @classmethod
    def expected_tensors(cls, spec, prefix: str, hidden_size: int):
        return [Expect(f"{prefix}.r1", ((spec.num_heads,),), init="positive"),
                Expect(f"{prefix}.r2", ((spec.num_heads,),), init="positive")]

    def __init__(self, spec, head_dim: int, build: BuildContext, prefix: str = "", tensors=None):
        pair = torch.stack([tensors[f"{prefix}.r1"].to(torch.float32), tensors[f"{prefix}.r2"].to(torch.float32)], dim=1)
        self.score_log_bias = pair.contiguous().to(build.device)

    def fused_rotation(self):
        return None


@register_part("rope_interleaved")
class InterleavedRope(PositionEncoding):
    """Rotary encoding whose pairs are neighbouring dimensions: (u, v) = dimensions (2i, 2i + 1) at position p
    become (u cos a - v sin a, v cos a + u sin a), a = p * theta^(-2i / rotary_dim); frequencies formed in float64
    and rounded to float32, angles, cos and sin in float32.  The mixers that use it turn their rows in kernels of
    their own (``pair_rotation``)."""
    graph_safe = True

    def __init__(self, spec, head_dim: int, build: BuildContext):
        self.rotary_dim = spec.rotary_dim
        scaling = getattr(spec, "scaling", None)
        frequencies = rotary_frequencies(spec.theta, spec.rotary_dim, scaling)
        self.inv_freq = torch.tensor(frequencies, dtype=torch.float64).to(torch.float32).to(build.device)
        self.magnitude = float(getattr(scaling, "magnitude", 1.0))

    def pair_rotation(self):
        return self.inv_freq, self.rotary_dim, True
