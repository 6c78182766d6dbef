"""Grouped-query causal attention over the paged cache."""
from __future__ import annotations

import torch

from ..cache.manager import KVNeed, StateNeed
from ..kernels import ops
from ..kernels.limits import ATTENTION_MAX_HEAD_DIM, CONV_MAX_TAPS, GRID_MOST, beyond
from ..weights.loader import Expect
from .base import BuildContext, Mixer, part_class, register_part
from .linear import Linear
from .position import rotary_frequencies


@register_part("attention")
class Attention(Mixer):
    """q, k, v projections (one fused product) -> position encoding of q and k -> K (encoded)
    and V written to the request's pages -> softmax(q.k * scale) . v over every visible
    cached key -> output projection.
    (reference: src/decoder.rs:1099-1161 projections, :953-962 RoPE and cache write,
    :4580-4670 scores with float32 softmax, :923-931 output; GQA pairing :4641-4647.)

    Values may have a width of their own (``value_dim``), the softmax may hold a sink (``sink``: a learned number
    per query head whose exponential is one more term of the denominator, with no key and no value), and the
    position encoding may be a bias on the scores; all three take the general attention kernel.

    Further forms, each a field of the spec: values that are the keys as projected (no v projection); an RMS norm
    over the whole q and the whole k projection before rotation; values turned by their position before they are
    cached and outputs turned back by the query's; a learned multiplier of every head's scores; sigmoid weights
    with a learned bias per head in place of the softmax; an RMS norm of every q and k head, before or after the
    rotation, with one weight for all heads or none; pairs of neighbouring dimensions turned, cosines and sines
    times a magnitude; a window that keeps a sequence's first keys; a sink of a fixed score; a short causal
    convolution over time behind the q, k and v projections, whose last rows are state of the request.  One kernel
    prepares a token's row for all of them (``ops.attention_prepare``: norms, rotations, cache write).

    Multipliers: ``in_multiplier`` scales the input of q/k/v (folded into their weights),
    ``key_multiplier`` the k projection's output (weights and bias), ``out_multiplier``
    the output projection's output."""
    graph_safe = True
    kernel_modules = ("common", "attention", "gemm", "mamba2")
    query_tile = 64          # tokens of one lane that a workgroup of the prompt attention kernels takes

    @classmethod
    def expected_tensors(cls, spec, prefix: str, hidden_size: int):
        q_rows = spec.num_heads * spec.head_dim
        kv_rows = spec.num_kv_heads * spec.head_dim
        v_rows = spec.num_kv_heads * spec.value_width
        out = [Expect(f"{prefix}.q_proj.weight", ((q_rows, hidden_size),)),
               Expect(f"{prefix}.k_proj.weight", ((kv_rows, hidden_size),))]
        if not spec.values_from_keys:
            out.append(Expect(f"{prefix}.v_proj.weight", ((v_rows, hidden_size),)))
        out.append(Expect(f"{prefix}.o_proj.weight", ((hidden_size, spec.num_heads * spec.value_width),)))
        if spec.qkv_bias:
            out += [Expect(f"{prefix}.q_proj.bias", ((q_rows,),), init="bias"),
                    Expect(f"{prefix}.k_proj.bias", ((kv_rows,),), init="bias")]
            if not spec.values_from_keys:
                out.append(Expect(f"{prefix}.v_proj.bias", ((v_rows,),), init="bias"))
        if spec.out_bias:
            out.append(Expect(f"{prefix}.o_proj.bias", ((hidden_size,),), init="bias"))
        if spec.sink:
            out.append(Expect(f"{prefix}.sink", ((spec.num_heads,),), init="logit"))
        if spec.projection_norm_eps is not None:
            out += [Expect(f"{prefix}.q_norm.weight", ((q_rows,),), init="norm"),
                    Expect(f"{prefix}.k_norm.weight", ((kv_rows,),), init="norm")]
        if spec.head_norm is not None and spec.head_norm_weight:
            out += [Expect(f"{prefix}.q_norm.weight", ((spec.head_dim,),), init="norm"),
                    Expect(f"{prefix}.k_norm.weight", ((spec.head_dim,),), init="norm")]
        if spec.conv_kernel > 0:
            names = (("q_proj", q_rows), ("k_proj", kv_rows)) + (() if spec.values_from_keys else (("v_proj", v_rows),))
            out += [Expect(f"{prefix}.{name}.conv.weight", ((rows, spec.conv_kernel),), init="conv") for name, rows in names]
        if spec.head_temperature:
            out.append(Expect(f"{prefix}.temp", ((spec.num_heads,),), init="positive"))
        if spec.score_bias:
            out.append(Expect(f"{prefix}.pb", ((spec.num_heads,),), init="logit"))
        out += part_class(spec.position).expected_tensors(spec.position, prefix, hidden_size)
        return out

    @classmethod
    def limits(cls, spec, hidden_size: int):
        return (beyond("attention", "head_dim", max(spec.head_dim, spec.value_width), ATTENTION_MAX_HEAD_DIM,
                       "a query row and its sums are kept in LDS and registers")
                + beyond("attention", "num_heads", spec.num_heads, GRID_MOST, "heads index a dimension of the launch")
                + beyond("attention", "conv_kernel", spec.conv_kernel, CONV_MAX_TAPS, "the taps of a channel are kept in registers")
                + part_class(spec.position).limits(spec.position, spec.head_dim))

    @classmethod
    def conv_width(cls, spec) -> int:
        """The channels of the projections' convolution: q, k and v side by side."""
        values = 0 if spec.values_from_keys else spec.num_kv_heads * spec.value_width
        return (spec.num_heads + spec.num_kv_heads) * spec.head_dim + values

    @classmethod
    def cache_needs(cls, spec):
        needs = [KVNeed(spec.num_kv_heads, spec.head_dim, spec.window,
                        None if spec.value_width == spec.head_dim else spec.value_width,
                        spec.keep_first if spec.window else 0)]
        if spec.conv_kernel > 1:       # the last taps - 1 projected rows of the request
            needs.append(StateNeed("conv", (spec.conv_kernel - 1, cls.conv_width(spec)), "activation"))
        return needs

    def __init__(self, spec, prefix: str, tensors, build: BuildContext):
        self.spec = spec
        self.build = build
        q_rows = spec.num_heads * spec.head_dim
        kv_rows = spec.num_kv_heads * spec.head_dim
        v_rows = spec.num_kv_heads * spec.value_width
        get = lambda name: tensors.get(f"{prefix}.{name}")
        if spec.values_from_keys:
            v_rows = 0
        weight_scale = torch.cat([torch.full((q_rows,), spec.in_multiplier),
                                  torch.full((kv_rows,), spec.in_multiplier * spec.key_multiplier),
                                  torch.full((v_rows,), spec.in_multiplier)])
        bias_scale = torch.cat([torch.ones(q_rows), torch.full((kv_rows,), spec.key_multiplier),
                                torch.ones(v_rows)])
        names = ("q_proj", "k_proj") if spec.values_from_keys else ("q_proj", "k_proj", "v_proj")
        self.qkv = Linear([get(f"{name}.weight") for name in names], [get(f"{name}.bias") for name in names], build,
                          weight_scale=weight_scale, bias_scale=bias_scale)
        self.out = Linear([get("o_proj.weight")], [get("o_proj.bias")], build,
                          weight_scale=spec.out_multiplier, bias_scale=spec.out_multiplier)
        position_class = part_class(spec.position)
        if getattr(position_class, "learned", False):        # an encoding with tensors of its own, beside the mixer's
            self.position = position_class(spec.position, spec.head_dim, build, prefix=prefix, tensors=tensors)
        else:
            self.position = position_class(spec.position, spec.head_dim, build)
        f32 = lambda name: get(name).to(torch.float32).contiguous().to(build.device)
        self.sink = f32("sink") if spec.sink else None
        self.fixed_sink = spec.fixed_sink
        # a sink of a fixed score is, to the kernels, a sink tensor with that score for every head
        self.sinks = self.sink
        if spec.fixed_sink is not None:
            self.sinks = torch.full((spec.num_heads,), float(spec.fixed_sink), dtype=torch.float32, device=build.device)
        self.keep_first = int(spec.keep_first) if spec.window else 0
        self.graph_safe = bool(getattr(self.position, "graph_safe", False))
        # the forms that ``ops.attention_prepare`` and the general kernel's extra terms serve
        self.head_scales = f32("temp") if spec.head_temperature else None
        self.score_bias = f32("pb") if spec.score_bias else None
        self.q_norm = f32("q_norm.weight") if spec.projection_norm_eps is not None else None
        self.k_norm = f32("k_norm.weight") if spec.projection_norm_eps is not None else None
        weighted = spec.head_norm is not None and spec.head_norm_weight
        self.q_head_weight = f32("q_norm.weight") if weighted else None
        self.k_head_weight = f32("k_norm.weight") if weighted else None
        self.conv_weight = None
        if spec.conv_kernel > 0:       # the three convolutions as one over the columns [q | k | v], taps in float32
            self.conv_weight = torch.cat([get(f"{name}.conv.weight").to(torch.float32).reshape(-1, spec.conv_kernel)
                                          for name in names]).contiguous().to(build.device)
        self.value_inv_freq = None
        if spec.value_rotation_theta is not None:
            turns = rotary_frequencies(spec.value_rotation_theta, spec.value_width)
            self.value_inv_freq = torch.tensor(turns, dtype=torch.float64).to(torch.float32).to(build.device)
            self.value_inv_freq_back = (-self.value_inv_freq).contiguous()
        pairs = self.position.pair_rotation()
        self.prepared = (spec.values_from_keys or spec.projection_norm_eps is not None
                         or spec.value_rotation_theta is not None or spec.head_temperature
                         or spec.weighting != "softmax" or spec.head_norm is not None or spec.conv_kernel > 0
                         or self.fixed_sink is not None or self.keep_first > 0
                         or (pairs is not None and (pairs[2] or self.position.magnitude != 1.0)))
        self.interleaved = False
        if self.prepared:
            if pairs is None or self.position.score_slopes is not None or self.position.score_log_bias is not None:
                raise ValueError(f"{prefix}: this form of attention turns q and k itself: the position encoding "
                                 f"{spec.position.kind!r} is no rotation by position")
            self.inv_freq, self.rotary_dim, self.interleaved = pairs
        # what only the general kernel knows: a bias on the scores, a sink, values of another width than the keys
        self.general_only = (self.position.score_slopes is not None or self.position.score_log_bias is not None
                             or self.sink is not None or spec.value_width != spec.head_dim or self.prepared)

    def projections(self):
        if self.general_only:          # the fused decode kernels know none of it: the layer runs part by part
            return None
        return self.qkv, self.out, self.spec.num_heads * self.spec.head_dim

    def forward(self, x: torch.Tensor, step, cache) -> torch.Tensor:
        spec = self.spec
        attended = torch.empty((x.shape[0], spec.num_heads * spec.value_width), dtype=x.dtype, device=x.device)
        self.mix(self.qkv(x), step, cache, attended)
        return self.out(attended)

    def mix(self, qkv: torch.Tensor, step, cache, attended: torch.Tensor) -> None:
        """From the projected rows [q | k | v] (rotated and stored in place) to the attended rows
        ``attended`` [T, Hq * dh]; both may be column views of wider matrices."""
        spec = self.spec
        geometry = (spec.num_heads, spec.num_kv_heads, spec.head_dim)
        slopes = self.position.score_slopes
        if self.prepared:
            self.mix_prepared(qkv, step, cache, attended)
            return
        if self.general_only:
            self.position.rotate(qkv, *geometry, step)
            if cache.owns_kv:
                ops.rope_kv_store(qkv, *geometry, step.positions, None, 0, step.slot_mappings[cache.group],
                                  cache.k_cache, cache.v_cache, value_dim=spec.value_width)
            tiles = {}
            if step.max_query_len > 1 and 0 < getattr(step, "query_tile", 0) < (1 << 20):
                tiles = dict(query_tiles=step.query_tiles, tile_tokens=step.query_tile, cu_seqlens=step.cu_seqlens)
            if (tiles and slopes is None and spec.value_width == spec.head_dim and step.query_tile == self.query_tile
                    and ops.prefill_attention_supported(qkv.dtype, *geometry, cache.k_cache.shape[2])
                    and qkv.stride(0) % 8 == 0 and qkv.data_ptr() % 16 == 0 and attended.stride(0) % 4 == 0
                    and attended.data_ptr() % 8 == 0):
                # prompt portions in bfloat16 with heads of 64 or 128: the matrix-core kernel knows the logarithmic
                # bias and the sink
                ops.prefill_attention(qkv, *geometry, cache.k_cache, cache.v_cache, step.block_tables[cache.group],
                                      step.query_tiles, step.cu_seqlens, step.start_pos, spec.scale, spec.window,
                                      attended, step.max_seq_len, log_bias=self.position.score_log_bias,
                                      sinks=self.sink)
                return
            ops.paged_attention(qkv, *geometry, cache.k_cache, cache.v_cache, step.block_tables[cache.group],
                                step.lane_of_token, step.positions, spec.scale, spec.window, attended,
                                step.max_seq_len, slopes, log_bias=self.position.score_log_bias, sinks=self.sink,
                                value_dim=spec.value_width, **tiles)
            return
        self.position.rotate_and_store(qkv, spec.num_heads, spec.num_kv_heads, spec.head_dim, step, cache)
        # lanes of several tokens: the general kernel shares a run of keys among the queries of a tile of the step's
        # table of runs (when the step was packed with one)
        tiles = {}
        if step.max_query_len > 1 and 0 < getattr(step, "query_tile", 0) < (1 << 20):
            tiles = dict(query_tiles=step.query_tiles, tile_tokens=step.query_tile, cu_seqlens=step.cu_seqlens)
        if slopes is not None:                           # a bias on the scores: the general kernel knows it
            ops.paged_attention(qkv, *geometry, cache.k_cache, cache.v_cache, step.block_tables[cache.group],
                                step.lane_of_token, step.positions, spec.scale, spec.window, attended,
                                step.max_seq_len, slopes, **tiles)
        elif step.max_query_len == 1 and ops.decode_attention_supported(qkv.dtype, *geometry, cache.k_cache.shape[2]):
            ops.decode_attention(qkv, *geometry, cache.k_cache, cache.v_cache, step.block_tables[cache.group],
                                 step.lane_of_token, step.positions, spec.scale, spec.window, step.max_seq_len,
                                 attended)
        elif ops.prefill_attention_supported(qkv.dtype, *geometry, cache.k_cache.shape[2]):
            ops.prefill_attention(qkv, *geometry, cache.k_cache, cache.v_cache, step.block_tables[cache.group],
                                  step.query_tiles, step.cu_seqlens, step.start_pos, spec.scale, spec.window,
                                  attended, step.max_seq_len)
        else:
            ops.paged_attention(qkv, *geometry, cache.k_cache, cache.v_cache, step.block_tables[cache.group],
                                step.lane_of_token, step.positions, spec.scale, spec.window, attended,
                                step.max_seq_len, **tiles)

    def mix_prepared(self, qkv: torch.Tensor, step, cache, attended: torch.Tensor) -> None:
        """The forms that go through ``ops.attention_prepare``: one launch norms the q and k projections, turns q
        (in place) and k, turns the values or takes the keys as projected for them, and writes the token's cache
        cells; the attention kernels then see ordinary cached keys and values."""
        spec = self.spec
        geometry = (spec.num_heads, spec.num_kv_heads, spec.head_dim)
        owns = cache.owns_kv
        if self.conv_weight is not None:
            qkv = self.convolve(qkv, step, cache)
        ops.attention_prepare(qkv, *geometry, spec.value_width, step.positions, self.inv_freq, self.rotary_dim,
                              step.slot_mappings[cache.group] if owns else None, cache.k_cache if owns else None,
                              cache.v_cache if owns else None, values_from_keys=spec.values_from_keys,
                              q_norm=self.q_norm, k_norm=self.k_norm, norm_eps=spec.projection_norm_eps or 0.0,
                              value_inv_freq=self.value_inv_freq, interleaved=self.interleaved,
                              turn_scale=self.position.magnitude, head_norm=spec.head_norm,
                              q_head_weight=self.q_head_weight, k_head_weight=self.k_head_weight,
                              head_eps=spec.head_norm_eps if spec.head_norm is not None else 0.0)
        target = attended
        if self.value_inv_freq is not None:         # the heads' outputs are turned back into ``attended`` below
            target = torch.empty((qkv.shape[0], spec.num_heads * spec.value_width), dtype=qkv.dtype, device=qkv.device)
        self.attend_prepared(qkv, step, cache, target)
        if target is not attended:
            ops.rotate_heads(target, 0, spec.value_width, spec.num_heads, spec.value_width, step.positions,
                             self.value_inv_freq_back, spec.value_width, False, attended, 0, spec.value_width)

    def convolve(self, qkv: torch.Tensor, step, cache) -> torch.Tensor:
        """The causal convolution over time of every column of the projected rows [q | k | v], the rows before a
        lane's first token from the request's tail, which then takes the lane's last rows.  Single tokens: in
        place, one launch."""
        width, taps = self.conv_weight.shape
        tail = cache.states["conv"] if taps > 1 else torch.empty((1, 0, width), dtype=qkv.dtype, device=qkv.device)
        if step.max_query_len == 1:
            ops.conv_step(qkv, 0, width, self.conv_weight, None, tail, step.slot_ids, activation=False)
            return qkv
        out = torch.empty((qkv.shape[0], width), dtype=qkv.dtype, device=qkv.device)
        ops.conv1d_silu(qkv, 0, width, self.conv_weight, None, tail, step.lane_of_token, step.cu_seqlens, step.slot_ids,
                        out, activation=False)
        if taps > 1:
            ops.conv_state_update(qkv, 0, width, taps, tail, step.cu_seqlens, step.slot_ids)
        return out

    def attend_prepared(self, qkv: torch.Tensor, step, cache, out: torch.Tensor) -> None:
        spec = self.spec
        geometry = (spec.num_heads, spec.num_kv_heads, spec.head_dim)
        sigmoid = spec.weighting == "sigmoid"
        tiles = {}
        if step.max_query_len > 1 and 0 < getattr(step, "query_tile", 0) < (1 << 20):
            tiles = dict(query_tiles=step.query_tiles, tile_tokens=step.query_tile, cu_seqlens=step.cu_seqlens)
        plain = not sigmoid and self.head_scales is None and spec.value_width == spec.head_dim
        aligned = (qkv.stride(0) % 8 == 0 and qkv.data_ptr() % 16 == 0 and out.stride(0) % 4 == 0
                   and out.data_ptr() % 8 == 0)
        kept, sinks = self.keep_first, self.sinks
        if (step.max_query_len == 1 and aligned
                and ops.decode_attention_supported(qkv.dtype, *geometry, cache.k_cache.shape[2], spec.value_width, kept)):
            ops.decode_attention(qkv, *geometry, cache.k_cache, cache.v_cache, step.block_tables[cache.group],
                                 step.lane_of_token, step.positions, spec.scale, spec.window, step.max_seq_len, out,
                                 value_dim=spec.value_width, head_scales=self.head_scales, score_bias=self.score_bias,
                                 sigmoid=sigmoid, keep_first=kept, sinks=sinks)
        elif (plain and tiles and aligned and step.query_tile == self.query_tile
                and ops.prefill_attention_supported(qkv.dtype, *geometry, cache.k_cache.shape[2])):
            ops.prefill_attention(qkv, *geometry, cache.k_cache, cache.v_cache, step.block_tables[cache.group],
                                  step.query_tiles, step.cu_seqlens, step.start_pos, spec.scale, spec.window, out,
                                  step.max_seq_len, sinks=sinks, keep_first=kept)
        elif kept > 0 or sinks is not None:
            # the general kernel knows every form
            ops.paged_attention(qkv, *geometry, cache.k_cache, cache.v_cache, step.block_tables[cache.group],
                                step.lane_of_token, step.positions, spec.scale, spec.window, out, step.max_seq_len,
                                sinks=sinks, value_dim=spec.value_width, head_scales=self.head_scales,
                                keep_first=kept, **tiles)
        elif (tiles and aligned and step.query_tile == self.query_tile
                and ops.prefill_attention_forms_supported(qkv.dtype, *geometry, spec.value_width, cache.k_cache.shape[2],
                                                          sigmoid, self.head_scales is not None)):
            # the matrix-core kernel's further forms: sigmoid weights, or values of another width than the keys
            ops.prefill_attention_forms(qkv, *geometry, spec.value_width, cache.k_cache, cache.v_cache,
                                        step.block_tables[cache.group], step.query_tiles, step.cu_seqlens,
                                        step.start_pos, spec.scale, spec.window, out, step.max_seq_len, sigmoid=sigmoid,
                                        head_scales=self.head_scales, score_bias=self.score_bias)
        else:
            ops.paged_attention(qkv, *geometry, cache.k_cache, cache.v_cache, step.block_tables[cache.group],
                                step.lane_of_token, step.positions, spec.scale, spec.window, out, step.max_seq_len,
                                value_dim=spec.value_width, head_scales=self.head_scales, score_bias=self.score_bias,
                                sigmoid=sigmoid, **tiles)
