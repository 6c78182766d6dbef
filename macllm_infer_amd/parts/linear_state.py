"""Mixers that carry a matrix-valued state per head from token to token instead of a cache of keys:
retention (a fixed decay per head) and the generalized delta rule (a decay per key channel and a removal of
what the state holds along the unit key).  Both keep their state [heads, value dim, key dim] in float32 in the
request's state slot and run through one scan kernel (``ops.linear_state_scan``), for prompt portions and for
single decoded tokens alike; rotation, decays, gates of the recurrence and unit keys are formed in float32 inside
it.  The head-wise root-mean-square norm, its weight and the output gate are one more launch.
"""
from __future__ import annotations

import torch

from ..cache.manager import StateNeed
from ..kernels import ops
from ..kernels.limits import GRID_MOST, LINEAR_STATE_MAX_KEY_DIM, beyond
from ..weights.loader import Expect
from .base import BuildContext, Mixer, part_class, register_part
from .linear import Linear


CHUNK_TOKENS = 128      # lanes longer than this scan in chunks of this many tokens, side by side


def scan_chunks(step):
    """The step's lanes cut into chunks when one of them is long enough for the scan in passes to pay, else None
    (the scan then walks every lane from end to end, which is what steps of single tokens and short portions want)."""
    if step.max_query_len <= CHUNK_TOKENS:
        return None
    table = step.chunk_tables.get(CHUNK_TOKENS)
    if table is not None:
        return table
    key = ("linear_state_chunks", CHUNK_TOKENS)              # a step that was packed without the table
    if key not in step.derived:
        step.derived[key] = ops.SsdChunks(step.lane_lengths, CHUNK_TOKENS, step.token_ids.device)
    return step.derived[key]


@register_part("retention")
class Retention(Mixer):
    """[q | k | v | g] = one projection of the normed rows; q and k rotated by position, k scaled;
    S <- decay[h] S + k v^T, o = S^T q per head; o / rms(o) per head, times SiLU(g), output projection."""
    graph_safe = True
    kernel_modules = ("common", "linear_state", "gemm")
    chunk_tokens = CHUNK_TOKENS

    @classmethod
    def expected_tensors(cls, spec, prefix: str, hidden_size: int):
        keys, values = spec.num_heads * spec.key_dim, spec.num_heads * spec.value_dim
        return [Expect(f"{prefix}.q.weight", ((keys, hidden_size),)),
                Expect(f"{prefix}.k.weight", ((keys, hidden_size),)),
                Expect(f"{prefix}.v.weight", ((values, hidden_size),)),
                Expect(f"{prefix}.g.weight", ((values, hidden_size),)),
                Expect(f"{prefix}.o.weight", ((hidden_size, values),))]

    @classmethod
    def limits(cls, spec, hidden_size: int):
        return (beyond("retention", "key_dim", spec.key_dim, LINEAR_STATE_MAX_KEY_DIM,
                       "a column of a head's state is spread over at most one wave")
                + beyond("retention", "num_heads", spec.num_heads, GRID_MOST, "heads index a dimension of the launch")
                + part_class(spec.position).limits(spec.position, spec.key_dim))

    @classmethod
    def cache_needs(cls, spec):
        return [StateNeed("state", (spec.num_heads, spec.value_dim, spec.key_dim), "float32")]

    def __init__(self, spec, prefix: str, tensors, build: BuildContext):
        self.spec = spec
        get = lambda name: tensors.get(f"{prefix}.{name}")
        self.in_proj = Linear([get("q.weight"), get("k.weight"), get("v.weight"), get("g.weight")],
                              [None, None, None, None], build)
        self.out_proj = Linear([get("o.weight")], [None], build)
        self.decay = torch.tensor(spec.decay, dtype=torch.float64).to(torch.float32).to(build.device)
        position = part_class(spec.position)(spec.position, spec.key_dim, build)
        rotation = position.fused_rotation()
        if rotation is None:
            raise ValueError(f"retention turns q and k inside its scan: the position encoding {spec.position.kind!r} "
                             "is no rotation by position")
        self.inv_freq, self.rotary_dim = rotation

    def forward(self, x: torch.Tensor, step, cache) -> torch.Tensor:
        spec = self.spec
        keys, values = spec.num_heads * spec.key_dim, spec.num_heads * spec.value_dim
        u = self.in_proj(x)                                              # [T, q | k | v | g]
        raw = torch.empty((x.shape[0], values), dtype=torch.float32, device=x.device)
        ops.linear_state_scan(u, q_col=0, k_col=keys, v_col=2 * keys, num_heads=spec.num_heads, key_dim=spec.key_dim,
                              value_dim=spec.value_dim, state=cache.states["state"], cu_seqlens=step.cu_seqlens,
                              slot_ids=step.slot_ids, out=raw, max_query_len=step.max_query_len,
                              head_decay=self.decay, key_scale=spec.key_scale, positions=step.positions,
                              inv_freq=self.inv_freq, rotary_dim=self.rotary_dim, chunks=scan_chunks(step))
        gated = torch.empty((x.shape[0], values), dtype=u.dtype, device=x.device)
        ops.head_norm_gate(raw, u[:, 2 * keys + values:], None, spec.num_heads, spec.norm_eps, "silu", gated)
        return self.out_proj(gated)


@register_part("general_delta")
class GeneralDelta(Mixer):
    """[r | k | v | g | a | w1] = one projection of the normed rows (a with its bias);
    decay logits = w2 tanh(w1 part) in float32; inside the scan w = exp(-floor * sigmoid(logits + w0)),
    a = sigmoid(a part), u = k / sqrt(sum k^2 + key_eps), S <- diag(w) S - (a u)(u^T S) + k v^T, o = S^T r;
    then o / rms(o) per head times the weight ``norm``, times sigmoid(g), output projection."""
    graph_safe = True
    kernel_modules = ("common", "linear_state", "gemm")
    chunk_tokens = CHUNK_TOKENS

    @classmethod
    def expected_tensors(cls, spec, prefix: str, hidden_size: int):
        inner = spec.num_heads * spec.head_dim
        rank = -1 if spec.decay_rank is None else spec.decay_rank
        return [Expect(f"{prefix}.r.weight", ((inner, hidden_size),)),
                Expect(f"{prefix}.k.weight", ((inner, hidden_size),)),
                Expect(f"{prefix}.v.weight", ((inner, hidden_size),)),
                Expect(f"{prefix}.g.weight", ((inner, hidden_size),)),
                Expect(f"{prefix}.a.weight", ((inner, hidden_size),)),
                Expect(f"{prefix}.a.bias", ((inner,),), init="bias"),
                Expect(f"{prefix}.w1.weight", ((rank, hidden_size),)),
                Expect(f"{prefix}.w2.weight", ((inner, rank),)),
                Expect(f"{prefix}.w0", ((inner,),), init="logit"),
                Expect(f"{prefix}.norm.weight", ((inner,),), init="norm"),
                Expect(f"{prefix}.o.weight", ((hidden_size, inner),))]

    @classmethod
    def limits(cls, spec, hidden_size: int):
        return (beyond("general_delta", "head_dim", spec.head_dim, LINEAR_STATE_MAX_KEY_DIM,
                       "a column of a head's state is spread over at most one wave")
                + beyond("general_delta", "num_heads", spec.num_heads, GRID_MOST, "heads index a dimension of the launch"))

    @classmethod
    def cache_needs(cls, spec):
        return [StateNeed("state", (spec.num_heads, spec.head_dim, spec.head_dim), "float32")]

    def __init__(self, spec, prefix: str, tensors, build: BuildContext):
        self.spec = spec
        get = lambda name: tensors.get(f"{prefix}.{name}")
        if get("w1.weight").shape[0] != get("w2.weight").shape[1]:
            raise ValueError(f"{prefix}: the decay's two projections do not fit each other: "
                             f"{tuple(get('w1.weight').shape)} and {tuple(get('w2.weight').shape)}")
        self.rank = get("w1.weight").shape[0]
        self.in_proj = Linear([get("r.weight"), get("k.weight"), get("v.weight"), get("g.weight"), get("a.weight"),
                               get("w1.weight")], [None, None, None, None, get("a.bias"), None], build)
        self.decay_proj = Linear([get("w2.weight")], [None], build)
        self.out_proj = Linear([get("o.weight")], [None], build)
        f32 = lambda tensor: tensor.to(torch.float32).contiguous().to(build.device)
        self.decay_bias = f32(get("w0"))
        self.norm_weight = f32(get("norm.weight"))

    def forward(self, x: torch.Tensor, step, cache) -> torch.Tensor:
        spec = self.spec
        inner = spec.num_heads * spec.head_dim
        u = self.in_proj(x)                                              # [T, r | k | v | g | a | w1]
        bent = torch.empty((x.shape[0], self.rank), dtype=u.dtype, device=x.device)
        ops.tanh_rows(u[:, 5 * inner:], bent)
        logits = ops.linear(bent, self.decay_proj.weight, None, keep_float32=True)     # float32 [T, inner]
        raw = torch.empty((x.shape[0], inner), dtype=torch.float32, device=x.device)
        ops.linear_state_scan(u, q_col=0, k_col=inner, v_col=2 * inner, num_heads=spec.num_heads,
                              key_dim=spec.head_dim, value_dim=spec.head_dim, state=cache.states["state"],
                              cu_seqlens=step.cu_seqlens, slot_ids=step.slot_ids, out=raw,
                              max_query_len=step.max_query_len, removal_col=4 * inner, decay_logits=logits,
                              decay_bias=self.decay_bias, decay_floor=spec.decay_floor, key_eps=spec.key_eps,
                              chunks=scan_chunks(step))
        gated = torch.empty((x.shape[0], inner), dtype=u.dtype, device=x.device)
        ops.head_norm_gate(raw, u[:, 3 * inner:4 * inner], self.norm_weight, spec.num_heads, spec.norm_eps, "sigmoid",
                           gated)
        return self.out_proj(gated)


@register_part("gated_linear_attention")
class GatedLinearAttention(Mixer):
    """[q | k | v | g | a1] = one projection of the normed rows; decay logits z = a2 (a1 part) in float32; inside the
    scan q is multiplied by ``query_scale`` and alpha = sigmoid(z + bias)^(1 / temperature) = exp(log sigmoid / temperature)
    decays every key channel of the state on its own, S <- diag(alpha) S + k v^T, o = S^T q; then o / rms(o) per head
    times a weight of value_dim numbers that the heads share, times SiLU(g), output projection."""
    graph_safe = True
    kernel_modules = ("common", "linear_state", "gemm")
    chunk_tokens = CHUNK_TOKENS

    @classmethod
    def expected_tensors(cls, spec, prefix: str, hidden_size: int):
        keys, values = spec.num_heads * spec.key_dim, spec.num_heads * spec.value_dim
        rank = -1 if spec.decay_rank is None else spec.decay_rank
        return [Expect(f"{prefix}.q.weight", ((keys, hidden_size),)),
                Expect(f"{prefix}.k.weight", ((keys, hidden_size),)),
                Expect(f"{prefix}.v.weight", ((values, hidden_size),)),
                Expect(f"{prefix}.g.weight", ((values, hidden_size),)),
                Expect(f"{prefix}.a1.weight", ((rank, hidden_size),)),
                Expect(f"{prefix}.a2.weight", ((keys, rank),)),
                Expect(f"{prefix}.a2.bias", ((keys,),), init="logit"),
                Expect(f"{prefix}.norm.weight", ((spec.value_dim,),), init="norm"),
                Expect(f"{prefix}.o.weight", ((hidden_size, values),))]

    @classmethod
    def limits(cls, spec, hidden_size: int):
        return (beyond("gated_linear_attention", "key_dim", spec.key_dim, LINEAR_STATE_MAX_KEY_DIM,
                       "a column of a head's state is spread over at most one wave")
                + beyond("gated_linear_attention", "num_heads", spec.num_heads, GRID_MOST,
                         "heads index a dimension of the launch"))

    @classmethod
    def cache_needs(cls, spec):
        return [StateNeed("state", (spec.num_heads, spec.value_dim, spec.key_dim), "float32")]

    def __init__(self, spec, prefix: str, tensors, build: BuildContext):
        self.spec = spec
        get = lambda name: tensors.get(f"{prefix}.{name}")
        if get("a1.weight").shape[0] != get("a2.weight").shape[1]:
            raise ValueError(f"{prefix}: the decay's two projections do not fit each other: "
                             f"{tuple(get('a1.weight').shape)} and {tuple(get('a2.weight').shape)}")
        self.rank = get("a1.weight").shape[0]
        self.in_proj = Linear([get("q.weight"), get("k.weight"), get("v.weight"), get("g.weight"), get("a1.weight")],
                              [None, None, None, None, None], build)
        self.decay_proj = Linear([get("a2.weight")], [None], build)
        self.out_proj = Linear([get("o.weight")], [None], build)
        f32 = lambda tensor: tensor.to(torch.float32).contiguous().to(build.device)
        self.decay_bias = f32(get("a2.bias"))
        self.norm_weight = f32(get("norm.weight")).repeat(spec.num_heads).contiguous()      # one copy a head

    def forward(self, x: torch.Tensor, step, cache) -> torch.Tensor:
        spec = self.spec
        keys, values = spec.num_heads * spec.key_dim, spec.num_heads * spec.value_dim
        u = self.in_proj(x)                                              # [T, q | k | v | g | a1]
        inner = u[:, 2 * keys + 2 * values:]
        if inner.stride(0) % 8 != 0 or inner.data_ptr() % 16 != 0:      # the product wants whole 16-byte pieces
            inner = inner.contiguous()
        logits = ops.linear(inner, self.decay_proj.weight, None, keep_float32=True)      # float32 [T, H * dk]
        raw = torch.empty((x.shape[0], values), dtype=torch.float32, device=x.device)
        ops.linear_state_scan(u, q_col=0, k_col=keys, v_col=2 * keys, num_heads=spec.num_heads, key_dim=spec.key_dim,
                              value_dim=spec.value_dim, state=cache.states["state"], cu_seqlens=step.cu_seqlens,
                              slot_ids=step.slot_ids, out=raw, max_query_len=step.max_query_len,
                              decay_logits=logits, decay_bias=self.decay_bias, gate_power=1.0 / spec.decay_temperature,
                              query_scale=spec.query_scale, chunks=scan_chunks(step))
        gated = torch.empty((x.shape[0], values), dtype=u.dtype, device=x.device)
        ops.head_norm_gate(raw, u[:, 2 * keys + values:2 * keys + 2 * values], self.norm_weight, spec.num_heads,
                           spec.norm_eps, "silu", gated)
        return self.out_proj(gated)
