"""Attention whose keys and values are kept as one low-rank latent per token."""
from __future__ import annotations

import torch

from ..cache.manager import KVNeed
from ..kernels import ops
from ..kernels.limits import ATTENTION_MAX_HEAD_DIM, GRID_MOST, beyond
from ..weights.loader import Expect
from .base import BuildContext, Mixer, part_class, register_part
from .linear import Linear


@register_part("latent_attention")
class LatentAttention(Mixer):
    """Queries through a latent (c_q = RMSNorm(W_dq x), q = W_uq c_q: per head ``head_dim`` plain and ``rope_dim``
    turned dimensions) or, without a ``q_rank``, projected directly (q = W_q x); keys and values through another (W_dkv x = [c before its RMSNorm | one turned key part for
    all heads]; a head's plain key is W_uk c, its value W_uv c).

    The cache holds, per token, c and the turned key part: one "key" of ``kv_rank + rope_dim`` numbers shared by
    all heads, whose first ``kv_rank`` numbers are also the "value".  The up-projections never touch the cache:
    q_plain . (W_uk c) = (W_uk^T q_plain) . c, so each head's query is taken into the latent space (a product per
    head with W_uk^T) and scored against the cached rows as they are, and sum_j p_j (W_uv c_j) = W_uv (sum_j p_j c_j),
    so the attended latent of a head is taken up by W_uv afterwards.  To the attention kernels this is attention with
    one key/value head, keys ``kv_rank + rope_dim`` wide and values ``kv_rank`` wide.

    One kernel forms both latents' RMS norms (float32), turns the shared key part and writes the token's cache
    cell; one turns the queries' ``rope_dim`` parts beside their latent-space parts."""
    graph_safe = True
    kernel_modules = ("common", "attention", "gemm", "latent")
    query_tile = 64          # tokens of one lane that a workgroup of the prompt attention kernels takes

    @classmethod
    def expected_tensors(cls, spec, prefix: str, hidden_size: int):
        heads = spec.num_heads
        if spec.q_rank is None:
            queries = [Expect(f"{prefix}.q.weight", ((heads * (spec.head_dim + spec.rope_dim), hidden_size),))]
        else:
            queries = [Expect(f"{prefix}.dq.weight", ((spec.q_rank, hidden_size),)),
                       Expect(f"{prefix}.dq.norm.weight", ((spec.q_rank,),), init="norm"),
                       Expect(f"{prefix}.uq.weight", ((heads * (spec.head_dim + spec.rope_dim), spec.q_rank),))]
        return queries + [
                Expect(f"{prefix}.dkv.weight", ((spec.kv_rank + spec.rope_dim, hidden_size),)),
                Expect(f"{prefix}.dkv.norm.weight", ((spec.kv_rank,),), init="norm"),
                Expect(f"{prefix}.uk.weight", ((heads * spec.head_dim, spec.kv_rank),)),
                Expect(f"{prefix}.uv.weight", ((heads * spec.value_dim, spec.kv_rank),)),
                Expect(f"{prefix}.o.weight", ((hidden_size, heads * spec.value_dim),))]

    @classmethod
    def limits(cls, spec, hidden_size: int):
        return (beyond("latent_attention", "cached_key_dim", spec.cached_key_dim, ATTENTION_MAX_HEAD_DIM,
                       "a query row in the latent space and its sums are kept in LDS and registers")
                + beyond("latent_attention", "num_heads", spec.num_heads, GRID_MOST, "heads index a dimension of the launch"))

    @classmethod
    def cache_needs(cls, spec):
        return [KVNeed(1, spec.cached_key_dim, spec.window, spec.kv_rank)]

    def __init__(self, spec, prefix: str, tensors, build: BuildContext):
        self.spec = spec
        self.build = build
        get = lambda name: tensors[f"{prefix}.{name}"]
        heads, dim, rope, rank = spec.num_heads, spec.head_dim, spec.rope_dim, spec.kv_rank
        # both down-projections read the same rows: one product, [query latent | key/value latent | turned key part];
        # without a query latent the queries themselves stand in its place
        self.direct = spec.q_rank is None
        self.q_width = heads * (dim + rope)
        if self.direct:
            self.down = Linear([get("q.weight"), get("dkv.weight")], [None, None], build)
            self.up_q = self.q_norm = None
        else:
            self.down = Linear([get("dq.weight"), get("dkv.weight")], [None, None], build)
            self.up_q = Linear([get("uq.weight")], [None], build)
            self.q_norm = get("dq.norm.weight").to(torch.float32).contiguous().to(build.device)
        self.out = Linear([get("o.weight")], [None], build)
        self.kv_norm = get("dkv.norm.weight").to(torch.float32).contiguous().to(build.device)
        # per head: W_uk^T [kv_rank, head_dim] takes a plain query into the latent space; W_uv [value_dim, kv_rank]
        # takes an attended latent up.  Both are what the product of a head contracts over its rows with.
        keep = torch.float32 if (build.dtype == torch.float32 or dim % 8 or rank % 8) else torch.bfloat16
        self.into_latent = (get("uk.weight").reshape(heads, dim, rank).transpose(1, 2)
                            .to(keep).contiguous().to(build.device))
        self.out_of_latent = get("uv.weight").reshape(heads, spec.value_dim, rank).to(keep).contiguous().to(build.device)
        if rope:
            self.position = part_class(spec.position)(spec.position, rope, build)
            rotation = self.position.pair_rotation()
            if rotation is None:
                raise ValueError("latent attention turns its rope_dim part by position: the encoding must be a rotation")
            self.inv_freq, self.rotary_dim, self.interleaved = rotation
        else:
            self.inv_freq, self.rotary_dim, self.interleaved = None, 0, False

    def forward(self, x: torch.Tensor, step, cache) -> torch.Tensor:
        spec = self.spec
        heads, dim, rope, rank = spec.num_heads, spec.head_dim, spec.rope_dim, spec.kv_rank
        tokens = x.shape[0]
        down = self.down(x)
        owns = cache.owns_kv
        cells = (step.slot_mappings[cache.group] if owns else None, cache.k_cache if owns else None,
                 cache.v_cache if owns else None)
        if self.direct:
            ops.latent_prepare(down[:, self.q_width:], 0, rank, rope, None, self.kv_norm, spec.norm_eps, step.positions,
                               self.inv_freq, self.rotary_dim, self.interleaved, *cells, None)
            q = down[:, :self.q_width]                                # [T, heads * (dim + rope)], a view
        else:
            query_latent = torch.empty((tokens, spec.q_rank), dtype=x.dtype, device=x.device)
            ops.latent_prepare(down, spec.q_rank, rank, rope, self.q_norm, self.kv_norm, spec.norm_eps, step.positions,
                               self.inv_freq, self.rotary_dim, self.interleaved, *cells, query_latent)
            q = self.up_q(query_latent)                               # [T, heads * (dim + rope)]
        width = rank + rope
        latent_q = torch.empty((tokens, heads * width), dtype=x.dtype, device=x.device)
        ops.head_linear(q, 0, dim + rope, self.into_latent, latent_q, 0, width)
        if rope:
            ops.rotate_heads(q, dim, dim + rope, heads, rope, step.positions, self.inv_freq, self.rotary_dim,
                             self.interleaved, latent_q, rank, width)
        attended = torch.empty((tokens, heads * rank), dtype=x.dtype, device=x.device)
        tiles = {}
        if step.max_query_len > 1 and 0 < getattr(step, "query_tile", 0) < (1 << 20):
            tiles = dict(query_tiles=step.query_tiles, tile_tokens=step.query_tile, cu_seqlens=step.cu_seqlens)
        fast = ops.latent_attention_supported(x.dtype, heads, rank, rope, cache.k_cache.shape[2])
        if fast and step.max_query_len == 1:
            # single decoded tokens: the context split over many waves, the heads as the products' columns
            ops.latent_decode_attention(latent_q, heads, rank, rope, cache.k_cache, cache.v_cache,
                                        step.block_tables[cache.group], step.lane_of_token, step.positions, spec.scale,
                                        spec.window, step.max_seq_len, attended)
        elif fast and tiles and step.query_tile == self.query_tile:
            ops.latent_attention(latent_q, heads, rank, rope, cache.k_cache, cache.v_cache,
                                 step.block_tables[cache.group], step.query_tiles, step.cu_seqlens, step.start_pos,
                                 spec.scale, spec.window, attended)
        else:
            ops.paged_attention(latent_q, heads, 1, width, cache.k_cache, cache.v_cache, step.block_tables[cache.group],
                                step.lane_of_token, step.positions, spec.scale, spec.window, attended,
                                step.max_seq_len, value_dim=rank, **tiles)
        values = torch.empty((tokens, heads * spec.value_dim), dtype=x.dtype, device=x.device)
        ops.head_linear(attended, 0, rank, self.out_of_latent, values, 0, spec.value_dim)
        return self.out(values)
