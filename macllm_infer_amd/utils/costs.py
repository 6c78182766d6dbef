"""What a step has to move and to compute, from the model's sizes: bytes read and written and flops, per
group of kernels.  ``bench.py`` takes its roofline figures from here and ``kernel_trace`` sets them against
the measured times of each group's kernels.

The figures are the least a step can do: every weight it uses read once, the cache and the state of the live
requests read once, what it has to write written once; activations between kernels (a few rows in a decode
step) are left out of a decode step and counted once per kernel boundary in a prompt step.
(The reference sizes the same quantities for its cache: src/architecture.rs:677-795.)
"""
from __future__ import annotations

import re
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

PEAK_HBM_BYTES = 8.0e12                                   # MI355X, published: 8 TB/s
PEAK_FLOPS = {"bf16": 2.5e15, "f32": 157.3e12}            # dense matrix cores, published


@dataclass
class Cost:
    read: float = 0.0        # bytes
    written: float = 0.0     # bytes
    flops: float = 0.0

    def __add__(self, other: "Cost") -> "Cost":
        return Cost(self.read + other.read, self.written + other.written, self.flops + other.flops)

    def times(self, factor: float) -> "Cost":
        return Cost(self.read * factor, self.written * factor, self.flops * factor)


def model_sizes(spec) -> dict:
    """Sums over the scheduled layers of a ``ModelSpec``: matrix elements by projection, K/V elements per
    token, state elements (float32) and conv tail elements (activation dtype) per request."""
    d = spec.hidden_size
    total = dict(in_weights=0, out_weights=0, gate_up=0, down=0, kv_per_token=0, state=0, conv_tail=0,
                 attention=0, scan=0, layers=len(spec.schedule), head=spec.vocab_size * d, hidden=d,
                 mixed=0, inner=0, in_width=0, windows=[], linear_scan=0, experts=[])
    for entry in spec.schedule:
        layer = spec.layers[entry.layer]
        for slot in layer.mixers:
            part = slot.spec
            if part.kind == "attention":
                q, kv = part.num_heads * part.head_dim, part.num_kv_heads * part.head_dim
                values, mixed = part.num_kv_heads * part.value_width, part.num_heads * part.value_width
                # values that are the keys as projected have no matrix of their own, but cells of their own in the cache
                projected = 0 if getattr(part, "values_from_keys", False) else values
                if getattr(part, "projection_norm_eps", None) is not None:
                    total["in_weights"] += q + kv                          # the norms' weights over whole projections
                total["in_weights"] += (q + kv + projected) * d
                total["out_weights"] += d * mixed
                total["kv_per_token"] += kv + values if entry.kv_from is None else 0
                # x 2 T^2 flops (causal: half of 4 T^2); a window w keeps min(i + 1, w) keys for the query at i
                total["attention"] += part.num_heads * (part.head_dim + part.value_width) / 2.0
                total["windows"].append((part.num_heads * (part.head_dim + part.value_width) / 2.0,
                                         (kv + values) if entry.kv_from is None else 0, part.window))
                total["mixed"] += mixed
                total["in_width"] += q + kv + projected
                if getattr(part, "conv_kernel", 0) > 1:                    # the tail of the projections' convolution
                    total["conv_tail"] += (part.conv_kernel - 1) * (q + kv + projected)
            elif part.kind == "gated_linear_attention":
                keys, values = part.num_heads * part.key_dim, part.num_heads * part.value_dim
                rank = part.decay_rank or 16
                total["in_weights"] += (2 * keys + 2 * values + rank) * d + keys * rank
                total["out_weights"] += d * values
                total["state"] += part.num_heads * part.key_dim * part.value_dim
                total["linear_scan"] += 5 * part.num_heads * part.key_dim * part.value_dim     # x T flops
                total["mixed"] += values
                total["in_width"] += 2 * keys + 2 * values + rank + 2 * keys                  # the decays in float32
            elif part.kind == "latent_attention":
                heads, rank, turned = part.num_heads, part.kv_rank, part.rope_dim
                q = heads * (part.head_dim + turned)
                # down-projections, the queries' up-projection and their way into the latent space; out of it and out
                if part.q_rank is None:                                    # the queries projected directly
                    total["in_weights"] += (q + rank + turned) * d + heads * part.head_dim * rank
                else:
                    total["in_weights"] += (part.q_rank + rank + turned) * d + q * part.q_rank + heads * part.head_dim * rank
                total["out_weights"] += heads * part.value_dim * rank + d * heads * part.value_dim
                cached = (rank + turned) if entry.kv_from is None else 0        # one latent and one turned part a token
                total["kv_per_token"] += cached
                # every head scores against the cached row and sums latents: keys rank + turned wide, values rank wide
                total["attention"] += heads * (2 * rank + turned) / 2.0
                total["windows"].append((heads * (2 * rank + turned) / 2.0, cached, part.window))
                total["mixed"] += heads * part.value_dim + heads * rank
                total["in_width"] += (part.q_rank or 0) + rank + turned + q + heads * (rank + turned)
            elif part.kind == "retention":
                keys, values = part.num_heads * part.key_dim, part.num_heads * part.value_dim
                total["in_weights"] += (2 * keys + 2 * values) * d
                total["out_weights"] += d * values
                total["state"] += part.num_heads * part.key_dim * part.value_dim
                total["linear_scan"] += 4 * part.num_heads * part.key_dim * part.value_dim     # x T flops
                total["mixed"] += values
                total["in_width"] += 2 * keys + 2 * values
            elif part.kind == "general_delta":
                inner, rank = part.num_heads * part.head_dim, part.decay_rank or 0
                total["in_weights"] += (5 * inner + rank) * d + inner * rank
                total["out_weights"] += d * inner
                total["state"] += part.num_heads * part.head_dim ** 2
                total["linear_scan"] += 10 * part.num_heads * part.head_dim ** 2               # x T flops
                total["mixed"] += inner
                total["in_width"] += 5 * inner + rank
            elif part.kind == "mamba2":
                total["in_weights"] += part.projection_width * d
                total["out_weights"] += d * part.inner_size
                total["state"] += part.num_heads * part.head_dim * part.state_size
                total["conv_tail"] += max(part.conv_kernel - 1, 0) * part.conv_width
                total["scan"] += part.num_heads * part.head_dim * part.state_size      # x 6 T flops
                total["mixed"] += part.inner_size
                total["in_width"] += part.projection_width
        if entry.before is not None and getattr(entry.before, "mix_name", None) is not None:
            total["in_weights"] += 2 * d * d                               # the stream mixed with the embedding output
        if layer.ffn is None:
            continue
        if layer.ffn.kind == "swiglu":
            total["gate_up"] += 2 * layer.ffn.intermediate_size * d
            total["down"] += d * layer.ffn.intermediate_size
            total["inner"] += layer.ffn.intermediate_size
        elif layer.ffn.kind == "routed_experts":
            ffn = layer.ffn
            shared = ffn.shared_size or 0
            # what every token uses whatever it chooses: the router, the shared expert and its gate
            total["gate_up"] += (ffn.num_experts + (1 if shared else 0)) * d + 2 * shared * d
            total["down"] += d * shared
            total["inner"] += shared + ffn.top_k * ffn.expert_size
            first = (2 if getattr(ffn.activation, "gated", True) else 1) * ffn.expert_size * d      # gate and up, or up alone
            total["experts"].append((ffn.num_experts, ffn.top_k, first, d * ffn.expert_size))
        elif layer.ffn.kind == "polynorm_ffn":
            total["gate_up"] += layer.ffn.intermediate_size * d
            total["down"] += d * layer.ffn.intermediate_size
            total["inner"] += layer.ffn.intermediate_size
    return total


def keys_seen(tokens: float, window) -> float:
    """Sum over the queries 0 .. tokens-1 of one prompt of the keys each sees: min(i + 1, window)."""
    if not window or window >= tokens:
        return tokens * (tokens + 1) / 2.0
    return window * (window + 1) / 2.0 + (tokens - window) * window


def experts_touched(experts: int, top_k: int, rows: float) -> float:
    """How many of ``experts`` a step of ``rows`` tokens reads when every token picks ``top_k`` at random."""
    return experts * (1.0 - (1.0 - top_k / experts) ** rows)


def decode_step_costs(spec, batch: int, context: float, element: int = 2) -> Dict[str, Cost]:
    """A step of ``batch`` single tokens whose requests hold ``context`` tokens each.  Routed experts: the matrices
    of as many experts as the step's tokens reach when they choose at random."""
    s = model_sizes(spec)
    rows = batch
    for experts, top_k, gate_up, down in s["experts"]:
        touched = experts_touched(experts, top_k, rows)
        s["gate_up"] += touched * gate_up * 1.0
        s["down"] += touched * down * 1.0
    routed_flops = sum(2.0 * rows * top_k * (gate_up + down) - 2.0 * rows * experts_touched(experts, top_k, rows) * (gate_up + down)
                       for experts, top_k, gate_up, down in s["experts"])
    kept = lambda window: min(context, window) if window else context          # keys a query still sees
    kv_read = sum(per_token * kept(window) for _, per_token, window in s["windows"])
    attention_flops = sum(4.0 * width * kept(window) for width, _, window in s["windows"])
    return {
        "input projections": Cost(s["in_weights"] * element, 0, 2.0 * rows * s["in_weights"]),
        "mixers": Cost(batch * (kv_read * element + s["state"] * 4 + s["conv_tail"] * element),
                       batch * (s["kv_per_token"] * element + s["state"] * 4 + s["conv_tail"] * element),
                       batch * (attention_flops + 6.0 * s["scan"] + s["linear_scan"])),
        "output projections": Cost(s["out_weights"] * element, 0, 2.0 * rows * s["out_weights"]),
        # (the flops of routed experts: every row times the experts it chose, not times the experts the step read)
        "gate and up projections": Cost(s["gate_up"] * element, 0, 2.0 * rows * s["gate_up"] + routed_flops),
        "down projections": Cost(s["down"] * element, 0, 2.0 * rows * s["down"]),
        "output head": Cost(s["head"] * element, batch * spec.vocab_size * 4, 2.0 * rows * s["head"]),
    }


def prefill_costs(spec, tokens: int, element: int = 2) -> Dict[str, Cost]:
    """One prompt of ``tokens`` tokens in one step (its last position's logits wanted)."""
    s = model_sizes(spec)
    T = tokens
    weights = s["in_weights"] + s["out_weights"] + s["gate_up"] + s["down"]
    # routed experts: every matrix is read (a long prompt reaches all of them), a token computes with top_k of them
    routed_read = sum(experts * (gate_up + down) for experts, _, gate_up, down in s["experts"])
    routed_flops = sum(2.0 * T * top_k * (gate_up + down) for _, top_k, gate_up, down in s["experts"])
    rows_moved = T * element * (s["hidden"] * 4 * s["layers"] + s["in_width"] + s["mixed"] + 3 * s["inner"])
    return {
        "matrix products": Cost((weights + routed_read) * element + rows_moved, 0,
                                2.0 * T * weights + routed_flops + 2.0 * s["head"]),
        "attention": Cost(T * s["kv_per_token"] * element, T * s["kv_per_token"] * element,
                          sum(4.0 * width * keys_seen(T, window) for width, _, window in s["windows"])),
        "state-space scan": Cost(s["state"] * 4, s["state"] * 4, 6.0 * s["scan"] * T + s["linear_scan"] * T),
    }


def total(costs: Dict[str, Cost]) -> Cost:
    out = Cost()
    for cost in costs.values():
        out = out + cost
    return out


# Which kernels do the work of which group (name patterns of this package's kernels and of the BLAS library's).
# fused_gemm_kernel<row tiles, prologue (0 norm, 1 plain, 2 merge of the attention runs), epilogue (0 plain,
# 1 SiLU(g)*u, 2 conv, 3 add to the residual stream), ...>; shared_rows_gemm_kernel<row tiles, feature tiles a
# wave, epilogue (0 float32 slabs, 1 SiLU(g)*u, 2 conv or plain rows)>.  A product with the plain epilogue that is
# launched once a step is the output head; launched more often, an output or down projection (the library's
# products carry no such mark and stay with the other kernels).
DECODE_GROUPS: List[Tuple[str, str]] = [
    (r"mixer_decode_kernel|mixer_merge_kernel|decode_attention_kernel|decode_merge_kernel|ssm_scan_kernel|conv_step_kernel|"
     r"gate_norm_kernel|rope_kv_store_kernel|paged_attention_kernel|paged_attention_tile_kernel|"
     r"paged_attention_merge_kernel|linear_state_|head_norm_gate_kernel|tanh_rows_kernel|latent_|rotate_heads_kernel|attention_prepare_kernel", "mixers"),
    (r"fused_gemm_kernel<\d+, \d+, 2|shared_rows_gemm_kernel<\d+, \d+, 2", "input projections"),
    (r"fused_gemm_kernel<\d+, \d+, 1|shared_rows_gemm_kernel<\d+, \d+, 1|moe_|clamped_glu_kernel", "gate and up projections"),
    (r"fused_gemm_kernel<\d+, \d+, 3|fused_gemm_kernel<\d+, 2, 0|shared_rows_gemm_kernel<\d+, \d+, 0|fused_gemm_split_kernel",
     "output projections + down projections"),
]
PLAIN_PRODUCT = r"fused_gemm_kernel<\d+, [01], 0"
PREFILL_GROUPS: List[Tuple[str, str]] = [
    (r"^Cijk_|gemm_f32_kernel|head_gemm_kernel|moe_expert_gemm", "matrix products"),
    (r"prefill_attention|paged_attention_kernel|paged_attention_tile_kernel|paged_attention_merge_kernel|"
     r"rope_kv_store_kernel|latent_|attention_prepare_kernel|rotate_heads_kernel", "attention"),
    (r"ssd_|ssm_scan_kernel|conv1d_silu|conv_state_update|gate_norm_kernel|linear_state_|head_norm_gate_kernel|"
     r"tanh_rows_kernel", "state-space scan"),
]


def group_of(kernel: str, groups: List[Tuple[str, str]], calls: int = 2) -> Optional[str]:
    """The group of a kernel by its name and, for the products that carry no other mark, by how often a step
    launches it (``calls``)."""
    for pattern, name in groups:
        if re.search(pattern, kernel):
            return name
    if groups is DECODE_GROUPS and re.search(PLAIN_PRODUCT, kernel):
        return "output head" if calls == 1 else "output projections + down projections"
    return None


def merged(costs: Dict[str, Cost], name: str) -> Cost:
    """The cost of a group whose name joins several of ``costs`` with " + "."""
    out = Cost()
    for piece in name.split(" + "):
        out = out + costs.get(piece, Cost())
    return out
