"""Pemarax on the GPU: the kernels it added against their plain PyTorch references, every mechanism alone against the
plain implementation (tests/pemarax_plain.py), and whole models through the step function, the scheduler and the
entry points: whole prompts, portions down to two tokens, token-by-token decoding, unequal batches, pages and slots
that are used again, keys far away and just inside and outside every window, the kept first tokens, long decoding
in a small pool, and sizes of many kinds."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import pemarax_configs
import pemarax_plain
import ref_ops
from part_harness import DEV, PartHarness

pytestmark = pytest.mark.gpu

F32_GATE = 2e-4
DTYPES = [torch.float32, torch.bfloat16]
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def close(got, want, dtype, what="", loose=1.0):
    scale = max(1.0, float(want.abs().max()))
    gate = (F32_GATE if dtype == torch.float32 else 4e-2) * scale * loose
    error = (got.double().cpu() - want.double().cpu()).abs()
    assert float(error.max()) <= gate, f"{what}: max error {float(error.max()):.3e}, gate {gate:.3e}"


def ops():
    from macllm_infer_amd.kernels import build, ops as module
    build.ensure_modules(["common", "gemm", "latent", "moe", "attention", "mamba2"])
    return module


def i32(values):
    return torch.tensor(values, dtype=torch.int32)


def rounded(tensors, dtype):
    return {name: value.to(dtype).to(torch.float32) for name, value in tensors.items()}


# ------------------------------------------------------------------ kernels against their references
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("Hq, Hkv, dh, dv, rotary, interleaved, magnitude, head_norm, weighted", [
    (4, 2, 16, 8, 16, True, 1.25, "after_rotation", False), (3, 1, 12, 20, 6, True, 1.0, "after_rotation", True),
    (2, 2, 8, 8, 0, False, 1.0, "before_rotation", True), (5, 5, 64, 32, 32, False, 0.9, "before_rotation", False),
    (4, 1, 128, 128, 128, True, 1.1386, "after_rotation", False), (2, 1, 24, 24, 8, False, 1.0, None, False)])
def test_a_row_is_made_ready_with_head_norms_and_neighbouring_pairs(dtype, Hq, Hkv, dh, dv, rotary, interleaved,
                                                                    magnitude, head_norm, weighted):
    T, page, pages = 21, 4, 9
    width = (Hq + Hkv) * dh + Hkv * dv
    qkv = rand(T, width + 3, seed=1).to(dtype)
    positions = i32([3 + 2 * t for t in range(T)])
    inv_freq = (torch.rand(rotary // 2, generator=torch.Generator().manual_seed(2)) + 0.01) if rotary else None
    q_weight = (rand(dh, seed=3) * 0.2 + 1.0) if weighted else None
    k_weight = (rand(dh, seed=4) * 0.2 + 1.0) if weighted else None
    cells = torch.randperm(page * pages, generator=torch.Generator().manual_seed(5))[:T].to(torch.int32)
    want_qkv = qkv.clone()
    want_k = torch.zeros((pages, Hkv, page, dh), dtype=dtype)
    want_v = torch.zeros((pages, Hkv, dv, page), dtype=dtype)
    more = dict(interleaved=interleaved, turn_scale=magnitude, head_norm=head_norm, q_head_weight=q_weight,
                k_head_weight=k_weight, head_eps=1e-5 if head_norm else 0.0)
    ref_ops.attention_prepare(want_qkv, Hq, Hkv, dh, dv, positions, inv_freq, rotary, cells, want_k, want_v, **more)
    storage = torch.zeros((pages, Hkv * page * (dh + dv)), dtype=dtype, device=DEV)
    got_k = storage[:, :Hkv * page * dh].unflatten(-1, (Hkv, page, dh))
    got_v = storage[:, Hkv * page * dh:].unflatten(-1, (Hkv, dv, page))
    got_qkv = qkv.clone().to(DEV)
    on = lambda tensor: None if tensor is None else tensor.to(DEV)
    ops().attention_prepare(got_qkv, Hq, Hkv, dh, dv, positions.to(DEV), on(inv_freq), rotary, cells.to(DEV), got_k, got_v,
                            interleaved=interleaved, turn_scale=magnitude, head_norm=head_norm, q_head_weight=on(q_weight),
                            k_head_weight=on(k_weight), head_eps=1e-5 if head_norm else 0.0)
    close(got_qkv[:, :Hq * dh].float(), want_qkv[:, :Hq * dh].float(), dtype, "queries")
    assert torch.equal(got_qkv[:, Hq * dh:].cpu(), qkv[:, Hq * dh:]), "only the queries are written back"
    close(got_k.float(), want_k.float(), dtype, "cached keys")
    close(got_v.float(), want_v.float(), dtype, "cached values")


def attention_case(Hq, Hkv, dh, dv, lengths, page, dtype, seed=0, sharpen=1.0):
    """Queries for the last ``new`` tokens of requests of ``lengths`` = [(context, new)], and caches that hold every
    key and value of theirs on pages dealt out in a shuffled order; cells that hold nothing are NaN."""
    lanes = len(lengths)
    most = max(context for context, _ in lengths)
    max_pages = -(-most // page)
    total_pages = lanes * max_pages + 2
    order = torch.randperm(total_pages, generator=torch.Generator().manual_seed(seed + 1)).tolist()
    k_cache = torch.full((total_pages, Hkv, page, dh), float("nan"))
    v_cache = torch.full((total_pages, Hkv, dv, page), float("nan"))
    tables = torch.full((lanes, max_pages), -1, dtype=torch.int32)
    rows, lane_of, positions, cu, starts = [], [], [], [0], []
    for lane, (context, new) in enumerate(lengths):
        for index in range(-(-context // page)):
            tables[lane, index] = order.pop()
        keys = rand(context, Hkv, dh, seed=seed + 10 + lane) * sharpen
        values = rand(context, Hkv, dv, seed=seed + 40 + lane)
        for position in range(context):
            k_cache[tables[lane, position // page], :, position % page, :] = keys[position]
            v_cache[tables[lane, position // page], :, :, position % page] = values[position]
        rows.append(rand(new, Hq * dh, seed=seed + 70 + lane) * sharpen)
        lane_of += [lane] * new
        positions += list(range(context - new, context))
        starts.append(context - new)
        cu.append(cu[-1] + new)
    q = torch.cat(rows).to(dtype)
    return (q, k_cache.to(dtype), v_cache.to(dtype), tables, i32(lane_of), i32(positions), i32(cu), i32(starts))


def paged(k_cache, v_cache):
    """The two caches on the device as views of one storage, a page of keys and its values side by side."""
    pages, Hkv, page, dh = k_cache.shape
    dv = v_cache.shape[2]
    storage = torch.empty((pages, Hkv * page * (dh + dv)), dtype=k_cache.dtype, device=DEV)
    keys = storage[:, :Hkv * page * dh].unflatten(-1, (Hkv, page, dh))
    values = storage[:, Hkv * page * dh:].unflatten(-1, (Hkv, dv, page))
    keys.copy_(k_cache)
    values.copy_(v_cache)
    return keys, values


def query_tiles_of(cu, tile):
    rows = []
    for lane in range(len(cu) - 1):
        for first in range(int(cu[lane]), int(cu[lane + 1]), tile):
            rows.append((lane, first))
    return i32(rows)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("Hq, Hkv, dh, dv, window, kept, lengths, page", [
    (4, 2, 16, 24, 9, 3, [(70, 70), (40, 1), (300, 33)], 8),
    (2, 1, 64, 64, 40, 21, [(600, 600), (41, 41), (530, 1), (61, 2)], 16),
    (3, 3, 32, 8, 300, 5, [(700, 100), (299, 299), (301, 1)], 4),
    (8, 2, 128, 128, 17, 260, [(900, 64), (280, 280)], 16)])
def test_the_general_kernels_keep_the_first_keys_and_a_sink(dtype, Hq, Hkv, dh, dv, window, kept, lengths, page):
    """Per-token and tiled general kernels, whole prompts, portions and single tokens side by side, with the keys
    behind the window gone from their pages (NaN cells) except the kept first ones."""
    q, k_cache, v_cache, tables, lane_of, positions, cu, _ = attention_case(Hq, Hkv, dh, dv, lengths, page, dtype)
    sinks = rand(Hq, seed=9)
    want = torch.empty((q.shape[0], Hq * dv), dtype=dtype)
    clean_k, clean_v = torch.nan_to_num(k_cache.float()).to(dtype), torch.nan_to_num(v_cache.float()).to(dtype)
    ref_ops.paged_attention(q, Hq, Hkv, dh, clean_k, clean_v, tables.clamp(min=0), lane_of, positions, 0.3, window, want,
                            sinks=sinks, value_dim=dv, keep_first=kept)
    # what no query of the step sees holds NaN: a kernel that reads a cell it should not shows it
    for lane, (context, new) in enumerate(lengths):
        for position in range(kept, max(0, context - new - window + 1)):
            k_cache[tables[lane, position // page], :, position % page, :] = float("nan")
            v_cache[tables[lane, position // page], :, :, position % page] = float("nan")
    args = (q.to(DEV), Hq, Hkv, dh, *paged(k_cache, v_cache), tables.clamp(min=0).to(DEV), lane_of.to(DEV),
            positions.to(DEV), 0.3, window)
    for tiled in (False, True):
        got = torch.empty(want.shape, dtype=dtype, device=DEV)
        more = dict(query_tiles=query_tiles_of(cu, 64).to(DEV), tile_tokens=64, cu_seqlens=cu.to(DEV)) if tiled else {}
        ops().paged_attention(*args, got, max(c for c, _ in lengths), sinks=sinks.to(DEV), value_dim=dv, keep_first=kept, **more)
        close(got.float(), want.float(), dtype, f"tiled={tiled}")
    fixed = torch.empty(want.shape, dtype=dtype, device=DEV)
    ops().paged_attention(*args, fixed, max(c for c, _ in lengths), value_dim=dv, keep_first=kept, fixed_sink=0.0)
    ref_ops.paged_attention(q, Hq, Hkv, dh, clean_k, clean_v, tables.clamp(min=0), lane_of, positions, 0.3, window, want,
                            value_dim=dv, keep_first=kept, fixed_sink=0.0)
    close(fixed.float(), want.float(), dtype, "a sink of score zero")


@pytest.mark.parametrize("Hq, Hkv, dh, window, kept, lengths, page", [
    (4, 2, 64, 40, 5, [(700, 700), (41, 41), (300, 37), (45, 2)], 16),
    (6, 2, 64, 150, 6, [(577, 577), (1300, 40)], 16),
    (2, 1, 128, 33, 70, [(400, 400), (120, 100)], 8),
    (8, 2, 64, 64, 64, [(257, 257), (64, 64), (65, 65)], 32),
    (3, 1, 128, 300, 1, [(900, 130)], 16)])
def test_the_matrix_core_prompt_kernel_keeps_the_first_keys_and_a_sink(Hq, Hkv, dh, window, kept, lengths, page):
    dtype = torch.bfloat16
    q, k_cache, v_cache, tables, lane_of, positions, cu, starts = attention_case(Hq, Hkv, dh, dh, lengths, page, dtype, seed=3)
    sinks = torch.zeros(Hq)
    want = torch.empty((q.shape[0], Hq * dh), dtype=dtype)
    clean_k, clean_v = torch.nan_to_num(k_cache.float()).to(dtype), torch.nan_to_num(v_cache.float()).to(dtype)
    ref_ops.paged_attention(q, Hq, Hkv, dh, clean_k, clean_v, tables.clamp(min=0), lane_of, positions, dh ** -0.5, window, want,
                            sinks=sinks, keep_first=kept)
    got = torch.empty(want.shape, dtype=dtype, device=DEV)
    ops().prefill_attention(q.to(DEV), Hq, Hkv, dh, *paged(clean_k, clean_v), tables.clamp(min=0).to(DEV),
                            query_tiles_of(cu, 64).to(DEV), cu.to(DEV), starts.to(DEV), dh ** -0.5, window, got,
                            max(c for c, _ in lengths), sinks=sinks.to(DEV), keep_first=kept)
    close(got.float(), want.float(), dtype, "prompt portions")


@pytest.mark.parametrize("Hq, Hkv, dh, dv, window, kept, contexts, page", [
    (6, 2, 64, 64, 150, 6, [1300, 151, 157, 5, 150], 16), (8, 2, 128, 128, 40, 100, [600, 41, 99, 101, 140], 8),
    (2, 2, 64, 96, 20, 3, [18, 21, 24, 300], 16), (6, 1, 128, 32, 512, 512, [2000, 1025, 1023], 64)])
def test_the_split_context_decode_kernel_keeps_the_first_keys_and_a_sink(Hq, Hkv, dh, dv, window, kept, contexts, page):
    dtype = torch.bfloat16
    lengths = [(context, 1) for context in contexts]
    q, k_cache, v_cache, tables, lane_of, positions, cu, _ = attention_case(Hq, Hkv, dh, dv, lengths, page, dtype, seed=5)
    sinks = rand(Hq, seed=2)
    want = torch.empty((q.shape[0], Hq * dv), dtype=dtype)
    clean_k, clean_v = torch.nan_to_num(k_cache.float()).to(dtype), torch.nan_to_num(v_cache.float()).to(dtype)
    ref_ops.paged_attention(q, Hq, Hkv, dh, clean_k, clean_v, tables.clamp(min=0), lane_of, positions, dh ** -0.5, window, want,
                            sinks=sinks, value_dim=dv, keep_first=kept)
    got = torch.empty(want.shape, dtype=dtype, device=DEV)
    ops().decode_attention(q.to(DEV), Hq, Hkv, dh, *paged(clean_k, clean_v), tables.clamp(min=0).to(DEV),
                           lane_of.to(DEV), positions.to(DEV), dh ** -0.5, window, max(contexts), got, value_dim=dv,
                           keep_first=kept, sinks=sinks.to(DEV))
    close(got.float(), want.float(), dtype, "single tokens")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C, K, lengths", [(24, 3, [5, 1, 2, 9]), (7, 4, [1, 1, 1]), (64, 2, [30]), (40, 1, [3, 2])])
def test_a_convolution_without_an_activation_and_its_tail(dtype, C, K, lengths):
    T, lanes = sum(lengths), len(lengths)
    u = rand(T, C + 5, seed=1).to(dtype)
    weight = rand(C, K, seed=2)
    state = rand(lanes + 2, max(K - 1, 0), C, seed=3).to(dtype)
    slots = i32(list(range(lanes, 0, -1)))
    cu = i32([0] + list(np.cumsum(lengths)))
    lane_of = i32([lane for lane, length in enumerate(lengths) for _ in range(length)])
    want, want_state = torch.empty((T, C), dtype=dtype), state.clone()
    ref_ops.conv1d_silu(u, 2, C, weight, None, want_state, lane_of, cu, slots, want, activation=False)
    ref_ops.conv_state_update(u, 2, C, K, want_state, cu, slots)
    got, got_state = torch.empty((T, C), dtype=dtype, device=DEV), state.clone().to(DEV)
    ops().conv1d_silu(u.to(DEV), 2, C, weight.to(DEV), None, got_state, lane_of.to(DEV), cu.to(DEV), slots.to(DEV), got,
                      activation=False)
    ops().conv_state_update(u.to(DEV), 2, C, K, got_state, cu.to(DEV), slots.to(DEV))
    close(got.float(), want.float(), dtype, "the sums")
    assert torch.equal(got_state.cpu(), want_state), "the tails"
    if all(length == 1 for length in lengths):
        rows, step_state = u.clone().to(DEV), state.clone().to(DEV)
        ops().conv_step(rows, 2, C, weight.to(DEV), None, step_state, slots.to(DEV), activation=False)
        close(rows[:, 2:2 + C].float(), want.float(), dtype, "single tokens in place")
        assert torch.equal(step_state.cpu(), want_state)


@pytest.mark.parametrize("T, experts, top", [(1, 5, 2), (37, 12, 3), (300, 70, 8), (9, 4, 4), (64, 130, 1)])
def test_the_largest_biased_logits_are_chosen_and_weighted_among_themselves(T, experts, top):
    logits = rand(T, experts + 2, seed=experts)
    bias = rand(experts, seed=1) * 0.5
    want_chosen, want_weights, _ = ref_ops.moe_route(logits, experts, top, bias, 1.0, 0.0, False, routing="top_then_softmax")
    chosen, weights, gate = ops().moe_route(logits.to(DEV), experts, top, bias.to(DEV), 1.0, 0.0, False,
                                            routing="top_then_softmax")
    assert gate is None and torch.equal(chosen.cpu(), want_chosen), "the choice, in the order of the logits"
    close(weights, want_weights, torch.float32, "weights")
    assert float((weights.sum(dim=-1) - 1.0).abs().max()) < 1e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T, experts, top, hidden, inner, pad", [(5, 4, 2, 40, 24, 16), (130, 6, 3, 64, 96, 64),
                                                                 (600, 3, 2, 128, 64, 128), (3, 9, 9, 20, 12, 16)])
def test_experts_without_a_gate_square_their_relu(dtype, T, experts, top, hidden, inner, pad):
    x = rand(T, hidden, seed=1).to(dtype)
    up = (rand(experts, inner, hidden, seed=2) / hidden ** 0.5).to(dtype)
    chosen = torch.stack([torch.randperm(experts, generator=torch.Generator().manual_seed(t))[:top] for t in range(T)]).to(torch.int32)
    plan = ops().moe_plan(chosen.to(DEV), experts, pad)
    want_plan = ref_ops.MoePlan(chosen, experts, pad)
    got = torch.empty((plan.capacity, inner), dtype=dtype, device=DEV)
    ops().moe_expert_gemm(x.to(DEV), plan, up.to(DEV), got, gather=True, glu=None, squared_relu=True)
    want = torch.empty((want_plan.capacity, inner), dtype=dtype)
    ref_ops.moe_expert_gemm(x, want_plan, up, want, True, None, squared_relu=True)
    # places are dealt out in another order on the device: compare token by token and choice by choice
    got_rows = got.float().cpu()[plan.place.cpu().long()]
    want_rows = want.float()[want_plan.place.long()]
    close(got_rows, want_rows, dtype, "activated rows")
    assert float(got_rows.min()) >= 0.0


@pytest.mark.parametrize("d, T, count", [(40, 19, 2), (256, 7, 1), (1500, 3, 3), (4104, 2, 4)])
def test_branches_are_normed_each_on_its_own_before_they_are_summed(d, T, count):
    branches = []
    for index in range(count):
        rows = rand(T, d, seed=index, scale=1.0 + 3.0 * index)
        rows = rows.to(torch.bfloat16) if index % 2 else rows
        branches.append((rows, 0.5 + 0.25 * index, rand(d, seed=10 + index) * 0.1 + 1.0, 1e-5))
    want = torch.empty((T, d))
    ref_ops.normed_sum(branches, want)
    got = torch.empty((T, d), device=DEV)
    ops().normed_sum([(rows.to(DEV), factor, weight.to(DEV), eps) for rows, factor, weight, eps in branches], got)
    close(got, want, torch.float32, "the sum")


# ------------------------------------------------------------------ every mechanism alone
def feed_every_way(make_harness, x, plain_rows, dtype, beside=None, loose=1.0):
    """Whole, in portions (down to two tokens and one), token by token, and beside another request: every fed row
    against ``plain_rows``; slots and pages of finished feeds are used again by the next."""
    T = x.shape[0]
    harness = make_harness()
    out, = harness.run([("whole", x)])
    close(out, plain_rows, dtype, "whole", loose)
    harness.cache.finish("whole")
    sizes, cursor, pieces = [7, 2, 5, 3, 11, 2, 1, 13, 2, 4, 130, 2], 0, []
    turn = 0
    while cursor < T:
        count = min(sizes[turn % len(sizes)], T - cursor)
        if beside is not None and turn % 3 == 1:
            got, _ = harness.run([("cut", x[cursor:cursor + count]), ("other", beside[turn:turn + 1])])
        else:
            got, = harness.run([("cut", x[cursor:cursor + count])])
        pieces.append(got)
        cursor += count
        turn += 1
    close(torch.cat(pieces), plain_rows, dtype, "portions", loose)
    harness.cache.finish("cut")
    head = max(1, T - 40)
    pieces = [harness.run([("tail", x[:head])])[0]]
    for position in range(head, T):
        pieces.append(harness.run([("tail", x[position:position + 1])])[0])
    close(torch.cat(pieces), plain_rows, dtype, "token by token", loose)


def attention_parts(hidden, H, G, dim, vdim, window, keep, conv, rot_dims, scaling, seed, base=300.0, sharpen=1.0):
    """(spec, tensors under the part's names, the design's mixer table, tensors under the stored names)."""
    table = pemarax_configs.attention(H, G, dim, vdim, window, keep, conv, rot_dims, scaling, base)["mixer"]
    from macllm_infer_amd.config.pemarax import _attention
    spec = _attention(table, "mixer", 1e-5)[0].spec
    shapes = {"q": (H * dim, hidden), "k": (G * dim, hidden), "v": (G * vdim, hidden), "o": (hidden, H * vdim)}
    stored = {name: rand(*shape, seed=seed + i) / shape[1] ** 0.5 for i, (name, shape) in enumerate(shapes.items())}
    stored["q"], stored["k"] = stored["q"] * sharpen, stored["k"] * sharpen
    if conv:
        for i, name in enumerate(("q", "k", "v")):
            stored[f"{name}.conv"] = rand(shapes[name][0], conv, seed=seed + 20 + i) / conv ** 0.5
    tensors = {}
    for name, value in stored.items():
        head, _, rest = name.partition(".")
        tensors[f"{head}_proj.{rest}.weight" if rest else f"{head}_proj.weight"] = value
    return spec, tensors, table, stored


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, G, dim, vdim, window, keep, conv, rot_dims, scaling", [
    (4, 2, 16, 8, 11, 3, 3, 16, (4.0, 64, 8.0, 1.0)), (3, 1, 12, 20, 6, 0, 4, 8, (8.0, 32, 4.0, 0.5)),
    (2, 2, 8, 8, 5, 2, 0, 0, None), (2, 1, 24, 24, 300, 7, 2, 24, None),
    # head sizes of the matrix-core kernels (bfloat16): prompt portions, single tokens, the kept keys on pages of their own
    (4, 1, 64, 64, 40, 4, 3, 64, (4.0, 128, 16.0, 1.0)), (4, 2, 128, 128, 33, 20, 2, 32, None), (8, 2, 64, 64, 64, 1, 3, 64, None)])
def test_attention_with_convolutions_unit_norms_kept_tokens_and_a_sink_alone(dtype, H, G, dim, vdim, window, keep, conv,
                                                                             rot_dims, scaling):
    hidden, T = 56, 170
    spec, tensors, table, stored = attention_parts(hidden, H, G, dim, vdim, window, keep, conv, rot_dims, scaling, 30)
    tensors, stored = rounded(tensors, dtype), rounded(stored, dtype)
    x = rand(T, hidden, seed=2).to(dtype).float()
    want = pemarax_plain.attention_mixer(x.double(), table, {k: v.double() for k, v in stored.items()}, 1e-5).float()
    feed_every_way(lambda: PartHarness(spec, tensors, hidden, dtype, page_size=8, capacity=600), x, want, dtype,
                   beside=rand(40, hidden, seed=3))


def crafted_attention(distance, T, window, keep, matrix):
    """An attention layer (no convolution, so that a token's key is its own row's) in which the key ``distance``
    tokens behind the last query would take nearly all of the last row's weight if it is seen: queries and keys are
    unit-normed, so the score is scale * cosine * dim, and the crafted row is the last row's own (cosine one) with a
    scale that makes exp(score) dwarf the other keys.  No rotation: the cosine does not depend on the distance."""
    hidden = 32
    dim = 64 if matrix else 16
    spec, tensors, table, stored = attention_parts(hidden, 2, 1, dim, dim, window, keep, 0, 0, None, 50)
    table["scale"] = 12.0 / dim                      # the crafted key scores 12, a random one about +-12 / sqrt(dim)
    from macllm_infer_amd.config.pemarax import _attention
    spec = _attention(table, "mixer", 1e-5)[0].spec
    # the key projection is the query projection of head 0: equal rows give cosine one
    tensors["k_proj.weight"] = tensors["q_proj.weight"][:dim].clone()
    stored["k"] = stored["q"][:dim].clone()
    dtype = torch.bfloat16 if matrix else torch.float32
    tensors, stored = rounded(tensors, dtype), rounded(stored, dtype)
    x = rand(T, hidden, seed=4).to(dtype).float()
    target = T - 1 - distance
    x[target] = 4.0 * x[T - 1]          # the same direction (after the unit norm the same key), a value four times as large
    names = {k: v.double() for k, v in stored.items()}
    want = pemarax_plain.attention_mixer(x.double(), table, names, 1e-5).float()
    blind = x.clone()
    blind[target] = -4.0 * x[T - 1]     # the opposite key: cosine minus one, no weight at all
    without = pemarax_plain.attention_mixer(blind.double(), table, names, 1e-5).float()
    share = float((want[-1] - without[-1]).abs().max() / want[-1].abs().max())
    return spec, tensors, x, want, share, dtype


@pytest.mark.parametrize("matrix", [False, True])
@pytest.mark.parametrize("feed", ["whole", "decoded", "cut"])
@pytest.mark.parametrize("distance, seen", [(1, True), (15, True), (16, True), (39, True), (40, False), (41, False),
                                             (300, False), (695, False), (696, True), (699, True)])
def test_a_key_counts_just_inside_the_window_and_among_the_kept_first_and_not_between(distance, seen, feed, matrix):
    """700 tokens, a window of 40 that keeps the first 4: the crafted key decides the last row when it is at most 39
    tokens back or one of the first four (696 to 699 back), and counts for nothing in between (there its share of
    the last row is exactly that of a key that is not there); from a prompt, decoded,
    and from a portion cut right behind the key; on pages of 16 tokens, whose older ones the window has given back."""
    T, window, keep = 700, 40, 4
    spec, tensors, x, want, share, dtype = crafted_attention(distance, T, window, keep, matrix)
    if seen:
        assert share > 0.3, f"the crafted key does not stand out: {share}"
    else:
        assert share < 1e-6, "the crafted key should not be seen"
    target = T - 1 - distance
    harness = PartHarness(spec, tensors, x.shape[1], dtype, page_size=16, capacity=720)
    if feed == "whole":
        got = harness.run([("r", x)])[0][-1]
    elif feed == "decoded":
        harness.run([("r", x[:T - 1])])
        got = harness.run([("r", x[T - 1:])])[0][-1]
    else:
        harness.run([("r", x[:target + 1])])
        got = harness.run([("r", x[target + 1:])])[0][-1]
    close(got, want[-1], dtype, f"distance {distance}")
    table = harness.cache.table(0, "r").pages
    assert table[0] >= 0 and table[1] == -1 and table[-1] >= 0, "the kept tokens' page stays, the passed ones are given back"


def test_the_sink_takes_its_share_of_a_single_key():
    """One token: the softmax over its own key and the sink.  A head's output is its value times e^s / (1 + e^s)
    with s = scale * q.k of the unit-normed query and key; without the sink it would be the value itself."""
    hidden, dim, H = 24, 16, 2
    spec, tensors, table, stored = attention_parts(hidden, H, 1, dim, dim, 8, 0, 0, 0, None, 70)
    x = rand(1, hidden, seed=5)
    names = {k: v.double() for k, v in stored.items()}
    want = pemarax_plain.attention_mixer(x.double(), table, names, 1e-5).float()
    unit = lambda v: v / torch.sqrt((v * v).mean() + 1e-5)
    key, value = unit(names["k"] @ x[0].double()), names["v"] @ x[0].double()
    heads = []
    for head in range(H):
        score = table["scale"] * float(unit((names["q"] @ x[0].double())[head * dim:(head + 1) * dim]) @ key)
        heads.append(value * (1.0 / (1.0 + torch.exp(torch.tensor(-score, dtype=torch.float64)))))
    by_hand = (names["o"] @ torch.cat(heads)).float()
    close(want[0], by_hand, torch.float32, "the plain implementation against the closed form")
    assert float((by_hand - (names["o"] @ value.repeat(H)).float()).abs().max()) > 0.05, "the sink changes nothing here"
    got = PartHarness(spec, tensors, hidden, torch.float32).run([("r", x)])[0]
    close(got, want, torch.float32, "one token")


def latent_parts(hidden, heads, dim, rot_dim, vdim, rank, window, rot_dims, seed, base=300.0, scale=None):
    table = pemarax_configs.latent(heads, dim, rot_dim, vdim, rank, window, rot_dims, base, scale)["mixer"]
    from macllm_infer_amd.config.pemarax import _latent_attention
    spec = _latent_attention(table, "mixer", 1e-5)[0].spec
    shapes = {"q": (heads * (dim + rot_dim), hidden), "dkv": (rank + rot_dim, hidden), "uk": (heads * dim, rank),
              "uv": (heads * vdim, rank), "o": (hidden, heads * vdim)}
    stored = {name: rand(*shape, seed=seed + i) / shape[1] ** 0.5 for i, (name, shape) in enumerate(shapes.items())}
    stored["dkv.norm"] = rand(rank, seed=seed + 9) * 0.1 + 1.0
    tensors = {f"{name}.weight": value for name, value in stored.items()}
    return spec, tensors, table, stored


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, dim, rot_dim, vdim, rank, window, rot_dims", [
    (3, 8, 8, 12, 16, 13, None), (2, 12, 4, 6, 20, 7, 2), (1, 16, 0, 16, 12, 100, None), (5, 24, 16, 8, 40, 300, 16),
    # widths the matrix-core kernels are built for (bfloat16)
    (4, 32, 32, 48, 64, 70, None), (6, 48, 32, 72, 96, 150, None), (3, 48, 64, 32, 128, 33, None)])
def test_latent_attention_with_direct_queries_and_a_window_alone(dtype, heads, dim, rot_dim, vdim, rank, window, rot_dims):
    hidden, T = 56, 170
    spec, tensors, table, stored = latent_parts(hidden, heads, dim, rot_dim, vdim, rank, window, rot_dims, 30)
    tensors, stored = rounded(tensors, dtype), rounded(stored, dtype)
    x = rand(T, hidden, seed=2).to(dtype).float()
    want = pemarax_plain.latent_attention_mixer(x.double(), table, {k: v.double() for k, v in stored.items()}, 1e-5).float()
    feed_every_way(lambda: PartHarness(spec, tensors, hidden, dtype, page_size=8, capacity=600), x, want, dtype,
                   beside=rand(40, hidden, seed=3))


@pytest.mark.parametrize("matrix", [False, True])
@pytest.mark.parametrize("feed", ["whole", "decoded", "cut"])
@pytest.mark.parametrize("distance, seen", [(1, True), (31, True), (32, True), (69, True), (70, False), (71, False), (400, False)])
def test_a_latent_key_counts_up_to_the_window_s_edge_and_not_beyond(distance, seen, feed, matrix):
    """The turned key part is a plain product of the token's row, so a row thirty times as large stands out; it
    decides the last row 69 tokens back (window 70) and is gone at 70."""
    hidden, T, window = 32, 500, 70
    spec, tensors, table, stored = (latent_parts(hidden, 3, 16, 32, 16, 32, window, None, 50, base=50.0, scale=0.5) if matrix else
                                    latent_parts(hidden, 2, 16, 8, 16, 16, window, None, 50, base=50.0, scale=1.0))
    dtype = torch.bfloat16 if matrix else torch.float32
    tensors, stored = rounded(tensors, dtype), rounded(stored, dtype)
    names = {k: v.double() for k, v in stored.items()}
    base = (rand(T, hidden, seed=4) * 0.3).to(dtype).float()
    target = T - 1 - distance
    best = None
    for sign in (1.0, -1.0):
        x = base.clone()
        x[target] = sign * 30.0 * base[target]
        want = pemarax_plain.latent_attention_mixer(x.double(), table, names, 1e-5).float()
        blind = base.clone()
        blind[target] = 0.0
        without = pemarax_plain.latent_attention_mixer(blind.double(), table, names, 1e-5).float()
        share = float((want[-1] - without[-1]).abs().max() / want[-1].abs().max())
        if best is None or share > best[2]:
            best = (x, want, share)
    x, want, share = best
    assert (share > 0.3) if seen else (share < 1e-6), f"the crafted key's share is {share}"
    harness = PartHarness(spec, tensors, hidden, dtype, page_size=16, capacity=520)
    if feed == "whole":
        got = harness.run([("r", x)])[0][-1]
    elif feed == "decoded":
        harness.run([("r", x[:T - 1])])
        got = harness.run([("r", x[T - 1:])])[0][-1]
    else:
        harness.run([("r", x[:target + 1])])
        got = harness.run([("r", x[target + 1:])])[0][-1]
    close(got, want[-1], dtype, f"distance {distance}")


def normed_attention_parts(hidden, H, G, dim, vdim, window, seed):
    table = {"dim": dim, "heads": H, "kv_heads": G, "vdim": vdim, "scale": dim ** -0.5, "mask": {"size": window}}
    from macllm_infer_amd.config.pemarax import _normed_attention
    spec = _normed_attention(table, "left", 1e-5)
    shapes = {"q": (H * dim, hidden), "k": (G * dim, hidden), "v": (G * vdim, hidden), "o": (hidden, H * vdim)}
    stored = {name: rand(*shape, seed=seed + i) / shape[1] ** 0.5 for i, (name, shape) in enumerate(shapes.items())}
    stored["q.norm"], stored["k.norm"] = rand(dim, seed=seed + 8) * 0.3 + 1.0, rand(dim, seed=seed + 9) * 0.3 + 1.0
    tensors = {f"{name}_proj.weight": stored[name] for name in ("q", "k", "v", "o")}
    tensors["q_norm.weight"], tensors["k_norm.weight"] = stored["q.norm"], stored["k.norm"]
    return spec, tensors, table, stored


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, G, dim, vdim, window", [(4, 2, 8, 12, 9), (2, 1, 12, 4, 30), (3, 3, 16, 16, 200),
                                                     (6, 2, 64, 128, 90), (4, 2, 128, 64, 33), (4, 4, 64, 64, 64)])
def test_windowed_attention_with_one_norm_weight_for_all_heads_alone(dtype, H, G, dim, vdim, window):
    hidden, T = 56, 170
    spec, tensors, table, stored = normed_attention_parts(hidden, H, G, dim, vdim, window, 30)
    tensors, stored = rounded(tensors, dtype), rounded(stored, dtype)
    x = rand(T, hidden, seed=2).to(dtype).float()
    want = pemarax_plain.windowed_attention(x.double(), table, {k: v.double() for k, v in stored.items()}, 1e-5).float()
    feed_every_way(lambda: PartHarness(spec, tensors, hidden, dtype, page_size=8, capacity=600), x, want, dtype,
                   beside=rand(40, hidden, seed=3))


@pytest.mark.parametrize("matrix", [False, True])
@pytest.mark.parametrize("feed", ["whole", "decoded", "cut"])
@pytest.mark.parametrize("distance, seen", [(1, True), (16, True), (52, True), (53, False), (54, False), (400, False)])
def test_a_normed_key_counts_up_to_its_window_s_edge_and_not_beyond(distance, seen, feed, matrix):
    """The left attention of a parallel layer, window 53, 500 tokens on pages of 16: the key projection is the query
    projection of head 0 and both norms share a weight, so a row in the last row's direction has cosine one with the
    last query whatever its length; four times as long, its value shows in the last row while the window holds it."""
    hidden, T, window = 32, 500, 53
    dim, vdim = (64, 128) if matrix else (16, 24)
    spec, tensors, table, stored = normed_attention_parts(hidden, 2, 1, dim, vdim, window, 60)
    table["scale"] = 12.0 / dim
    from macllm_infer_amd.config.pemarax import _normed_attention
    spec = _normed_attention(table, "left", 1e-5)
    tensors["k_proj.weight"] = tensors["q_proj.weight"][:dim].clone()
    stored["k"] = stored["q"][:dim].clone()
    tensors["k_norm.weight"] = tensors["q_norm.weight"].clone()
    stored["k.norm"] = stored["q.norm"].clone()
    dtype = torch.bfloat16 if matrix else torch.float32
    tensors, stored = rounded(tensors, dtype), rounded(stored, dtype)
    names = {k: v.double() for k, v in stored.items()}
    x = rand(T, hidden, seed=4).to(dtype).float()
    target = T - 1 - distance
    x[target] = 4.0 * x[T - 1]
    want = pemarax_plain.windowed_attention(x.double(), table, names, 1e-5).float()
    blind = x.clone()
    blind[target] = -4.0 * x[T - 1]
    without = pemarax_plain.windowed_attention(blind.double(), table, names, 1e-5).float()
    share = float((want[-1] - without[-1]).abs().max() / want[-1].abs().max())
    assert (share > 0.3) if seen else (share < 1e-6), f"the crafted key's share is {share}"
    harness = PartHarness(spec, tensors, hidden, dtype, page_size=16, capacity=520)
    if feed == "whole":
        got = harness.run([("r", x)])[0][-1]
    elif feed == "decoded":
        harness.run([("r", x[:T - 1])])
        got = harness.run([("r", x[T - 1:])])[0][-1]
    else:
        harness.run([("r", x[:target + 1])])
        got = harness.run([("r", x[target + 1:])])[0][-1]
    close(got, want[-1], dtype, f"distance {distance}")


def state_space_parts(hidden, heads, vdim, state, groups, norm_groups, conv, seed):
    table = {"conv": conv, "groups": groups, "heads": heads, "norm_groups": norm_groups, "state": state, "vdim": vdim}
    from macllm_infer_amd.config.pemarax import _state_space
    spec = _state_space(table, "right", 1e-5)
    inner, channels = heads * vdim, heads * vdim + 2 * groups * state
    stored = {"in": rand(2 * inner + 2 * groups * state + heads, hidden, seed=seed) / hidden ** 0.5,
              "conv": rand(channels, conv, seed=seed + 1) / conv ** 0.5, "conv.b": rand(channels, seed=seed + 2) * 0.1,
              "dt_bias": rand(heads, seed=seed + 3) * 0.5 - 1.0, "A_log": torch.log(torch.rand(heads, generator=torch.Generator().manual_seed(seed)) * 3.0 + 0.5),
              "D": rand(heads, seed=seed + 5) * 0.1 + 1.0, "norm": rand(inner, seed=seed + 6) * 0.1 + 1.0,
              "o": rand(hidden, inner, seed=seed + 7) / inner ** 0.5}
    tensors = {"in_proj.weight": stored["in"], "conv1d.weight": stored["conv"], "conv1d.bias": stored["conv.b"],
               "dt_bias": stored["dt_bias"], "A_log": stored["A_log"], "D": stored["D"], "norm.weight": stored["norm"],
               "out_proj.weight": stored["o"]}
    return spec, tensors, table, stored


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, vdim, state, groups, norm_groups, conv", [
    (3, 8, 12, 1, 1, 4), (4, 6, 8, 2, 2, 2), (5, 40, 24, 1, 1, 3), (4, 32, 32, 1, 2, 3), (8, 64, 128, 2, 4, 4), (2, 16, 64, 2, 1, 2)])
def test_the_state_space_mixer_with_groups_and_a_gated_norm_in_parts_alone(dtype, heads, vdim, state, groups, norm_groups, conv):
    hidden, T = 56, 170
    spec, tensors, table, stored = state_space_parts(hidden, heads, vdim, state, groups, norm_groups, conv, 30)
    keep = ("dt_bias", "A_log", "D")
    tensors = {k: (v if k in keep else v.to(dtype).float()) for k, v in tensors.items()}
    stored = {k: (v if k in keep else v.to(dtype).float()) for k, v in stored.items()}
    x = rand(T, hidden, seed=2).to(dtype).float()
    want = pemarax_plain.state_space(x.double(), table, {k: v.double() for k, v in stored.items()}, 1e-5).float()
    feed_every_way(lambda: PartHarness(spec, tensors, hidden, dtype, page_size=8, capacity=600), x, want, dtype,
                   beside=rand(40, hidden, seed=3), loose=2.0)


@pytest.mark.parametrize("cut", [None, 1, 2, 127, 128, 129, 300])
def test_the_state_keeps_its_first_token_over_hundreds_and_chunk_edges(cut):
    """Decays close to one and a first row ten times as large: what the first token left in the state still shows in
    the last row, 399 tokens on, whole and cut at and around the scan's chunks; a slot that is used again starts
    from zero."""
    hidden, T = 32, 400
    for dtype in DTYPES:
        spec, tensors, table, stored = state_space_parts(hidden, 2, 32, 32, 1, 1, 3, 11)
        tensors["A_log"] = stored["A_log"] = torch.full((2,), -6.0)          # exp(-exp(-6) dt): nearly no decay
        keep = ("dt_bias", "A_log", "D")
        tensors = {k: (v if k in keep else v.to(dtype).float()) for k, v in tensors.items()}
        stored = {k: (v if k in keep else v.to(dtype).float()) for k, v in stored.items()}
        x = (rand(T, hidden, seed=3) * 0.5).to(dtype).float()
        x[0] *= 10.0
        names = {k: v.double() for k, v in stored.items()}
        want = pemarax_plain.state_space(x.double(), table, names, 1e-5).float()
        blind = x.clone()
        blind[0] = 0.0
        without = pemarax_plain.state_space(blind.double(), table, names, 1e-5).float()
        assert float((want[-1] - without[-1]).abs().max()) > 0.05 * float(want[-1].abs().max()), "the first token left nothing"
        harness = PartHarness(spec, tensors, hidden, dtype, page_size=8, capacity=512)
        if cut is None:
            got = harness.run([("r", x)])[0]
        else:
            got = torch.cat([harness.run([("r", x[:cut])])[0], harness.run([("r", x[cut:])])[0]])
        close(got, want, dtype, f"cut {cut}", loose=2.0)
        harness.cache.finish("r")
        again = harness.run([("s", x[:50])])[0]
        close(again, want[:50], dtype, "a slot used again", loose=2.0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden, experts, top, inner, T", [(40, 5, 2, 24, 33), (64, 12, 4, 80, 200), (48, 4, 4, 8, 1),
                                                            (128, 7, 1, 64, 700)])
def test_the_mixture_of_ungated_experts_alone(dtype, hidden, experts, top, inner, T):
    from macllm_infer_amd.config.pemarax import _moe
    from macllm_infer_amd.kernels import build
    from macllm_infer_amd.parts import BuildContext, part_class
    table = pemarax_configs.moe(experts, top, inner)
    spec = _moe(table, "mlp")
    stored = {"router": rand(experts, hidden, seed=1) / hidden ** 0.5, "router.b": rand(experts, seed=2) * 0.3}
    for e in range(experts):
        stored[f"e{e}.up"] = rand(inner, hidden, seed=10 + e) / hidden ** 0.5
        stored[f"e{e}.down"] = rand(hidden, inner, seed=50 + e) / inner ** 0.5
    stored = rounded(stored, dtype)
    x = rand(T, hidden, seed=3).to(dtype).float()
    names = {k: v.double() for k, v in stored.items()}
    want = pemarax_plain.mixture(x.double(), table, names).float()
    margin = pemarax_plain.router_choice(x.double(), table, names)[2]
    tensors = {}
    for name, value in stored.items():
        tensors["p." + ("router.bias" if name == "router.b" else name + ".weight")] = value
    cls = part_class(spec)
    build.ensure_modules(cls.kernel_modules)
    part = cls(spec, "p", tensors, BuildContext(hidden_size=hidden, dtype=dtype, device=torch.device(DEV), max_context=64))
    got = part.forward(x.to(dtype).to(DEV)).float().cpu()
    clear = margin > (0.0 if dtype == torch.float32 else 0.02)           # 16-bit rounding may turn a close choice
    assert int(clear.sum()) >= T // 2
    close(got[clear], want[clear], dtype, "tokens whose choice is clear")


# ------------------------------------------------------------------ whole models
def model_dir(name, folder, dtype):
    return pemarax_configs.make_model_dir(name, folder, storage_dtype=torch.bfloat16 if dtype == "bfloat16" else torch.float32)


def engine_for(name, folder, dtype, capacity=512, page=8, requests=4, **more):
    from macllm_infer_amd.engine import Engine
    raw, tensors = model_dir(name, folder, dtype)
    engine = Engine(str(folder), dtype=dtype, device=DEV, kv_cache_block_tokens=page, kv_cache_capacity_tokens=capacity,
                    max_active_sequences=requests, **more)
    return engine, raw, tensors


def tokens_for(raw, count, seed):
    return torch.randint(0, raw["vocab"], (count,), generator=torch.Generator().manual_seed(seed)).tolist()


class Plain:
    """The plain model's logits of a sequence and, when asked, how far 16-bit rounding of the activations alone
    moves them at every position (``pemarax_plain.rounding_noise``)."""

    def __init__(self, raw, tensors, tokens):
        self.raw, self.tensors, self.tokens = raw, tensors, tokens
        self.logits = pemarax_plain.forward(raw, tensors, tokens).float()
        self._noise = self._margin = None

    @property
    def margin(self):
        """Per position, by how much its closest choice of experts is decided (in any layer)."""
        if self._margin is None:
            self._margin = pemarax_plain.choice_margins(self.raw, self.tensors, self.tokens).float()
        return self._margin

    @property
    def noise(self):
        if self._noise is None:
            self._noise = pemarax_plain.rounding_noise(self.raw, self.tensors, self.tokens, samples=6).float()
        return self._noise


def same(got, plain, rows, dtype, what):
    """Float32: every position within 2e-4 of the logits' scale.  Bfloat16: these small random models amplify
    rounding (a choice of experts that turns, a gated norm that divides by little), so the gate at a position is what
    rounding alone does to the plain model there: four times that, or 8 % of the scale where that is more; and the
    median position within 3 % of the scale or twice the plain model's median.  A position one of whose choices of
    experts is decided by less than 0.01 is left out, with the three positions behind it that the convolutions'
    taps carry it to (a few samples of the rounding need not turn that choice, the engine's may); at most half of
    the positions are."""
    want = plain.logits[rows]
    got = got.float().cpu()
    scale = max(1.0, float(plain.logits.abs().max()))
    if dtype == "float32":
        error = float((got - want).abs().max())
        assert error <= F32_GATE * scale, f"{what}: max error {error:.3e}"
        return
    noise = plain.noise[rows]
    error = (got - want).abs().max(dim=-1).values
    near = plain.margin < 0.01
    for reach in (1, 2, 3):
        near[reach:] |= plain.margin[:-reach] < 0.01
    close_call = near[rows]
    assert int(close_call.sum()) * 2 <= max(len(rows), 2), f"{what}: too many positions with close choices"
    error = torch.where(close_call, torch.zeros_like(error), error)
    gate = torch.maximum(4.0 * noise, torch.full_like(noise, 0.08 * scale))
    worst = int((error - gate).argmax())
    assert bool((error <= gate).all()), (f"{what}: row {rows[worst]} is off by {float(error[worst]):.3f} of {scale:.2f}; "
                                         f"rounding alone moves the plain model by {float(noise[worst]):.3f} there")
    if len(rows) >= 8:
        assert float(error.median()) <= max(0.03 * scale, 2.0 * float(noise.median())), \
            f"{what}: the median position is off by {float(error.median()):.3f} of {scale:.2f}"


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_the_stream_behind_every_layer(tmp_path, name, monkeypatch):
    """The residual stream after each layer in float32, against the plain model's: a fault shows in its layer."""
    engine, raw, tensors = engine_for(name, tmp_path, "float32")
    from macllm_infer_amd.engine import Lane
    from macllm_infer_amd.parts import norm as norm_module
    tokens = tokens_for(raw, 90, 5)
    _, behind = pemarax_plain.forward(raw, tensors, tokens, streams=True)
    seen = []
    blocks = engine.model.blocks
    for block in blocks:
        original = block.forward

        def wrapped(residual, step, caches, original=original):
            original(residual, step, caches)
            norm_module.fold_pending(residual)
            seen.append(residual.h.clone())
        monkeypatch.setattr(block, "forward", wrapped)
    engine.add_request("r")
    engine.step([Lane("r", tokens, [])])
    assert len(seen) == len(behind)
    for index, (got, want) in enumerate(zip(seen, behind)):
        error = float((got.cpu().double() - want).abs().max())
        assert error <= 2e-4 * max(1.0, float(want.abs().max())), f"layer {index} ({raw['layers'][index]['type']}): {error:.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_cut_decoded_and_mixed_steps_match_the_plain_model(tmp_path, name, dtype):
    from macllm_infer_amd.engine import Lane
    engine, raw, tensors = engine_for(name, tmp_path, dtype, capacity=640, page=8)
    long_tokens, short_tokens, other_tokens = tokens_for(raw, 230, 1), tokens_for(raw, 37, 2), tokens_for(raw, 95, 3)
    long_plain, short_plain, other_plain = (Plain(raw, tensors, t) for t in (long_tokens, short_tokens, other_tokens))
    # whole
    engine.add_request("whole")
    got = engine.step([Lane("whole", long_tokens, list(range(230)))])
    same(got, long_plain, list(range(230)), dtype, "whole")
    engine.finish("whole")
    # in portions of many sizes, down to two tokens and one, in the slot and on the pages the first request gave back
    engine.add_request("cut")
    sizes, cursor, pieces = [9, 2, 31, 1, 1, 64, 2, 17, 3, 100], 0, []
    for size in sizes:
        pieces.append(engine.step([Lane("cut", long_tokens[cursor:cursor + size], list(range(size)))]))
        cursor += size
    same(torch.cat(pieces), long_plain, list(range(230)), dtype, "portions")
    engine.finish("cut")
    # a prompt and then token by token
    engine.add_request("decode")
    pieces = [engine.step([Lane("decode", long_tokens[:150], [149])])]
    for position in range(150, 230):
        pieces.append(engine.step([Lane("decode", long_tokens[position:position + 1], [0])]))
    same(torch.cat(pieces), long_plain, list(range(149, 230)), dtype, "decoded")
    engine.finish("decode")
    # unequal requests side by side: portions of one beside single tokens of others, one joining late, one leaving early
    for request in ("a", "b"):
        engine.add_request(request)
    rows = {"a": [], "b": [], "c": []}
    at = {"a": 0, "b": 0, "c": 0}
    feeds = {"a": long_tokens, "b": short_tokens, "c": other_tokens}
    plan = [dict(a=40, b=1), dict(a=1, b=2), dict(a=64, b=1), dict(a=2, b=30, c=7), dict(a=1, b=1, c=1), dict(a=100, b=2, c=60),
            dict(a=1, c=1), dict(a=21, c=26)]
    for turn in plan:
        if "c" in turn and at["c"] == 0:
            engine.add_request("c")
        lanes = []
        for request, count in turn.items():
            lanes.append(Lane(request, feeds[request][at[request]:at[request] + count], list(range(count))))
            at[request] += count
        got = engine.step(lanes)
        cursor = 0
        for request, count in turn.items():
            rows[request].append(got[cursor:cursor + count])
            cursor += count
        if at["b"] == len(short_tokens) and engine.has_request("b"):
            engine.finish("b")
    for request, plain in (("a", long_plain), ("b", short_plain), ("c", other_plain)):
        same(torch.cat(rows[request]), plain, list(range(at[request])), dtype, f"request {request} beside others")
    engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_in_a_small_pool_and_the_first_tokens(tmp_path, dtype):
    """400 tokens decoded one by one on a pool of 192 cells: every attention layer has a window, so passed pages come
    back and are used again while the kept first tokens' page stays; and the logits of the very first tokens."""
    from macllm_infer_amd.engine import Lane
    engine, raw, tensors = engine_for("A", tmp_path, dtype, capacity=192, page=8, requests=2)
    tokens = tokens_for(raw, 400, 7)
    plain = Plain(raw, tensors, tokens)
    engine.add_request("r")
    pieces = [engine.step([Lane("r", tokens[:1], [0])]), engine.step([Lane("r", tokens[1:3], [0, 1])])]
    for position in range(3, 400):
        pieces.append(engine.step([Lane("r", tokens[position:position + 1], [0])]))
    same(torch.cat(pieces), plain, list(range(400)), dtype, "long decoding")
    stats = engine.cache.stats()
    assert all(group["used_pages"] < group["total_pages"] for group in stats["groups"])
    engine.cache.check()


def replay(folder, dtype, steps, max_tokens, out):
    lines = "".join(json.dumps(step) + "\n" for step in steps)
    done = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(folder), "--dtype", dtype,
                           "--out", str(out), "--max-tokens", str(max_tokens), "--page-tokens", "16"],
                          input=lines, capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    assert [line for line in done.stdout.splitlines() if line.startswith("done ")] == [f"done {s['step']}" for s in steps]


@pytest.mark.parametrize("name, dtype", [("A", "float32"), ("B", "bfloat16"), ("C", "float32"), ("C", "bfloat16")])
def test_replays_through_the_trace_runner_match_the_plain_model(tmp_path, name, dtype):
    raw, tensors = model_dir(name, tmp_path / "model", dtype)
    first, second, third = tokens_for(raw, 200, 1), tokens_for(raw, 70, 2), tokens_for(raw, 3, 3)
    plains = {"x": Plain(raw, tensors, first), "y": Plain(raw, tensors, second), "z": Plain(raw, tensors, third)}
    steps = [
        {"step": 0, "entries": [{"id": "x", "tokens": first[:90], "want": [0, 89]}, {"id": "z", "tokens": third[:2], "want": [1]}], "end": []},
        {"step": 1, "entries": [{"id": "x", "tokens": first[90:92], "want": [0, 1]}, {"id": "y", "tokens": second[:64], "want": [63]},
                                {"id": "z", "tokens": third[2:], "want": [0]}], "end": ["z"]},
        {"step": 2, "entries": [{"id": "y", "tokens": second[64:65], "want": []}], "end": []},
        {"step": 3, "entries": [{"id": "x", "tokens": first[92:200], "want": [107]}, {"id": "y", "tokens": second[65:], "want": [0, 4]}],
         "end": ["x", "y"]},
    ]
    wanted = {0: [("x", 0), ("x", 89), ("z", 1)], 1: [("x", 90), ("x", 91), ("y", 63), ("z", 2)], 3: [("x", 199), ("y", 65), ("y", 69)]}
    out = tmp_path / "out"
    replay(tmp_path / "model", dtype, steps, 384, out)
    assert not (out / "2.f32").exists(), "a step that wants nothing writes nothing"
    for step, rows in wanted.items():
        got = torch.from_numpy(np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(len(rows), raw["vocab"]))
        for index, (request, position) in enumerate(rows):
            same(got[index:index + 1], plains[request], [position], dtype, f"step {step} row {index}")


@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_entry_point(tmp_path, name):
    from macllm_infer_amd import LLM, EngineConfig, SamplingParams
    raw, tensors = model_dir(name, tmp_path, "float32")
    prompts = [tokens_for(raw, 33, 1), tokens_for(raw, 5, 2), tokens_for(raw, 61, 3)]
    llm = LLM(str(tmp_path), dtype="float32", kv_cache_block_tokens=8, kv_cache_capacity_tokens=384,
              engine_config=EngineConfig(max_active_sequences=2, scheduler_token_budget=24, prefill_token_quantum=7))
    greedy = SamplingParams(max_new_tokens=12, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0)
    results = llm.generate(prompts, greedy)
    for prompt, result in zip(prompts, results):
        assert result.finish_reason == "length" and len(result.token_ids) == 12
        logits = pemarax_plain.forward(raw, tensors, prompt + result.token_ids).float()
        for index, token in enumerate(result.token_ids):
            row = logits[len(prompt) - 1 + index]
            assert row[token] >= row.max() - 1e-3 * row.abs().max(), f"token {index} is not the plain model's best"


# ------------------------------------------------------------------ configurations drawn at random
def drawn_configuration(seed):
    """A configuration whose every size, option and order of layers is drawn: head sizes of 16 to 128 (also ones
    no matrix-core kernel takes), one to six heads, values narrower and wider than keys, windows of 3 to 200 keys,
    0 to 40 kept tokens, 0 to 5 taps, partial rotations with and without the ramp, latent ranks of 8 to 128 with
    turned parts of 0 to 64, one to three state-space groups and norm parts, 2 to 9 experts, layers without a
    feed-forward."""
    import random
    draw = random.Random(seed)
    width = draw.choice([24, 40, 56, 64, 96])

    def window():
        return draw.choice([3, 8, 17, 33, 64, 100, 200])

    def one_attention():
        dim = draw.choice([16, 24, 48, 64, 80, 128])
        G = draw.choice([1, 2, 3])
        rot = draw.choice([0, dim, dim // 2 if (dim // 2) % 2 == 0 else dim])
        scaling = draw.choice([None, (draw.choice([2.0, 4.0, 16.0]), draw.choice([16, 64, 256]), draw.choice([4.0, 16.0]), draw.choice([0.5, 1.0]))])
        return pemarax_configs.attention(G * draw.choice([1, 2]), G, dim, draw.choice([dim, dim // 2, dim + 16]), window(),
                                         draw.choice([0, 1, 7, 40]), draw.choice([0, 1, 2, 3, 5]), rot, scaling if rot else None,
                                         base=draw.choice([100.0, 1e4, 1e6]), scale=draw.choice([None, 0.2]))

    def one_latent():
        rot_dim = draw.choice([0, 8, 32, 64])
        return pemarax_configs.latent(draw.choice([1, 2, 5]), draw.choice([8, 16, 40]), rot_dim, draw.choice([8, 24, 48]),
                                      draw.choice([8, 24, 64, 96, 128]), window(), draw.choice([None, rot_dim // 2]) if rot_dim >= 8 else None,
                                      base=draw.choice([50.0, 1e5]))

    def one_parallel():
        G = draw.choice([1, 2])
        dim = draw.choice([16, 48, 64, 128])
        groups = draw.choice([1, 2, 3])
        heads = groups * draw.choice([1, 2])
        vdim = draw.choice([8, 16, 32, 64])
        parts = draw.choice([1, 2, heads]) if (heads * vdim) % 2 == 0 else 1
        return pemarax_configs.parallel((G * draw.choice([1, 3]), G, dim, draw.choice([dim, 2 * dim, 8]), window()),
                                        (heads, vdim, draw.choice([8, 16, 32, 64]), groups, parts, draw.choice([2, 3, 4])))

    layers = []
    for _ in range(draw.choice([2, 3, 4])):
        layer = draw.choice([one_attention, one_latent, one_parallel])()
        experts = draw.choice([2, 3, 5, 9])
        mlp = None if draw.random() < 0.25 else pemarax_configs.moe(experts, draw.randint(1, experts), draw.choice([8, 16, 40]))
        layers.append(pemarax_configs.with_mlp(layer, mlp))
    return {"architecture": "Pemarax", "width": width, "vocab": draw.choice([31, 100, 257]), "norm": {"eps": draw.choice([1e-5, 1e-6])},
            "residual_mult": draw.choice([0.3, 0.5, 1.0, 1.4]), "layers": layers}


DRAWN = [(seed, "float32") for seed in range(4100, 4116)] + [(seed, "bfloat16") for seed in (4102, 4104, 4106, 4110, 4113, 4115)]


@pytest.mark.parametrize("seed, dtype", DRAWN)
def test_randomly_drawn_configurations_whole_cut_and_side_by_side(tmp_path, seed, dtype):
    """Whole, in portions beside another request's single tokens, and decoded: float32 at every position, bfloat16
    (where head and state sizes that the matrix-core kernels take meet ones they do not) by the rounding gate."""
    from macllm_infer_amd.engine import Engine, Lane
    raw = drawn_configuration(seed)
    raw, tensors = pemarax_configs.make_model_dir(raw, tmp_path, seed=seed,
                                                  storage_dtype=torch.float32 if dtype == "float32" else torch.bfloat16)
    engine = Engine(str(tmp_path), dtype=dtype, device=DEV, kv_cache_block_tokens=draw_page(seed), kv_cache_capacity_tokens=640,
                    max_active_sequences=3)
    tokens, other = tokens_for(raw, 150, seed), tokens_for(raw, 30, seed + 1)
    plain, beside = Plain(raw, tensors, tokens), Plain(raw, tensors, other)
    engine.add_request("whole")
    same(engine.step([Lane("whole", tokens, list(range(150)))]), plain, list(range(150)), dtype, f"seed {seed} whole")
    engine.finish("whole")
    engine.add_request("cut")
    engine.add_request("other")
    pieces, others, cursor, fed = [], [], 0, 0
    for size in (5, 2, 40, 1, 1, 23, 64, 2, 12):
        lanes = [Lane("cut", tokens[cursor:cursor + size], list(range(size)))]
        if fed < 30:
            count = 1 if fed else 4
            lanes.append(Lane("other", other[fed:fed + count], list(range(count))))
        got = engine.step(lanes)
        pieces.append(got[:size])
        if fed < 30:
            others.append(got[size:])
            fed += count
        cursor += size
    same(torch.cat(pieces), plain, list(range(150)), dtype, f"seed {seed} portions")
    same(torch.cat(others), beside, list(range(fed)), dtype, f"seed {seed} the request beside")
    engine.cache.check()


def draw_page(seed):
    return (4, 8, 16, 32)[seed % 4]
