"""Motolix on the GPU: every mechanism alone against the plain implementation (tests/motolix_plain.py), and whole
models through the step function, the scheduler and the entry points: whole prompts, portions down to two tokens,
token-by-token decoding, unequal batches, pages and slots that are used again, keys far away and at page borders,
chunk edges of the state scan, the first tokens, long decoding, and sizes of many kinds."""
import math

import numpy as np
import pytest
import torch

import motolix_configs
import motolix_plain
import traces
from gates import BF16_MAX, BF16_RMS, bfloat16_close
from part_harness import DEV, PartHarness

pytestmark = pytest.mark.gpu

F32_GATE = 2e-4
EPS = 3e-6


def rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def stored(tensors, prefix="p"):
    """A part's tensors under the names the plain implementation reads: ``q_proj.weight`` -> ``p.q``,
    ``q_proj.bias`` -> ``p.q.b``, ``q_norm.weight`` -> ``p.q.norm``."""
    out = {}
    for name, value in tensors.items():
        name = name.replace("q_norm.", "q.norm.").replace("k_norm.", "k.norm.").replace("_proj.", ".")
        name = name[:-len(".weight")] if name.endswith(".weight") else name
        name = name[:-len(".bias")] + ".b" if name.endswith(".bias") else name
        out[f"{prefix}.{name}"] = value.to(torch.float64)
    return out


def rounded(tensors, dtype):
    return {name: value.to(dtype).float() if value.dim() >= 2 else value for name, value in tensors.items()}


def close(got, want, dtype, what=""):
    scale = max(1.0, float(want.abs().max()))
    gate = (F32_GATE if dtype == torch.float32 else 4e-2) * scale
    error = (got.double() - want.double()).abs()
    assert float(error.max()) <= gate, f"{what}: max error {float(error.max()):.3e} at row {int(error.max(dim=-1).values.argmax())}, gate {gate:.3e}"


def feed_every_way(make_harness, x, plain_rows, dtype, beside=None):
    """Whole, in portions (down to two tokens and one), token by token, and beside another request: every fed row
    against ``plain_rows``; slots and pages of finished feeds are used again by the next."""
    T = x.shape[0]
    harness = make_harness()
    out, = harness.run([("whole", x)])
    close(out, plain_rows, dtype, "whole")
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
    close(torch.cat(pieces), plain_rows, dtype, "portions")
    head = max(1, T - 40)
    pieces = [harness.run([("tail", x[:head])])[0]]
    for position in range(head, T):
        pieces.append(harness.run([("tail", x[position:position + 1])])[0])
    close(torch.cat(pieces), plain_rows, dtype, "token by token")


def rope_spec(rotation):
    from macllm_infer_amd.config import RopeSpec, WavelengthScalingSpec
    scaling = rotation.get("scaling")
    return RopeSpec(theta=rotation["base"], rotary_dim=rotation["dims"],
                    scaling=None if scaling is None else WavelengthScalingSpec(**scaling))


# ------------------------------------------------------------------ sigmoid attention whose values are its keys
def sigmoid_tensors(hidden, H, G, D, seed):
    return {"q_proj.weight": rand(H * D, hidden, seed=seed + 1, scale=hidden ** -0.5),
            "k_proj.weight": rand(G * D, hidden, seed=seed + 2, scale=hidden ** -0.5),
            "o_proj.weight": rand(hidden, H * D, seed=seed + 4, scale=(H * D) ** -0.5),
            "q_proj.bias": rand(H * D, seed=seed + 5, scale=0.2), "k_proj.bias": rand(G * D, seed=seed + 6, scale=0.2),
            "o_proj.bias": rand(hidden, seed=seed + 7, scale=0.2),
            "temp": rand(H, seed=seed + 8).abs() + 0.3, "pb": rand(H, seed=seed + 9) - 3.0}


def sigmoid_spec(H, G, D, scale, rotation):
    from macllm_infer_amd.config import AttentionSpec
    return AttentionSpec(num_heads=H, num_kv_heads=G, head_dim=D, scale=scale, position=rope_spec(rotation),
                         qkv_bias=True, out_bias=True, values_from_keys=True, head_temperature=True,
                         weighting="sigmoid", score_bias=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, G, D, rot_dims, scaling", [
    (6, 2, 16, 16, None), (3, 3, 24, 12, (8.0, 1.0, 4.0, 64)), (4, 2, 64, 32, (2.0, 1.0, 4.0, 512)),
    (2, 2, 128, 128, None), (5, 1, 8, 2, None), (1, 1, 80, 80, (16.0, 2.0, 8.0, 128)),
    (8, 1, 64, 64, None), (3, 1, 128, 64, None), (10, 2, 64, 16, None)])
def test_sigmoid_attention_alone(dtype, H, G, D, rot_dims, scaling):
    hidden = 40
    rotation = motolix_configs.rot(700.0, rot_dims, scaling)
    tensors = rounded(sigmoid_tensors(hidden, H, G, D, seed=D), dtype)
    mixer = {"heads": H, "kv_heads": G, "dim": D, "scale": 0.9 / math.sqrt(D), "rot": rotation}
    x = rand(230, hidden, seed=3).to(dtype).float()
    want = motolix_plain.sigmoid_attention(x.double(), "p", stored(tensors), mixer)
    make = lambda: PartHarness(sigmoid_spec(H, G, D, mixer["scale"], rotation), tensors, hidden, dtype, page_size=8)
    feed_every_way(make, x, want, dtype, beside=rand(64, hidden, seed=4))


def crafted_sigmoid(distance, length):
    """One head; a bias of -12 shuts every key out (weight 6e-6) except one: the last token's query and the key
    ``distance`` tokens before it have a score of +36.  The values are the keys, so that key's own first dim (6.0)
    shows in the output.  Nothing is turned that matters: the marked dims lie beyond the rotated ones."""
    hidden, D = 24, 8
    block = lambda first: torch.cat([torch.zeros(D, first), torch.eye(D), torch.zeros(D, hidden - first - D)], dim=1)
    tensors = {"q_proj.weight": block(8), "k_proj.weight": block(0),
               "o_proj.weight": torch.cat([torch.eye(D), torch.zeros(hidden - D, D)], dim=0),
               "q_proj.bias": torch.zeros(D), "k_proj.bias": torch.zeros(D), "o_proj.bias": torch.zeros(hidden),
               "temp": torch.tensor([1.0]), "pb": torch.tensor([-12.0])}
    x = rand(length, hidden, seed=distance, scale=0.05)
    query, key = length - 1, length - 1 - distance
    x[query, 8 + 7] = 6.0                          # the query's last dim (not turned: two dims are)
    x[key, 7] = 6.0                                # the key's last dim, which is also its value's
    return tensors, x, query, key, hidden


@pytest.mark.parametrize("feed", ["whole", "decoded", "cut"])
@pytest.mark.parametrize("distance", [0, 1, 7, 8, 15, 16, 17, 255, 256, 700])
def test_one_far_key_decides_a_sigmoid_head(distance, feed):
    """Keys the query's own, next to it, at the last cell of a page and the first of the next (pages of 8), and
    hundreds of tokens back; in a prompt, in decoding, and with the portion cut between the key and the query."""
    length = distance + 13
    tensors, x, query, key, hidden = crafted_sigmoid(distance, length)
    rotation = motolix_configs.rot(100.0, 2)
    mixer = {"heads": 1, "kv_heads": 1, "dim": 8, "scale": 1.0, "rot": rotation}
    want = motolix_plain.sigmoid_attention(x.double(), "p", stored(tensors), mixer)
    assert float(want[query, 7]) > 5.0                      # the plain model shows the key
    harness = PartHarness(sigmoid_spec(1, 1, 8, 1.0, rotation), tensors, hidden, torch.float32, page_size=8, capacity=1024)
    if feed == "whole":
        got = harness.run([("r", x)])[0]
    elif feed == "decoded":
        got = torch.cat([harness.run([("r", x[:key + 1])])[0]] +
                        [harness.run([("r", x[t:t + 1])])[0] for t in range(key + 1, length)])
    else:
        middle = min(length - 2, key + max(1, distance // 2))
        got = torch.cat([harness.run([("r", x[:middle])])[0], harness.run([("r", x[middle:])])[0]])
    close(got, want, torch.float32, f"distance {distance}, {feed}")
    assert float(got[query, 7]) > 5.0


def test_sigmoid_weights_are_not_normalized_and_the_bias_and_multiplier_count():
    """With a bias of +9 every key weighs about one: the output is the sum of the keys seen so far (it grows with
    the position), which no softmax gives; one head's multiplier and bias differ from the other's."""
    H, G, D, hidden = 2, 1, 16, 24
    tensors = sigmoid_tensors(hidden, H, G, D, seed=5)
    tensors["pb"] = torch.tensor([9.0, -1.0])
    tensors["temp"] = torch.tensor([0.01, 2.5])
    rotation = motolix_configs.rot(50.0, 16)
    mixer = {"heads": H, "kv_heads": G, "dim": D, "scale": 0.25, "rot": rotation}
    x = rand(90, hidden, seed=6)
    want = motolix_plain.sigmoid_attention(x.double(), "p", stored(tensors), mixer)
    other = motolix_plain.sigmoid_attention(x.double(), "p", stored(dict(tensors, temp=torch.tensor([0.01, 0.01]))), mixer)
    assert float((want - other).abs().max()) > 0.05
    harness = PartHarness(sigmoid_spec(H, G, D, 0.25, rotation), tensors, hidden, torch.float32, page_size=4)
    got = torch.cat([harness.run([("r", x[:61])])[0]] + [harness.run([("r", x[t:t + 1])])[0] for t in range(61, 90)])
    close(got, want, torch.float32, "unnormalized weights")


# ------------------------------------------------------------------ softmax attention, normed projections, turned values
def softmax_tensors(hidden, H, G, D, V, seed):
    return {"q_proj.weight": rand(H * D, hidden, seed=seed + 1, scale=hidden ** -0.5),
            "k_proj.weight": rand(G * D, hidden, seed=seed + 2, scale=hidden ** -0.5),
            "v_proj.weight": rand(G * V, hidden, seed=seed + 3, scale=hidden ** -0.5),
            "o_proj.weight": rand(hidden, H * V, seed=seed + 4, scale=(H * V) ** -0.5),
            "q_norm.weight": 1.0 + rand(H * D, seed=seed + 5, scale=0.3),
            "k_norm.weight": 1.0 + rand(G * D, seed=seed + 6, scale=0.3)}


def softmax_spec(H, G, D, V, scale, rotation):
    from macllm_infer_amd.config import AttentionSpec
    return AttentionSpec(num_heads=H, num_kv_heads=G, head_dim=D, scale=scale, position=rope_spec(rotation),
                         value_dim=V, projection_norm_eps=EPS, value_rotation_theta=rotation["base"])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, G, D, V, rot_dims, scaling", [
    (6, 2, 16, 16, 16, None), (3, 3, 24, 40, 12, None), (4, 1, 64, 64, 64, (4.0, 1.0, 4.0, 128)),
    (6, 2, 64, 80, 32, None), (2, 2, 128, 128, 128, None), (5, 1, 8, 24, 4, None), (2, 1, 48, 6, 48, None),
    (4, 2, 64, 128, 64, None), (2, 1, 128, 160, 64, None), (3, 1, 64, 32, 64, None), (8, 1, 64, 96, 32, None),
    (5, 1, 128, 72, 128, None), (1, 1, 64, 256, 64, None), (3, 1, 128, 12, 32, None), (2, 2, 64, 200, 64, None)])
def test_softmax_attention_with_normed_projections_and_turned_values_alone(dtype, H, G, D, V, rot_dims, scaling):
    hidden = 40
    rotation = motolix_configs.rot(3000.0, rot_dims, scaling)
    tensors = rounded(softmax_tensors(hidden, H, G, D, V, seed=D + V), dtype)
    mixer = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 4.0 / math.sqrt(D), "rot": rotation}
    x = rand(230, hidden, seed=3).to(dtype).float()
    want = motolix_plain.softmax_attention(x.double(), "p", stored(tensors), mixer, EPS)
    make = lambda: PartHarness(softmax_spec(H, G, D, V, mixer["scale"], rotation), tensors, hidden, dtype, page_size=8)
    feed_every_way(make, x, want, dtype, beside=rand(64, hidden, seed=4))


def test_the_projection_norm_runs_over_all_heads_at_once():
    """One head's query rows are made a hundred times larger: a norm per head would undo that, the norm over the
    whole projection shrinks every other head instead, and the plain model shows the difference."""
    H, G, D, V, hidden = 3, 1, 16, 16, 32
    tensors = softmax_tensors(hidden, H, G, D, V, seed=9)
    tensors["q_proj.weight"][:D] *= 100.0
    rotation = motolix_configs.rot(1000.0, 16)
    mixer = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 1.5, "rot": rotation}
    x = rand(70, hidden, seed=2)
    want = motolix_plain.softmax_attention(x.double(), "p", stored(tensors), mixer, EPS)
    harness = PartHarness(softmax_spec(H, G, D, V, 1.5, rotation), tensors, hidden, torch.float32, page_size=8)
    got = torch.cat([harness.run([("r", x[:50])])[0]] + [harness.run([("r", x[t:t + 1])])[0] for t in range(50, 70)])
    close(got, want, torch.float32, "norm over the whole projection")


@pytest.mark.parametrize("sigmoid, H, G, D, V", [(True, 4, 2, 64, 64), (True, 2, 1, 128, 128), (False, 6, 2, 64, 80),
                                                 (False, 2, 1, 128, 160), (False, 4, 4, 64, 32)])
def test_prompt_portions_in_bfloat16_run_on_the_matrix_cores(monkeypatch, sigmoid, H, G, D, V):
    """Heads of 64 and 128 in bfloat16: portions of prompts (alone and beside single tokens) go through the
    matrix-core kernel's forms for sigmoid weights and for values of another width than the keys, steps of single
    tokens through the kernel that splits a context over workgroups (several splits here); both against the plain
    model, and each is seen to have run."""
    from macllm_infer_amd.kernels import ops
    calls = {"forms": 0, "general": 0, "decode": 0}
    forms, general, decode = ops.prefill_attention_forms, ops.paged_attention, ops.decode_attention

    def spy_forms(*args, **more):
        calls["forms"] += 1
        return forms(*args, **more)

    def spy_general(*args, **more):
        calls["general"] += 1
        return general(*args, **more)

    def spy_decode(*args, **more):
        calls["decode"] += 1
        return decode(*args, **more)
    monkeypatch.setattr(ops, "prefill_attention_forms", spy_forms)
    monkeypatch.setattr(ops, "decode_attention", spy_decode)
    monkeypatch.setattr(ops, "paged_attention", spy_general)
    hidden, dtype = 64, torch.bfloat16
    rotation = motolix_configs.rot(2000.0, D // 2)
    x = rand(200, hidden, seed=11).to(dtype).float()
    if sigmoid:
        tensors = rounded(sigmoid_tensors(hidden, H, G, D, seed=V), dtype)
        mixer = {"heads": H, "kv_heads": G, "dim": D, "scale": 1.0 / math.sqrt(D), "rot": rotation}
        want = motolix_plain.sigmoid_attention(x.double(), "p", stored(tensors), mixer)
        spec = sigmoid_spec(H, G, D, mixer["scale"], rotation)
    else:
        tensors = rounded(softmax_tensors(hidden, H, G, D, V, seed=V), dtype)
        mixer = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 3.0 / math.sqrt(D), "rot": rotation}
        want = motolix_plain.softmax_attention(x.double(), "p", stored(tensors), mixer, EPS)
        spec = softmax_spec(H, G, D, V, mixer["scale"], rotation)
    harness = PartHarness(spec, tensors, hidden, dtype, page_size=16)
    first, = harness.run([("r", x[:70])])
    second, _ = harness.run([("r", x[70:170]), ("other", x[:1])])
    assert calls == {"forms": 2, "general": 0, "decode": 0}
    rows = [first, second]
    for position in range(170, 200):
        if position % 2:
            rows.append(harness.run([("r", x[position:position + 1])])[0])
        else:
            rows.append(harness.run([("other", x[position - 169:position - 168]), ("r", x[position:position + 1])])[1])
    assert calls == {"forms": 2, "general": 0, "decode": 30}
    close(torch.cat(rows), want, dtype, "portions on the matrix cores, single tokens over split contexts")


def crafted_softmax(distance, length, V=8):
    """One head whose last query and the key ``distance`` tokens back stand out (score about 30 against about 0);
    the key's value is (5, 0, 0, ...) before it is turned, so the output's first dim is 5 only if the value was
    turned by the key's position and the sum turned back by the query's, with a fast frequency (base 4)."""
    hidden, D = 24, 8
    block = lambda rows, first: torch.cat([torch.zeros(rows, first), torch.eye(rows), torch.zeros(rows, hidden - first - rows)], dim=1)
    tensors = {"q_proj.weight": block(D, 8), "k_proj.weight": block(D, 0), "v_proj.weight": block(V, 16),
               "o_proj.weight": torch.cat([torch.eye(V), torch.zeros(hidden - V, V)], dim=0),
               "q_norm.weight": torch.ones(D), "k_norm.weight": torch.ones(D)}
    x = rand(length, hidden, seed=distance, scale=0.05)
    query, key = length - 1, length - 1 - distance
    x[:, 0] = 1.0                                  # every key points along dim 0 once it is normed
    x[query, 8 + 7] = 30.0                         # normed to about sqrt(8): the score is about 8 * scale
    x[key, 7] = 30.0
    x[key, 16] = 5.0
    return tensors, x, query, key, hidden


@pytest.mark.parametrize("feed", ["whole", "decoded", "cut"])
@pytest.mark.parametrize("distance", [0, 1, 7, 8, 9, 16, 63, 64, 65, 300, 999])
def test_one_far_key_decides_a_softmax_head_and_its_value_is_turned_there_and_back(distance, feed):
    length = distance + 11
    tensors, x, query, key, hidden = crafted_softmax(distance, length)
    rotation = motolix_configs.rot(4.0, 2)
    mixer = {"heads": 1, "kv_heads": 1, "dim": 8, "vdim": 8, "scale": 4.0, "rot": rotation}
    want = motolix_plain.softmax_attention(x.double(), "p", stored(tensors), mixer, EPS)
    forward_only = motolix_plain.turn(torch.tensor([[[5.0, 0, 0, 0, 0, 0, 0, 0]]], dtype=torch.float64),
                                      torch.tensor([key]), motolix_plain.frequencies(4.0, 8), 8)
    if distance:
        back = motolix_plain.turn(forward_only, torch.tensor([query]), motolix_plain.frequencies(4.0, 8), 8, backwards=True)
        assert float((want[query, :8] - back[0, 0]).abs().max()) < 0.3        # the plain model shows the two turns
        assert float((back[0, 0] - forward_only[0, 0]).abs().max()) > 0.5
    harness = PartHarness(softmax_spec(1, 1, 8, 8, 4.0, rotation), tensors, hidden, torch.float32, page_size=8, capacity=1024)
    if feed == "whole":
        got = harness.run([("r", x)])[0]
    elif feed == "decoded":
        got = torch.cat([harness.run([("r", x[:key + 1])])[0]] +
                        [harness.run([("r", x[t:t + 1])])[0] for t in range(key + 1, length)])
    else:
        middle = min(length - 2, key + max(1, distance // 2))
        got = torch.cat([harness.run([("r", x[:middle])])[0], harness.run([("r", x[middle:])])[0]])
    close(got, want, torch.float32, f"distance {distance}, {feed}")


# ------------------------------------------------------------------ gated linear attention
def gated_tensors(hidden, H, D, V, rank, seed):
    return {"q.weight": rand(H * D, hidden, seed=seed + 1, scale=hidden ** -0.5),
            "k.weight": rand(H * D, hidden, seed=seed + 2, scale=hidden ** -0.5),
            "v.weight": rand(H * V, hidden, seed=seed + 3, scale=hidden ** -0.5),
            "g.weight": rand(H * V, hidden, seed=seed + 4, scale=hidden ** -0.5),
            "a1.weight": rand(rank, hidden, seed=seed + 5, scale=hidden ** -0.5),
            "a2.weight": rand(H * D, rank, seed=seed + 6, scale=2.0 * rank ** -0.5),
            "a2.bias": rand(H * D, seed=seed + 7) + 1.0,
            "norm.weight": 1.0 + rand(V, seed=seed + 8, scale=0.2),
            "o.weight": rand(hidden, H * V, seed=seed + 9, scale=(H * V) ** -0.5)}


def gated_spec(H, D, V, tau, rank=None):
    from macllm_infer_amd.config import GatedLinearAttentionSpec
    return GatedLinearAttentionSpec(num_heads=H, key_dim=D, value_dim=V, decay_temperature=tau, query_scale=D ** -0.5,
                                    norm_eps=EPS, decay_rank=rank)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, D, V, tau, rank", [(3, 16, 16, 16.0, 8), (2, 24, 40, 1.0, 5), (1, 64, 128, 4.0, 16),
                                                (4, 48, 32, 8.0, 12), (2, 72, 8, 2.5, 1), (1, 6, 262, 32.0, 3),
                                                (2, 130, 20, 16.0, 7)])
def test_gated_linear_attention_alone(dtype, H, D, V, tau, rank):
    """300 tokens: whole prompts run in passes over chunks of the scan, portions and single tokens walk from end to
    end, and all of them agree; a temperature of one makes the state forget within tens of tokens, 32 keeps it."""
    hidden = 48
    tensors = rounded(gated_tensors(hidden, H, D, V, rank, seed=D + V), dtype)
    mixer = {"heads": H, "dim": D, "vdim": V, "tau": tau}
    x = rand(300, hidden, seed=7).to(dtype).float()
    want, _ = motolix_plain.gated_linear(x.double(), "p", stored(tensors), mixer, EPS)
    feed_every_way(lambda: PartHarness(gated_spec(H, D, V, tau, rank), tensors, hidden, dtype, page_size=8), x, want,
                   dtype, beside=rand(64, hidden, seed=8))


@pytest.mark.parametrize("cut", [None, 1, 2, 127, 128, 129, 256, 399])
def test_the_state_keeps_the_first_token_over_hundreds_and_chunk_edges(cut):
    """One key channel never decays (its gate's bias is +40) and only the first token writes to it; the last token
    alone asks for it: what comes out is the first token's value whether the prompt runs whole (in chunks of the
    scan), is cut at a chunk's edge or next to it, right behind the first token, or before the last."""
    hidden, H, D, V, length = 16, 1, 8, 8, 400
    zero = lambda rows: torch.zeros(rows, hidden)
    tensors = {"q.weight": zero(D), "k.weight": zero(D), "v.weight": zero(V), "g.weight": zero(V),
               "a1.weight": zero(2), "a2.weight": torch.zeros(D, 2), "a2.bias": torch.full((D,), -2.0),
               "norm.weight": torch.ones(V), "o.weight": torch.cat([torch.eye(V), torch.zeros(hidden - V, V)], dim=0)}
    tensors["a2.bias"][0] = 40.0
    tensors["k.weight"][0, 0] = 1.0                # key channel 0 <- input 0
    tensors["q.weight"][0, 1] = 1.0                # query channel 0 <- input 1
    tensors["v.weight"][:, 2:2 + V] = torch.eye(V)
    tensors["g.weight"][:, 15] = 1.0               # the gate is SiLU(input 15) for every value channel
    x = torch.zeros(length, hidden)
    x[:, 15] = 3.0
    x[:, 2:10] = rand(length, 8, seed=1)
    x[1:, 3] += 0.2 * rand(length - 1, seed=2)
    x[0, 0] = 2.0                                  # only the first token has a key
    x[-1, 1] = 1.0                                 # only the last token has a query
    mixer = {"heads": H, "dim": D, "vdim": V, "tau": 2.0}
    want, _ = motolix_plain.gated_linear(x.double(), "p", stored(tensors), mixer, EPS)
    value = x[0, 2:10].double()
    expect = value / torch.sqrt((value * value).mean() + EPS) * (3.0 / (1.0 + math.exp(-3.0)))
    assert float((want[-1, :V] - expect).abs().max()) < 1e-3       # the plain model shows the first token's value
    harness = PartHarness(gated_spec(H, D, V, 2.0), tensors, hidden, torch.float32, page_size=8, capacity=512)
    if cut is None:
        got = harness.run([("r", x)])[0]
    else:
        got = torch.cat([harness.run([("r", x[:cut])])[0], harness.run([("r", x[cut:])])[0]])
    close(got, want, torch.float32, f"cut {cut}")
    assert float((got[-1, :V].double() - expect).abs().max()) < 1e-3


def test_a_state_slot_that_is_used_again_starts_from_zero():
    H, D, V, hidden = 2, 16, 16, 32
    tensors = gated_tensors(hidden, H, D, V, 4, seed=3)
    tensors["a2.bias"] += 6.0                      # a long memory: what a slot held before would show
    mixer = {"heads": H, "dim": D, "vdim": V, "tau": 8.0}
    harness = PartHarness(gated_spec(H, D, V, 8.0), tensors, hidden, torch.float32, page_size=8, requests=2)
    for index in range(5):
        x = rand(20 + index, hidden, seed=10 + index, scale=2.0)
        want, _ = motolix_plain.gated_linear(x.double(), "p", stored(tensors), mixer, EPS)
        other = rand(3, hidden, seed=20 + index)
        got, _ = harness.run([(f"r{index}", x[:9]), (f"o{index}", other)])
        rest, = harness.run([(f"r{index}", x[9:])])
        close(torch.cat([got, rest]), want, torch.float32, f"request {index}")
        harness.cache.finish(f"r{index}")
        harness.cache.finish(f"o{index}")


# ------------------------------------------------------------------ the feed-forward, the norms, the stream's mix
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden, inner, T", [(56, 136, 37), (328, 344, 5), (2560, 4104, 9)])
def test_the_gelu_gated_feed_forward_alone(dtype, hidden, inner, T):
    from macllm_infer_amd.config import SwiGLUSpec
    from macllm_infer_amd.kernels import build
    from macllm_infer_amd.parts import BuildContext, part_class
    context = BuildContext(hidden_size=hidden, dtype=dtype, device=torch.device(DEV), max_context=64)
    build.ensure_modules(("common", "gemm"))
    tensors = rounded({"p.gate_proj.weight": rand(inner, hidden, seed=1, scale=2.0 * hidden ** -0.5),
                       "p.up_proj.weight": rand(inner, hidden, seed=2, scale=hidden ** -0.5),
                       "p.down_proj.weight": rand(hidden, inner, seed=3, scale=inner ** -0.5)}, dtype)
    spec = SwiGLUSpec(intermediate_size=inner, activation="gelu_tanh")
    ffn = part_class(spec)(spec, "p", tensors, context)
    x = rand(T, hidden, seed=4, scale=1.5).to(dtype)
    got = ffn.forward(x.to(DEV)).float().cpu()
    names = {"p.gate": tensors["p.gate_proj.weight"].double(), "p.up": tensors["p.up_proj.weight"].double(),
             "p.down": tensors["p.down_proj.weight"].double()}
    want = motolix_plain.feed_forward(x.double(), "p", names)
    silu = (torch.nn.functional.silu(x.double() @ names["p.gate"].T) * (x.double() @ names["p.up"].T)) @ names["p.down"].T
    assert float((want - silu).abs().max()) > 0.02          # the two activations differ where it counts
    close(got, want, dtype, "feed-forward")


@pytest.mark.parametrize("hidden, inner, T", [(256, 136, 1), (64, 48, 9), (2560, 4104, 16), (96, 8, 17)])
def test_small_steps_in_bfloat16_gate_in_the_epilogue_of_their_product(monkeypatch, hidden, inner, T):
    """Weights stored in bfloat16 and up to 16 rows: act(gate) * up leaves the skinny product's epilogue (seen to have
    run, with the GELU), more rows go through the separate kernel; both against the plain implementation."""
    from macllm_infer_amd.config import SwiGLUSpec
    from macllm_infer_amd.kernels import build, ops
    from macllm_infer_amd.parts import BuildContext, part_class
    calls = []
    fused = ops.fused_gemm

    def spy(*args, **more):
        calls.append((more.get("epilogue"), more.get("gate_activation")))
        return fused(*args, **more)
    monkeypatch.setattr(ops, "fused_gemm", spy)
    dtype = torch.bfloat16
    context = BuildContext(hidden_size=hidden, dtype=dtype, device=torch.device(DEV), max_context=64)
    build.ensure_modules(("common", "gemm", "decode"))
    tensors = {"p.gate_proj.weight": rand(inner, hidden, seed=1, scale=2.0 * hidden ** -0.5).to(dtype),
               "p.up_proj.weight": rand(inner, hidden, seed=2, scale=hidden ** -0.5).to(dtype),
               "p.down_proj.weight": rand(hidden, inner, seed=3, scale=inner ** -0.5).to(dtype)}
    spec = SwiGLUSpec(intermediate_size=inner, activation="gelu_tanh")
    ffn = part_class(spec)(spec, "p", tensors, context)
    x = rand(T, hidden, seed=4, scale=1.5).to(dtype)
    got = ffn.forward(x.to(DEV)).float().cpu()
    names = {"p.gate": tensors["p.gate_proj.weight"].double(), "p.up": tensors["p.up_proj.weight"].double(),
             "p.down": tensors["p.down_proj.weight"].double()}
    want = motolix_plain.feed_forward(x.double(), "p", names)
    assert ((ops.EPI_SWIGLU, "gelu_tanh") in calls) == (T <= 16)
    close(got, want, dtype, "feed-forward")


# few rows keep a row in registers (one to eight elements a thread), many rows or wide ones lay it in LDS
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden, T, count", [(40, 19, 2), (328, 7, 1), (1500, 64, 2), (4104, 3, 2), (8192, 2, 1),
                                              (9000, 2, 1), (328, 300, 2), (2560, 257, 1)])
def test_a_branch_joins_the_stream_through_a_norm_of_its_own(dtype, hidden, T, count):
    """x <- x + LN_b(sum of factor * branch), then LN(x): the stream stays float32, the sum of the branches is
    never rounded; with an offset in the branches that a norm without centring would keep."""
    from macllm_infer_amd.config import LayerNormSpec
    from macllm_infer_amd.kernels import build
    from macllm_infer_amd.parts import BuildContext, part_class
    from macllm_infer_amd.parts.base import NormedBranches, Residual
    context = BuildContext(hidden_size=hidden, dtype=dtype, device=torch.device(DEV), max_context=64)
    build.ensure_modules(("common",))
    spec = LayerNormSpec(eps=EPS)
    weight, bias = 1.0 + rand(hidden, seed=1, scale=0.2), rand(hidden, seed=2, scale=0.3)
    norm = part_class(spec)(spec, "n", {"n.weight": weight, "n.bias": bias}, context)
    post_w, post_b = 1.0 + rand(hidden, seed=3, scale=0.2), rand(hidden, seed=4, scale=0.3)
    h = rand(T, hidden, seed=5)
    branches = [((rand(T, hidden, seed=6 + index) + 2.0).to(dtype), 1.3 - 0.6 * index) for index in range(count)]
    residual = Residual(h.clone().to(DEV))
    residual.pending = [NormedBranches([(rows.to(DEV), factor) for rows, factor in branches], post_w.to(DEV),
                                       post_b.to(DEV), EPS)]
    normed = norm.forward(residual).float().cpu()
    summed = sum(rows.double() * factor for rows, factor in branches)
    stream = h.double() + motolix_plain.layer_norm(summed, post_w.double(), post_b.double(), EPS)
    assert float((residual.h.cpu().double() - stream).abs().max()) < 2e-5
    close(normed, motolix_plain.layer_norm(stream, weight.double(), bias.double(), EPS), dtype, "norm")


# ------------------------------------------------------------------ whole models through the step function
def model_dir(name, folder, dtype):
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    return motolix_configs.make_model_dir(name, folder, dtype=storage)


def engine_for(name, folder, dtype, capacity=512, page=8, requests=4, **more):
    from macllm_infer_amd.engine import Engine
    raw, tensors = model_dir(name, folder, dtype)
    engine = Engine(str(folder), dtype=dtype, device=DEV, kv_cache_block_tokens=page, kv_cache_capacity_tokens=capacity,
                    max_active_sequences=requests, **more)
    return engine, raw, tensors


def tokens_for(raw, count, seed):
    return torch.randint(0, raw["vocab"], (count,), generator=torch.Generator().manual_seed(seed)).tolist()


def plain(raw, tensors, tokens):
    return motolix_plain.forward(tokens, tensors, raw)


def noise_of(raw, tensors, tokens, rows=None):
    """What rounding activations to bfloat16 alone does to the plain model's logits at ``rows`` of ``tokens``."""
    def measure():
        noise = motolix_plain.rounding_noise(tokens, tensors, raw, plain(raw, tensors, tokens)).numpy()
        return noise if rows is None else noise[rows]
    return measure


def same(got, want, dtype, what, noise=None):
    """float32: the float32 gate.  bfloat16: the plain gate (6 % of the scale at the worst place, 3 % relative
    RMS); where a model amplifies rounding beyond it at single positions (a branch whose output nearly cancels is
    stretched to unit variance by the norm behind it), position by position at most four times what rounding alone
    does to the plain model there (``noise``: callables giving it for the rows of ``want``, in order), and at the
    median position within 3 % of the scale or twice the median of that noise."""
    got, want = got.float().cpu().numpy(), want.float().numpy()
    error = np.abs(got - want).max(axis=-1)
    if dtype == "float32":
        gate = F32_GATE * max(1.0, float(np.abs(want).max()))
        assert error.max() <= gate, f"{what}: max error {error.max():.3e} at row {int(np.argmax(error))}, gate {gate:.3e}"
        return
    if bfloat16_close(got, want):
        return
    scale = float(np.abs(want).max())
    text = f"{what}: max error {error.max():.3e} at row {int(np.argmax(error))} of scale {scale:.2f}"
    assert noise is not None, text
    measured = np.concatenate([np.atleast_1d(one()) for one in (noise if isinstance(noise, (list, tuple)) else [noise])])
    allowed = np.maximum(BF16_MAX * scale, 4.0 * measured)
    beyond = np.nonzero(error > allowed)[0]
    assert beyond.size == 0 and np.median(error) <= max(BF16_RMS * scale, 2.0 * float(np.median(measured))), \
        f"{text}; rounding alone: {measured.max():.3e}; rows beyond four times their own noise: {beyond.tolist()[:8]}"


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_the_stream_behind_every_run_of_a_layer(tmp_path, name):
    """Layer by layer in float32: the residual stream behind every run (a looped layer counts each time), read
    from the engine's own step through a hook on the blocks."""
    from macllm_infer_amd.engine import Lane
    from macllm_infer_amd.parts.norm import fold_pending
    engine, raw, tensors = engine_for(name, tmp_path, "float32")
    tokens = tokens_for(raw, 37, 4)
    want = []
    motolix_plain.forward(tokens, tensors, raw, stream_after=want)
    seen = []
    for block in engine.model.blocks:
        inner = block.forward

        def hooked(residual, step, caches, inner=inner):
            inner(residual, step, caches)
            fold_pending(residual)
            seen.append(residual.h.detach().float().cpu().clone())
        block.forward = hooked
    engine.add_request("r")
    engine.step([Lane("r", tokens, [36])])
    assert len(seen) == len(want)
    for index, (got, rows) in enumerate(zip(seen, want)):
        close(got, rows, torch.float32, f"behind run {index}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_whole_cut_decoded_and_mixed_steps_match_the_plain_model(tmp_path, name, dtype):
    """One request whole (long enough for the scans to run in chunks); the same tokens in portions of many sizes in
    a slot and pages that were used before; its tail token by token; then unequal requests side by side, portions
    beside single tokens, one of them sitting out a step."""
    from macllm_infer_amd.engine import Lane
    engine, raw, tensors = engine_for(name, tmp_path, dtype, capacity=640)
    first, second, third = tokens_for(raw, 300, 1), tokens_for(raw, 41, 2), tokens_for(raw, 150, 3)
    want = {0: plain(raw, tensors, first), 1: plain(raw, tensors, second), 2: plain(raw, tensors, third)}
    engine.add_request("whole")
    same(engine.step([Lane("whole", first, list(range(300)))]), want[0], dtype, "whole", noise_of(raw, tensors, first))
    engine.finish("whole")
    engine.add_request("cut")
    outputs, cursor, turn = [], 0, 0
    sizes = [7, 2, 5, 3, 11, 2, 1, 1, 13, 2, 131, 2, 9, 1, 1, 64]
    while cursor < 260:
        size = min(sizes[turn % len(sizes)], 260 - cursor)
        outputs.append(engine.step([Lane("cut", first[cursor:cursor + size], list(range(size)))]))
        cursor, turn = cursor + size, turn + 1
    for position in range(260, 300):
        outputs.append(engine.step([Lane("cut", first[position:position + 1], [0])]))
    same(torch.cat(outputs), want[0], dtype, "portions and single tokens", noise_of(raw, tensors, first))
    engine.finish("cut")
    for request in "cde":
        engine.add_request(request)
    one = engine.step([Lane("c", first[:20], [19]), Lane("d", second[:3], [0, 1, 2]), Lane("e", third[:140], [0, 139])])
    two = engine.step([Lane("d", second[3:30], list(range(27))), Lane("c", first[20:21], [0])])
    three = engine.step([Lane("c", first[21:22], [0]), Lane("e", third[140:141], [0]), Lane("d", second[30:41], [10])])
    four = engine.step([Lane("e", third[141:150], [8]), Lane("c", first[22:170], [147])])
    got = torch.cat([one, two, three, four])
    rows = torch.cat([want[0][19:20], want[1][:3], want[2][0:1], want[2][139:140], want[1][3:30], want[0][20:21],
                      want[0][21:22], want[2][140:141], want[1][40:41], want[2][149:150], want[0][169:170]])
    same(got, rows, dtype, "mixed steps", [
        noise_of(raw, tensors, first, [19]), noise_of(raw, tensors, second, [0, 1, 2]), noise_of(raw, tensors, third, [0, 139]),
        noise_of(raw, tensors, second, list(range(3, 30))), noise_of(raw, tensors, first, [20, 21]),
        noise_of(raw, tensors, third, [140]), noise_of(raw, tensors, second, [40]), noise_of(raw, tensors, third, [149]),
        noise_of(raw, tensors, first, [169])])
    engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_the_first_tokens(tmp_path, dtype):
    """Three tokens of a prompt and 330 decoded one by one: the states are carried through hundreds of steps and
    the keys of every pass fill page after page; beside it requests of one and two tokens come and go in the same
    slot and pages."""
    from macllm_infer_amd.engine import Lane
    engine, raw, tensors = engine_for("D", tmp_path, dtype, capacity=352, page=8, requests=2)
    tokens = tokens_for(raw, 333, 5)
    want = plain(raw, tensors, tokens)
    short = tokens_for(raw, 2, 6)
    want_short = plain(raw, tensors, short)
    engine.add_request("long")
    outputs = [engine.step([Lane("long", tokens[:3], [0, 1, 2])])]
    for position in range(3, 333):
        if position % 50 == 10:
            engine.add_request("short")
            both = engine.step([Lane("short", short[:1], [0]), Lane("long", tokens[position:position + 1], [0])])
            same(both[:1], want_short[:1], dtype, "a sequence's first token", noise_of(raw, tensors, short, [0]))
            outputs.append(both[1:])
        elif position % 50 == 11:
            both = engine.step([Lane("long", tokens[position:position + 1], [0]), Lane("short", short[1:], [0])])
            same(both[1:], want_short[1:], dtype, "a sequence's second token", noise_of(raw, tensors, short, [1]))
            outputs.append(both[:1])
            engine.finish("short")
        else:
            outputs.append(engine.step([Lane("long", tokens[position:position + 1], [0])]))
    same(torch.cat(outputs), want, dtype, "long decoding", noise_of(raw, tensors, tokens))
    engine.finish("long")
    engine.cache.check()


@pytest.mark.parametrize("name, dtype", [("A", "float32"), ("B", "bfloat16"), ("C", "float32"), ("D", "bfloat16")])
def test_replays_of_every_kind_match_the_plain_model(tmp_path, name, dtype):
    """Through the replay program, which drives the engine's step function as generation does: whole, the tail
    decoded, portions, and up to four live requests in a pool that holds the peak and no more."""
    folder = tmp_path / "model"
    raw, tensors = model_dir(name, folder, dtype)
    generator = torch.Generator().manual_seed(9)
    requests = {f"r{index}": torch.randint(0, raw["vocab"], (length,), generator=generator).tolist()
                for index, length in enumerate([5, 64, 65, 190])}
    steps, families = [], {}
    for label, family in (("whole", traces.whole), ("tail", traces.tail_decoded), ("portions", traces.portions)):
        renamed = {f"{label}_{key}": tokens for key, tokens in requests.items()}
        families.update(renamed)
        steps += family(renamed)
    mixed = {f"m{index}": torch.randint(0, raw["vocab"], (length,), generator=generator).tolist()
             for index, length in enumerate([50, 97, 64, 33, 120, 71, 16])}
    families.update(mixed)
    steps += traces.mixed(mixed, seed=3)
    traces.number(steps)
    traces.replay(str(folder), dtype, steps, max_tokens=max(traces.peak_tokens(steps), 256), out_dir=tmp_path / "out")
    got = traces.collect(steps, tmp_path / "out", raw["vocab"], {key: len(tokens) for key, tokens in families.items()})
    for key, tokens in families.items():
        assert not np.isnan(got[key]).any(), f"{key}: a wanted row was not written"
        same(torch.from_numpy(got[key]), plain(raw, tensors, tokens), dtype, key, noise_of(raw, tensors, tokens))


@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_entry_point(tmp_path, name):
    """``LLM.generate``: the scheduler admits, cuts prompts into portions beside decoded tokens, samples (greedy) and
    finishes; more requests than slots, so slots and pages are used again."""
    from macllm_infer_amd import LLM, EngineConfig, SamplingParams
    raw, tensors = model_dir(name, tmp_path, "float32")
    llm = LLM(str(tmp_path), dtype="float32", device=DEV, kv_cache_block_tokens=8, kv_cache_capacity_tokens=384,
              engine_config=EngineConfig(max_active_sequences=3, scheduler_token_budget=40, prefill_token_quantum=16))
    prompts = [tokens_for(raw, length, 20 + length) for length in (17, 5, 150, 1, 33)]
    params = SamplingParams(max_new_tokens=8, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0, ignore_eos=True)
    results = llm.generate(prompts, params)
    for prompt, result in zip(prompts, results):
        want = motolix_plain.greedy(prompt, tensors, raw, 8)
        if list(result.token_ids) != want:
            # a near tie between two tokens may fall the other way: then the plain model must show the tie
            place = next(i for i, (a, b) in enumerate(zip(result.token_ids, want)) if a != b)
            logits = plain(raw, tensors, prompt + want[:place])[-1]
            top = torch.topk(logits, 2).values
            assert float(top[0] - top[1]) < 1e-3, f"prompt of {len(prompt)}: token {place} differs without a tie"
