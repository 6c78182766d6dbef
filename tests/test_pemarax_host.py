"""Pemarax through the engine on the CPU, the kernels replaced by their plain PyTorch references: configuration,
tensor names, cache and state handling, the step function and the scheduler against the plain whole-sequence
implementation (tests/pemarax_plain.py)."""
import json

import pytest
import torch

import pemarax_configs
import pemarax_plain
import ref_ops
from macllm_infer_amd.cache import CacheManager
from macllm_infer_amd.cache.manager import KVNeed
from macllm_infer_amd.config import ConfigError, PemaraxConfig, config_from_dict
from macllm_infer_amd.engine import Engine, EngineConfig, Lane, Scheduler
from macllm_infer_amd.engine.model import DecoderModel
from macllm_infer_amd.parts.position import rotary_frequencies
from macllm_infer_amd.sampling import Sampler, SamplingParams


@pytest.fixture
def host_ops(monkeypatch):
    ref_ops.install(monkeypatch)


def engine_for(name, folder, capacity=256, page=8, requests=4):
    raw, tensors = pemarax_configs.make_model_dir(name, folder)
    engine = Engine(str(folder), dtype="float32", device="cpu", kv_cache_block_tokens=page,
                    kv_cache_capacity_tokens=capacity, max_active_sequences=requests, check_device=False)
    return engine, raw, tensors


def tokens_for(raw, count, seed):
    return torch.randint(0, raw["vocab"], (count,), generator=torch.Generator().manual_seed(seed)).tolist()


def plain(raw, tensors, tokens):
    return pemarax_plain.forward(raw, tensors, tokens).to(torch.float32)


def test_the_configuration_is_read_from_its_own_keys_and_round_trips():
    config = config_from_dict(pemarax_configs.PEM_A)
    assert isinstance(config, PemaraxConfig)
    spec = config.to_model_spec()
    assert spec.hidden_size == 48 and spec.vocab_size == 101 and len(spec.layers) == 4
    assert [len(layer.mixers) for layer in spec.layers] == [2, 1, 1, 1]
    assert all(layer.branch_multiplier == 0.6 and layer.mixer_norm.weight_offset == 1.0 for layer in spec.layers)
    left, right = spec.layers[0].mixers
    assert (left.name, right.name, left.weight, right.weight) == ("mix.left", "mix.right", 0.5, 0.5)
    assert left.post_norm.weight_offset == 0.0 and right.post_norm.eps == 1e-5
    assert (left.spec.num_heads, left.spec.num_kv_heads, left.spec.head_dim, left.spec.value_dim, left.spec.window) == (4, 2, 8, 12, 9)
    assert left.spec.head_norm == "before_rotation" and left.spec.head_norm_weight and left.spec.position.kind == "none"
    assert left.spec.fixed_sink is None and left.spec.conv_kernel == 0
    assert (right.spec.num_heads, right.spec.head_dim, right.spec.state_size, right.spec.num_groups, right.spec.norm_parts,
            right.spec.conv_kernel) == (3, 8, 12, 1, 1, 4)
    attention = spec.layers[1].mixers[0].spec
    assert (attention.window, attention.keep_first, attention.conv_kernel, attention.fixed_sink) == (11, 3, 3, 0.0)
    assert attention.head_norm == "after_rotation" and not attention.head_norm_weight
    assert attention.position.kind == "rope_interleaved" and attention.position.scaling.factor == 4.0
    latent = spec.layers[2].mixers[0].spec
    assert latent.q_rank is None and (latent.kv_rank, latent.rope_dim, latent.window) == (16, 8, 13)
    assert latent.position.kind == "rope" and spec.layers[2].ffn is None
    ffn = spec.layers[3].ffn
    assert (ffn.num_experts, ffn.top_k, ffn.expert_size, ffn.routing) == (6, 1, 16, "top_then_softmax")
    assert not ffn.activation.gated
    assert PemaraxConfig.from_dict(json.loads(json.dumps(config.to_dict()))) == config
    names = {spec.stored_name(expect.name) for expect in DecoderModel.expected_tensors(spec)}
    assert {"embed", "head", "final.norm", "l0.norm1", "l0.norm2", "l0.mix.left.q", "l0.mix.left.q.norm", "l0.mix.left.k.norm",
            "l0.mix.left.o", "l0.mix.left.out", "l0.mix.right.in", "l0.mix.right.conv", "l0.mix.right.conv.b",
            "l0.mix.right.dt_bias", "l0.mix.right.A_log", "l0.mix.right.D", "l0.mix.right.norm", "l0.mix.right.o",
            "l0.mix.right.out", "l0.mlp.router", "l0.mlp.router.b", "l0.mlp.e0.up", "l0.mlp.e4.down", "l1.mix.q",
            "l1.mix.q.conv", "l1.mix.k.conv", "l1.mix.v.conv", "l1.mix.o", "l2.mix.q", "l2.mix.dkv", "l2.mix.dkv.norm",
            "l2.mix.uk", "l2.mix.uv", "l2.mix.o"} <= names
    assert not any(name.endswith(".gate") or "correction" in name or ".dq" in name for name in names)
    other = config_from_dict(pemarax_configs.PEM_B).to_model_spec()
    assert other.layers[0].branch_multiplier == 1.0 and other.layers[2].ffn is None
    assert other.layers[4].mixers[0].spec.conv_kernel == 0 and other.layers[4].mixers[0].spec.position.kind == "none"
    assert other.layers[3].mixers[0].spec.rope_dim == 0 and other.layers[2].mixers[1].spec.norm_parts == 2


@pytest.mark.parametrize("broken, text", [
    (dict(width=None), "width"), (dict(layers=[]), "layers"), (dict(norm={}), "norm.eps"),
    (dict(layers=[{"type": "conv", "mixer": {}}]), "type"),
    (dict(layers=[dict(pemarax_configs.PEM_A["layers"][1], mlp={"kind": "dense"})]), "mlp.kind"),
    (dict(layers=[dict(pemarax_configs.PEM_A["layers"][2], mixer={"heads": 2})]), "mixer.rot_dim|mixer.dim")])
def test_a_broken_configuration_names_its_key(broken, text):
    raw = dict(pemarax_configs.PEM_A, **broken)
    if broken.get("width", 1) is None:
        del raw["width"]
    with pytest.raises(ConfigError, match=text):
        config_from_dict(raw)


def test_ramp_scaled_frequencies_against_the_plain_ones():
    from macllm_infer_amd.config import RampScalingSpec
    for base, dims, numbers in ((10000.0, 16, (4.0, 64, 8.0, 1.0)), (777.0, 12, (8.0, 32, 4.0, 0.5)), (250000.0, 48, (6.0, 1024, 24.0, 2.0)),
                                (100.0, 8, (2.0, 16, 1.0, 1.0))):
        scaling = RampScalingSpec(*numbers)
        want, magnitude = pemarax_plain.rotary_frequencies(base, dims, dict(zip(("factor", "original", "fast", "slow"), numbers)))
        got = rotary_frequencies(base, dims, scaling)
        assert max(abs(a - b) / b for a, b in zip(got, want)) < 1e-12 and abs(scaling.magnitude - magnitude) < 1e-12
        assert any(abs(a - b) > 1e-9 for a, b in zip(got, rotary_frequencies(base, dims))), "the scaling changes nothing"


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_cut_and_token_by_token_match_the_plain_model(host_ops, tmp_path, name):
    engine, raw, tensors = engine_for(name, tmp_path)
    tokens = tokens_for(raw, 61, 3)
    expected = plain(raw, tensors, tokens)
    engine.add_request("whole")
    got = engine.step([Lane("whole", tokens, list(range(len(tokens))))])
    assert torch.allclose(got, expected, atol=2e-4, rtol=1e-4)
    engine.add_request("cut")
    rows, at = [], 0
    for size in (2, 7, 1, 1, 9, 2, 19, 1, 1, 1, 17):          # portions down to two tokens, single tokens between
        rows.append(engine.step([Lane("cut", tokens[at:at + size], list(range(size)))]))
        at += size
    assert at == len(tokens)
    assert torch.allclose(torch.cat(rows), expected, atol=2e-4, rtol=1e-4)
    engine.finish("whole")
    engine.finish("cut")
    engine.cache.check()


def test_unequal_requests_in_one_batch_and_reused_slots_and_pages(host_ops, tmp_path):
    engine, raw, tensors = engine_for("A", tmp_path, capacity=96, page=8, requests=3)
    prompts = {name: tokens_for(raw, count, seed) for name, count, seed in (("a", 21, 1), ("b", 5, 2), ("c", 33, 3))}
    expected = {name: plain(raw, tensors, tokens) for name, tokens in prompts.items()}
    for turn in range(2):                                      # the second turn takes the slots and pages of the first
        for name in prompts:
            engine.add_request(name)
        at = {name: 0 for name in prompts}
        got = {name: [] for name in prompts}
        sizes = {"a": [4, 1, 1, 15], "b": [1, 1, 1, 2], "c": [16, 9, 7, 1]}
        for step in range(4):
            lanes = [Lane(name, prompts[name][at[name]:at[name] + sizes[name][step]], list(range(sizes[name][step])))
                     for name in prompts]
            rows = engine.step(lanes)
            first = 0
            for name in prompts:
                size = sizes[name][step]
                got[name].append(rows[first:first + size])
                first += size
                at[name] += size
        for name in prompts:
            assert torch.allclose(torch.cat(got[name]), expected[name], atol=2e-4, rtol=1e-4), (turn, name)
            engine.finish(name)
        engine.cache.check()


def test_a_window_gives_pages_back_but_never_those_of_the_kept_first_tokens():
    """Two groups on pages of 4: a window of 6 that keeps the first 5 tokens (two pages stay for good), and a plain
    window of 6."""
    needs = {(0, "kept"): [KVNeed(1, 8, 6, None, 5)], (1, "plain"): [KVNeed(1, 8, 6)]}
    cache = CacheManager(needs, {}, 4, 64, 2, torch.float32, "cpu")
    cache.add_request("r")
    for _ in range(5):
        cache.reserve([("r", 8)])
        cache.commit("r", 8)
    kept, plain_pages = cache.table(0, "r").pages, cache.table(1, "r").pages
    assert len(kept) == len(plain_pages) == 10
    # the next query, at position 40, sees keys from 35 on: pages 0 to 7 are passed
    assert [page >= 0 for page in plain_pages] == [False] * 8 + [True] * 2
    assert [page >= 0 for page in kept] == [True, True] + [False] * 6 + [True] * 2
    cache.check()
    cache.finish("r")
    assert all(group["free_pages"] == group["total_pages"] for group in cache.stats()["groups"])


def test_long_decoding_in_a_pool_smaller_than_the_request(host_ops, tmp_path):
    """Every attention layer of B has a window (the longest 100 keys), so a request outgrows the pool: 190 tokens on
    128 cells."""
    engine, raw, tensors = engine_for("B", tmp_path, capacity=128, page=4, requests=2)
    tokens = tokens_for(raw, 190, 9)
    expected = plain(raw, tensors, tokens)
    engine.add_request("r")
    rows = [engine.step([Lane("r", tokens[:40], list(range(40)))])]
    for position in range(40, 190):
        rows.append(engine.step([Lane("r", tokens[position:position + 1], [0])]))
    assert torch.allclose(torch.cat(rows), expected, atol=3e-4, rtol=1e-4)
    engine.cache.check()


def test_greedy_generation_through_the_scheduler(host_ops, tmp_path):
    engine, raw, tensors = engine_for("A", tmp_path, capacity=256, page=8, requests=3)
    sampler = Sampler(engine.vocab_size, "cpu", check_device=False)
    scheduler = Scheduler(engine, sampler, EngineConfig(max_active_sequences=3, scheduler_token_budget=24,
                                                        prefill_token_quantum=7))
    prompts = [tokens_for(raw, 19, 1), tokens_for(raw, 3, 2), tokens_for(raw, 8, 3), tokens_for(raw, 1, 4)]
    greedy = SamplingParams(max_new_tokens=5, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0)
    for index, prompt in enumerate(prompts):
        scheduler.submit(index, prompt, greedy)
    finished = scheduler.run()
    for index, prompt in enumerate(prompts):
        tokens = list(prompt)
        for _ in range(5):
            tokens.append(int(plain(raw, tensors, tokens)[-1].argmax()))
        assert finished[index].generated == tokens[len(prompt):], index
    stats = engine.cache.stats()
    assert stats["live_requests"] == 0 and stats["free_slots"] == 3
