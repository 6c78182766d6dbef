"""Motolix through the engine on the CPU, the kernels replaced by their plain PyTorch references: configuration,
tensor names, cache and state handling, the step function and the scheduler against the plain whole-sequence
implementation (tests/motolix_plain.py)."""
import copy
import json

import pytest
import torch

import motolix_configs
import motolix_plain
import ref_ops
from macllm_infer_amd.config import ConfigError, MotolixConfig, config_from_dict
from macllm_infer_amd.engine import Engine, EngineConfig, Lane, Scheduler
from macllm_infer_amd.engine.model import DecoderModel
from macllm_infer_amd.sampling import Sampler, SamplingParams
from macllm_infer_amd.weights.loader import WeightError


@pytest.fixture
def host_ops(monkeypatch):
    ref_ops.install(monkeypatch)


def engine_for(name, folder, capacity=256, page=8, requests=4):
    raw, tensors = motolix_configs.make_model_dir(name, folder)
    engine = Engine(str(folder), dtype="float32", device="cpu", kv_cache_block_tokens=page,
                    kv_cache_capacity_tokens=capacity, max_active_sequences=requests, check_device=False)
    return engine, raw, tensors


def tokens_for(raw, count, seed):
    return torch.randint(0, raw["vocab"], (count,), generator=torch.Generator().manual_seed(seed)).tolist()


def plain(raw, tensors, tokens):
    return motolix_plain.forward(tokens, tensors, raw).to(torch.float32)


def test_the_configuration_is_read_from_its_own_keys_and_round_trips():
    config = config_from_dict(motolix_configs.MOT_D)
    assert isinstance(config, MotolixConfig)
    spec = config.to_model_spec()
    assert spec.hidden_size == 80 and spec.vocab_size == 57 and len(spec.layers) == 4
    assert [slot.spec.kind for layer in spec.layers for slot in layer.mixers] == \
        ["attention", "attention", "gated_linear_attention", "attention", "attention", "gated_linear_attention"]
    # the looped layers 1 and 2 run twice, each run an entry of its own; a pass begins with the stream's mix
    assert [entry.layer for entry in spec.schedule] == [0, 1, 2, 1, 2, 3]
    begins = [(index, entry.before.row) for index, entry in enumerate(spec.schedule) if entry.before is not None]
    assert begins == [(1, 0), (3, 1)] and spec.schedule[1].before.mix_name == "loop.in"
    first = spec.layers[0].mixers[0].spec
    assert (first.num_heads, first.num_kv_heads, first.head_dim, first.value_width) == (5, 1, 16, 16)
    assert first.weighting == "sigmoid" and first.values_from_keys and first.head_temperature and first.score_bias
    left, right = (slot.spec for slot in spec.layers[1].mixers)
    assert (left.num_heads, left.num_kv_heads, left.head_dim, left.value_width) == (2, 2, 48, 16)
    assert left.position.rotary_dim == 24 and left.value_rotation_theta == 2e4 and left.projection_norm_eps == 2e-5
    assert (right.num_heads, right.key_dim, right.value_dim, right.decay_temperature) == (5, 16, 8, 32.0)
    assert [slot.weight for slot in spec.layers[1].mixers] == [1.0, 2.0]
    assert spec.layers[2].ffn is None and spec.layers[0].ffn.intermediate_size == 48
    assert spec.layers[2].mixers[0].spec.position.scaling.factor == 16.0
    assert spec.embedding_multiplier == 5.0 and spec.logit_multiplier == 2.0
    assert MotolixConfig.from_dict(json.loads(json.dumps(config.to_dict()))) == config
    names = {spec.stored_name(expect.name) for expect in DecoderModel.expected_tensors(spec)}
    assert {"embed", "head", "final.norm", "final.norm.b", "loop.in", "loop.step", "l0.norm1", "l0.norm1.b", "l0.norm1b",
            "l0.norm2b.b", "l0.mix.q", "l0.mix.q.b", "l0.mix.k.b", "l0.mix.o.b", "l0.mix.temp", "l0.mix.pb",
            "l1.mix.left.q", "l1.mix.left.q.norm", "l1.mix.left.k.norm", "l1.mix.left.v", "l1.mix.left.o",
            "l1.mix.right.a1", "l1.mix.right.a2", "l1.mix.right.a2.b", "l1.mix.right.g", "l1.mix.right.norm",
            "l1.mlp.gate", "l1.mlp.up", "l1.mlp.down"} <= names
    assert "l0.mix.v" not in names and "l1.mix.left.q.b" not in names


def test_the_run_order_of_every_loop():
    for raw, order in ((motolix_configs.MOT_A, [0, 1, 0, 1, 0, 1, 2]), (motolix_configs.MOT_B, [0, 1, 2]),
                       (motolix_configs.MOT_C, [0, 1, 2, 3])):
        config = config_from_dict(raw)
        assert [entry.layer for entry in config.run_order()] == order
    config = config_from_dict(motolix_configs.MOT_C)
    assert [index for index, entry in enumerate(config.run_order()) if entry.before is not None] == [2]
    # keys and values of every run count: layer 1 of configuration A runs three times
    assert config_from_dict(motolix_configs.MOT_A).kv_bytes_per_token(2) == 2 * (3 * (2 * (16 + 8) + 2 * 32) + 1 * 64)


def broken(path, value):
    raw = copy.deepcopy(motolix_configs.MOT_A)
    table = raw
    for key in path[:-1]:
        table = table[key]
    if value is None:
        del table[path[-1]]
    else:
        table[path[-1]] = value
    return raw


@pytest.mark.parametrize("path, value, text", [
    (("width",), None, "width"), (("layers",), [], "layers"), (("norm",), {}, "norm"),
    (("layers", 0, "type"), "conv", "type"), (("layers", 1, "mixer", "vdim"), 8, "vdim"),
    (("layers", 0, "mixer", "right", "tau"), None, "tau"), (("layers", 0, "mixer", "left", "rot"), None, "rot"),
    (("layers", 1, "mixer", "kv_heads"), 3, "multiple"), (("loop", "stop"), 9, "loop"),
    (("layers", 1, "mlp", "kind"), "experts", "kind")])
def test_a_broken_configuration_names_its_key(path, value, text):
    with pytest.raises(ConfigError, match=text):
        config_from_dict(broken(path, value))


def test_the_decay_width_comes_from_the_tensors_and_a_tensor_too_many_is_refused(host_ops, tmp_path):
    from macllm_infer_amd.weights.safetensors_io import write_safetensors
    raw, tensors = motolix_configs.make_model_dir("B", tmp_path)
    rank = tensors["l1.mix.right.a1"].shape[0]
    assert tensors["l1.mix.right.a2"].shape == (3 * 8, rank)
    tokens = tokens_for(raw, 12, 5)
    engine = Engine(str(tmp_path), dtype="float32", device="cpu", kv_cache_block_tokens=8,
                    kv_cache_capacity_tokens=64, max_active_sequences=2, check_device=False)
    engine.add_request("a")
    assert (engine.step([Lane("a", tokens, list(range(12)))]) - plain(raw, tensors, tokens)).abs().max() < 2e-4
    write_safetensors(str(tmp_path / "model.safetensors"), dict(tensors, **{"l0.mix.v": torch.zeros(72, 48)}))
    with pytest.raises(WeightError, match="l0.mix.v"):
        Engine(str(tmp_path), dtype="float32", device="cpu", check_device=False, kv_cache_capacity_tokens=64)


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_whole_cut_and_mixed_steps_match_the_plain_model(host_ops, tmp_path, name):
    engine, raw, tensors = engine_for(name, tmp_path, capacity=160, page=8)
    first, second = tokens_for(raw, 60, 1), tokens_for(raw, 41, 2)
    want_first, want_second = plain(raw, tensors, first), plain(raw, tensors, second)
    engine.add_request("whole")
    got = engine.step([Lane("whole", first, list(range(60)))])
    assert (got - want_first).abs().max() < 2e-4
    engine.finish("whole")
    engine.add_request("cut")                                  # its slot and pages were used before
    outputs, cursor = [], 0
    for size in [7, 2, 5, 3, 11, 2, 1, 1, 13, 2, 2, 9, 1, 1]:
        outputs.append(engine.step([Lane("cut", first[cursor:cursor + size], list(range(size)))]))
        cursor += size
    assert cursor == 60 and (torch.cat(outputs) - want_first).abs().max() < 2e-4
    engine.finish("cut")
    engine.add_request("c")
    engine.add_request("d")
    one = engine.step([Lane("c", first[:20], [19]), Lane("d", second[:3], [0, 1, 2])])
    two = engine.step([Lane("d", second[3:30], list(range(27))), Lane("c", first[20:21], [0])])
    three = engine.step([Lane("c", first[21:22], [0]), Lane("d", second[30:41], [10])])
    assert (one[0] - want_first[19]).abs().max() < 2e-4 and (one[1:] - want_second[:3]).abs().max() < 2e-4
    assert (two[:27] - want_second[3:30]).abs().max() < 2e-4 and (two[27] - want_first[20]).abs().max() < 2e-4
    assert (three[0] - want_first[21]).abs().max() < 2e-4 and (three[1] - want_second[40]).abs().max() < 2e-4
    engine.cache.check()


def test_every_pass_of_the_loop_has_a_cache_and_a_state_of_its_own(host_ops, tmp_path):
    """Configuration A runs its first two layers three times: three caches of keys and three states for the same
    weights; all of them go back to the pool when the request ends."""
    engine, raw, tensors = engine_for("A", tmp_path, capacity=64, page=8, requests=2)
    keys = [key for key in engine.cache.entries if key[1] == "mix.left"] if hasattr(engine.cache, "entries") else None
    tokens = tokens_for(raw, 30, 3)
    engine.add_request("a")
    got = engine.step([Lane("a", tokens, list(range(30)))])
    assert (got - plain(raw, tensors, tokens)).abs().max() < 2e-4
    stats = engine.cache.stats()
    assert stats["live_requests"] == 1
    engine.finish("a")
    stats = engine.cache.stats()
    assert stats["live_requests"] == 0 and stats["free_slots"] == 2
    assert all(group["used_pages"] == 0 for group in stats["groups"])
    if keys is not None:
        assert len(keys) == 4                                   # three runs of layer 0 and the one of layer 2
    engine.cache.check()


def test_greedy_generation_through_the_scheduler(host_ops, tmp_path):
    engine, raw, tensors = engine_for("D", tmp_path, capacity=256, page=8, requests=3)
    sampler = Sampler(engine.vocab_size, "cpu", check_device=False)
    scheduler = Scheduler(engine, sampler, EngineConfig(max_active_sequences=3, scheduler_token_budget=24,
                                                        prefill_token_quantum=7))
    prompts = [tokens_for(raw, 17, 21), tokens_for(raw, 5, 22), tokens_for(raw, 30, 23), tokens_for(raw, 1, 24)]
    greedy = SamplingParams(max_new_tokens=6, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0)
    for index, prompt in enumerate(prompts):
        scheduler.submit(index, prompt, greedy)
    finished = scheduler.run()
    for index, prompt in enumerate(prompts):
        assert finished[index].generated == motolix_plain.greedy(prompt, tensors, raw, 6)
    stats = engine.cache.stats()
    assert stats["live_requests"] == 0 and stats["free_slots"] == 3
