"""Mukutar through the engine on the CPU, the kernels replaced by their plain PyTorch references: configuration,
tensor names, cache and state handling, the step function and the scheduler against the plain whole-sequence
implementation (tests/mukutar_plain.py)."""
import json

import pytest
import torch

import mukutar_configs
import mukutar_plain
import ref_ops
from macllm_infer_amd.config import ConfigError, MukutarConfig, config_from_dict
from macllm_infer_amd.engine import Engine, EngineConfig, Lane, Scheduler
from macllm_infer_amd.engine.model import DecoderModel
from macllm_infer_amd.sampling import Sampler, SamplingParams
from macllm_infer_amd.weights.loader import WeightError


@pytest.fixture
def host_ops(monkeypatch):
    ref_ops.install(monkeypatch)


def engine_for(name, folder, capacity=256, page=8, requests=4):
    raw, tensors = mukutar_configs.make_model_dir(name, folder)
    engine = Engine(str(folder), dtype="float32", device="cpu", kv_cache_block_tokens=page,
                    kv_cache_capacity_tokens=capacity, max_active_sequences=requests, check_device=False)
    return engine, raw, tensors


def tokens_for(raw, count, seed):
    return torch.randint(0, raw["vocab"], (count,), generator=torch.Generator().manual_seed(seed)).tolist()


def plain(raw, tensors, tokens):
    return mukutar_plain.forward(raw, tensors, tokens).to(torch.float32)


def test_the_configuration_is_read_from_its_own_keys_and_round_trips():
    config = config_from_dict(mukutar_configs.MUK_B)
    assert isinstance(config, MukutarConfig)
    spec = config.to_model_spec()
    assert spec.hidden_size == 48 and spec.vocab_size == 131 and len(spec.layers) == 5
    assert [slot.spec.kind for layer in spec.layers for slot in layer.mixers] == \
        ["attention", "retention", "general_delta", "attention", "retention"]
    first = spec.layers[0].mixers[0].spec
    assert (first.num_heads, first.num_kv_heads, first.head_dim, first.value_width, first.window) == (3, 1, 32, 16, 21)
    assert first.scale == 0.3 and first.sink and first.position.kind == "log_distance"
    assert spec.layers[1].ffn is None and spec.layers[0].ffn.intermediate_size == 56
    assert spec.layers[1].mixers[0].spec.position.rotary_dim == 12
    assert spec.layers[4].mixers[0].spec.position.kind == "none"
    assert spec.final_norm.weight_offset == 1.0
    assert MukutarConfig.from_dict(json.loads(json.dumps(config.to_dict()))) == config
    names = {spec.stored_name(expect.name) for expect in DecoderModel.expected_tensors(spec)}
    assert {"embed", "head", "final.norm", "l0.norm1", "l0.ls1", "l0.mix.q", "l0.mix.q.b", "l0.mix.r1", "l0.mix.sink",
            "l0.mix.o", "l0.mlp.up", "l0.mlp.act", "l1.mix.g", "l2.mix.w1", "l2.mix.w0", "l2.mix.a.b",
            "l2.mix.norm"} <= names


@pytest.mark.parametrize("broken, text", [
    (dict(width=None), "width"), (dict(layers=[]), "layers"), (dict(norm={}), "norm.eps"),
    (dict(layers=[{"type": "conv", "mixer": {}}]), "type"),
    (dict(layers=[{"type": "retention", "mixer": {"dim": 8, "heads": 2, "decay": [0.9]}}]), "decay"),
    (dict(layers=[{"type": "attention", "mixer": {"dim": 8, "heads": 3, "kv_heads": 2, "scale": 1.0}}]), "multiple")])
def test_a_broken_configuration_names_its_key(broken, text):
    raw = dict(mukutar_configs.MUK_A, **broken)
    if broken.get("width", 1) is None:
        del raw["width"]
    with pytest.raises(ConfigError, match=text):
        config_from_dict(raw)


def test_the_decay_rank_comes_from_the_tensors_when_the_configuration_has_none(host_ops, tmp_path):
    raw, tensors = mukutar_configs.make_model_dir("A", tmp_path)
    del raw["layers"][0]["mixer"]["decay_rank"]
    with open(tmp_path / "config.json", "w") as handle:
        json.dump(raw, handle)
    engine = Engine(str(tmp_path), dtype="float32", device="cpu", kv_cache_block_tokens=8,
                    kv_cache_capacity_tokens=64, max_active_sequences=2, check_device=False)
    tokens = tokens_for(raw, 12, 5)
    engine.add_request("a")
    got = engine.step([Lane("a", tokens, list(range(12)))])
    assert (got - plain(raw, tensors, tokens)).abs().max() < 2e-4


def test_a_layer_without_a_feed_forward_may_or_may_not_store_its_second_norm(host_ops, tmp_path):
    from macllm_infer_amd.weights.safetensors_io import write_safetensors
    raw, tensors = mukutar_configs.make_model_dir("B", tmp_path)
    assert "l1.norm2" in tensors                                   # the writer stores it; the model does not use it
    tokens = tokens_for(raw, 9, 3)
    want = plain(raw, tensors, tokens)
    for drop in (False, True):
        stored = {name: tensor for name, tensor in tensors.items() if not (drop and name in ("l1.norm2", "l1.ls2"))}
        write_safetensors(str(tmp_path / "model.safetensors"), stored)
        engine = Engine(str(tmp_path), dtype="float32", device="cpu", kv_cache_block_tokens=8,
                        kv_cache_capacity_tokens=64, max_active_sequences=2, check_device=False)
        engine.add_request("a")
        assert (engine.step([Lane("a", tokens, list(range(9)))]) - want).abs().max() < 2e-4
    stored["l1.mix.extra"] = torch.zeros(3)
    write_safetensors(str(tmp_path / "model.safetensors"), stored)
    with pytest.raises(WeightError, match="l1.mix.extra"):
        Engine(str(tmp_path), dtype="float32", device="cpu", check_device=False, kv_cache_capacity_tokens=64)


@pytest.mark.parametrize("name", ["A", "B"])
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


def test_windows_give_their_pages_back_and_a_small_pool_serves_a_long_request(host_ops, tmp_path):
    """The attention layers of configuration A see 9 tokens: a pool of 32 tokens is enough for a request of 120,
    decoded token by token after a prompt in portions, and what the logits are does not depend on it."""
    engine, raw, tensors = engine_for("A", tmp_path, capacity=32, page=4, requests=2)
    tokens = tokens_for(raw, 120, 7)
    want = plain(raw, tensors, tokens)
    engine.add_request("long")
    outputs, cursor = [], 0
    for size in [10, 6, 12, 2] + [1] * 90:
        outputs.append(engine.step([Lane("long", tokens[cursor:cursor + size], list(range(size)))]))
        cursor += size
    assert cursor == 120 and (torch.cat(outputs) - want).abs().max() < 3e-4
    assert engine.cache.stats()["groups"][0]["used_pages"] <= 4
    engine.finish("long")
    engine.cache.check()


def test_greedy_generation_through_the_scheduler(host_ops, tmp_path):
    engine, raw, tensors = engine_for("B", tmp_path, capacity=256, page=8, requests=3)
    sampler = Sampler(engine.vocab_size, "cpu", check_device=False)
    scheduler = Scheduler(engine, sampler, EngineConfig(max_active_sequences=3, scheduler_token_budget=24,
                                                        prefill_token_quantum=7))
    prompts = [tokens_for(raw, 17, 21), tokens_for(raw, 5, 22), tokens_for(raw, 30, 23), tokens_for(raw, 1, 24)]
    greedy = SamplingParams(max_new_tokens=6, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0)
    for index, prompt in enumerate(prompts):
        scheduler.submit(index, prompt, greedy)
    finished = scheduler.run()
    for index, prompt in enumerate(prompts):
        assert finished[index].generated == mukutar_plain.greedy(raw, tensors, prompt, 6)
    stats = engine.cache.stats()
    assert stats["live_requests"] == 0 and stats["free_slots"] == 3
