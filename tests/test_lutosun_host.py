"""Lutosun through the engine on the CPU, the kernels replaced by their plain PyTorch references: configuration,
tensor names, cache and state handling, the step function and the scheduler against the plain whole-sequence
implementation (tests/lutosun_plain.py)."""
import json

import pytest
import torch

import lutosun_configs
import lutosun_plain
import ref_ops
from macllm_infer_amd.config import ConfigError, LutosunConfig, config_from_dict
from macllm_infer_amd.engine import Engine, EngineConfig, Lane, Scheduler
from macllm_infer_amd.engine.model import DecoderModel
from macllm_infer_amd.sampling import Sampler, SamplingParams


@pytest.fixture
def host_ops(monkeypatch):
    ref_ops.install(monkeypatch)


def engine_for(name, folder, capacity=256, page=8, requests=4):
    raw, tensors = lutosun_configs.make_model_dir(name, folder)
    engine = Engine(str(folder), dtype="float32", device="cpu", kv_cache_block_tokens=page,
                    kv_cache_capacity_tokens=capacity, max_active_sequences=requests, check_device=False)
    return engine, raw, tensors


def tokens_for(raw, count, seed):
    return torch.randint(0, raw["vocab"], (count,), generator=torch.Generator().manual_seed(seed)).tolist()


def plain(raw, tensors, tokens):
    return lutosun_plain.forward(tokens, tensors, raw).to(torch.float32)


def test_the_configuration_is_read_from_its_own_keys_and_round_trips():
    config = config_from_dict(lutosun_configs.LUT_A)
    assert isinstance(config, LutosunConfig)
    spec = config.to_model_spec()
    assert spec.hidden_size == 48 and spec.vocab_size == 97 and len(spec.layers) == 4
    # the two middle layers run three times in a row, each run with a cache of its own
    assert [entry.layer for entry in spec.schedule] == [0, 1, 2, 1, 2, 1, 2, 3]
    before = [entry.before for entry in spec.schedule]
    assert [one is not None for one in before] == [False, True, False, True, False, True, False, False]
    assert (before[1].embedding, before[1].row) == (False, 0) and (before[3].embedding, before[3].row) == (True, 1)
    assert before[5].row == 2 and before[5].vector_name == "loop.step"
    mixer = spec.layers[0].mixers[0].spec
    assert (mixer.num_heads, mixer.head_dim, mixer.rope_dim, mixer.value_dim, mixer.q_rank, mixer.kv_rank) == (3, 16, 8, 12, 20, 24)
    assert mixer.position.kind == "rope_interleaved" and mixer.position.rotary_dim == 8
    ffn = spec.layers[0].ffn
    assert (ffn.num_experts, ffn.top_k, ffn.expert_size, ffn.shared_size, ffn.route_scale) == (5, 2, 24, 16, 1.3)
    assert ffn.activation.limit == 0.7 and ffn.shared_activation.limit == 0.9 and ffn.activation.alpha == 1.702
    assert spec.layers[0].branch_multiplier == 0.7 and spec.logit_softcap == 9.0 and spec.embedding_multiplier == 3.0
    assert spec.bigram.buckets == 53 and (spec.bigram.mul_prev, spec.bigram.mul_cur) == (13, 7)
    assert LutosunConfig.from_dict(json.loads(json.dumps(config.to_dict()))) == config
    names = {spec.stored_name(expect.name) for expect in DecoderModel.expected_tensors(spec)}
    assert {"embed", "bigram", "loop.step", "head", "final.norm", "final.norm.b", "l0.norm1", "l0.norm1.b", "l0.mix.dq",
            "l0.mix.dq.norm", "l0.mix.uq", "l0.mix.dkv", "l0.mix.dkv.norm", "l0.mix.uk", "l0.mix.uv", "l0.mix.o",
            "l0.mlp.router", "l0.mlp.correction", "l0.mlp.e0.gate", "l0.mlp.e4.down", "l0.mlp.shared.up",
            "l0.mlp.shared.sg"} <= names
    other = config_from_dict(lutosun_configs.LUT_B).to_model_spec()
    assert other.layers[1].ffn is None and other.layers[2].ffn.shared_size is None
    assert other.layers[0].mixers[0].spec.position.rotary_dim == 12
    assert config_from_dict(lutosun_configs.LUT_C).to_model_spec().bigram is None


@pytest.mark.parametrize("broken, text", [
    (dict(width=None), "width"), (dict(layers=[]), "layers"), (dict(norm={}), "norm.eps"),
    (dict(loop={"start": 2, "stop": 1, "times": 2}), "loop"),
    (dict(layers=[{"type": "conv", "mixer": {}}]), "type"),
    (dict(layers=[dict(lutosun_configs.LUT_A["layers"][0], mlp={"kind": "dense"})]), "mlp.kind")])
def test_a_broken_configuration_names_its_key(broken, text):
    raw = dict(lutosun_configs.LUT_A, **broken)
    if broken.get("width", 1) is None:
        del raw["width"]
    if "layers" in broken and "loop" not in broken:
        raw.pop("loop")
    with pytest.raises(ConfigError, match=text):
        config_from_dict(raw)


def test_sizes_that_no_kernel_takes_are_refused_at_load_with_their_key():
    raw = json.loads(json.dumps(lutosun_configs.LUT_A))
    raw["layers"][1]["mixer"].update(kv_rank=250, rot_dim=8)              # a cached row of 258 numbers
    with pytest.raises(ConfigError, match=r"kv_rank \+ rot_dim.*258"):
        Engine(config=raw, tensors=None, dtype="float32", device="cpu", check_device=False)
    raw = json.loads(json.dumps(lutosun_configs.LUT_A))
    raw["layers"][0]["mlp"]["router"]["experts"] = 1025
    with pytest.raises(ConfigError, match=r"router.experts.*1025"):
        Engine(config=raw, tensors=None, dtype="float32", device="cpu", check_device=False)


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_cut_and_token_by_token_match_the_plain_model(host_ops, tmp_path, name):
    engine, raw, tensors = engine_for(name, tmp_path)
    tokens = tokens_for(raw, 29, 3)
    expected = plain(raw, tensors, tokens)
    engine.add_request("whole")
    got = engine.step([Lane("whole", tokens, list(range(len(tokens))))])
    assert torch.allclose(got, expected, atol=2e-4, rtol=1e-4)
    engine.add_request("cut")
    rows, at = [], 0
    for size in (2, 7, 1, 1, 9, 2, 7):                        # portions down to two tokens, single tokens between
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


def test_the_token_before_a_portion_is_the_request_s_own(host_ops, tmp_path):
    """Two requests decode side by side; each one's bigram row comes from its own previous token, also after the
    slot of a finished request is used again."""
    engine, raw, tensors = engine_for("B", tmp_path, requests=2)
    first, second, third = tokens_for(raw, 6, 5), tokens_for(raw, 9, 6), tokens_for(raw, 4, 7)
    engine.add_request("x")
    engine.add_request("y")
    engine.step([Lane("x", first[:3]), Lane("y", second[:8])])
    rows = engine.step([Lane("x", first[3:4], [0]), Lane("y", second[8:], [0])])
    assert torch.allclose(rows[0], plain(raw, tensors, first[:4])[-1], atol=2e-4, rtol=1e-4)
    assert torch.allclose(rows[1], plain(raw, tensors, second)[-1], atol=2e-4, rtol=1e-4)
    engine.finish("y")
    engine.add_request("z")                                    # in y's slot: its first token takes the table's last row
    rows = engine.step([Lane("z", third, [0, 3]), Lane("x", first[4:], [1])])
    expected = plain(raw, tensors, third)
    assert torch.allclose(rows[:2], expected[[0, 3]], atol=2e-4, rtol=1e-4)
    assert torch.allclose(rows[2], plain(raw, tensors, first)[-1], atol=2e-4, rtol=1e-4)


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
