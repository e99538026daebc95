"""Mukutar on the GPU: every mechanism alone against the plain implementation (tests/mukutar_plain.py), the scan
kernels against their reference, and whole models through the step function, the scheduler and the entry points:
whole prompts, portions down to two tokens, token-by-token decoding, unequal batches, pages and slots that are used
again, windows' edges, long decoding, and sizes of many kinds."""
import math

import numpy as np
import pytest
import torch

import mukutar_configs
import mukutar_plain
import ref_ops
import traces
from gates import bfloat16_close
from part_harness import DEV, PartHarness

pytestmark = pytest.mark.gpu

F32_GATE = 2e-4


def rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def stored(tensors):
    """A part's tensors under the names the plain implementation reads: no ``_proj``, no ``.weight``, ``.b``."""
    out = {}
    for name, value in tensors.items():
        name = name.replace("_proj.", ".")
        name = name[:-len(".weight")] if name.endswith(".weight") else name
        name = name[:-len(".bias")] + ".b" if name.endswith(".bias") else name
        out[name] = value.to(torch.float64)
    return out


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


# ------------------------------------------------------------------ the scan kernels against their reference
def scan_case(delta, H, dk, dv, lengths, dtype, rotary, seed):
    from macllm_infer_amd.kernels import ops
    T = sum(lengths)
    lanes = len(lengths)
    generator = torch.Generator().manual_seed(seed)
    width = 1 + 3 * H * dk + H * dv + 3
    u = (torch.randn(T, width, generator=generator) * 0.7).to(dtype)
    state = torch.randn(lanes + 2, H, dv, dk, generator=generator) * 0.3
    cu = torch.tensor([0] + list(np.cumsum(lengths)), dtype=torch.int32)
    slots = torch.randperm(lanes + 2, generator=generator)[:lanes].to(torch.int32)
    starts = torch.randint(0, 5000, (lanes,), generator=generator)
    positions = torch.cat([torch.arange(length) + starts[lane] for lane, length in enumerate(lengths)]).to(torch.int32)
    common = dict(q_col=1, k_col=1 + H * dk, v_col=1 + 2 * H * dk, num_heads=H, key_dim=dk, value_dim=dv,
                  max_query_len=max(lengths))
    if delta:
        common.update(removal_col=1 + 2 * H * dk + H * dv, decay_logits=torch.randn(T, H * dk, generator=generator),
                      decay_bias=torch.randn(H * dk, generator=generator), decay_floor=math.exp(-0.5), key_eps=1e-6)
    else:
        common.update(head_decay=torch.tensor([1.0 - 2.0 ** (-2 - head) for head in range(H)]), key_scale=dk ** -0.5)
        if rotary:
            common.update(positions=positions, rotary_dim=rotary,
                          inv_freq=torch.tensor([1e4 ** (-2.0 * i / rotary) for i in range(rotary // 2)]))
    want_out, want_state = torch.zeros(T, H * dv), state.clone()
    ref_ops.linear_state_scan(u, state=want_state, cu_seqlens=cu, slot_ids=slots, out=want_out, **common)
    on = lambda value: value.to(DEV) if isinstance(value, torch.Tensor) else value
    device = {name: on(value) for name, value in common.items()}
    results = []
    for chunked in (False, True):
        got_out = torch.zeros(T, H * dv, device=DEV)
        got_state = state.clone().to(DEV)
        chunks = ops.SsdChunks(lengths, 16, DEV) if chunked else None       # short chunks: many of them, ragged ends
        ops.linear_state_scan(u.to(DEV), state=got_state, cu_seqlens=cu.to(DEV), slot_ids=slots.to(DEV), out=got_out,
                              chunks=chunks, **device)
        torch.cuda.synchronize()
        results.append((got_out.cpu(), got_state.cpu()))
    return want_out, want_state, results


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("delta, H, dk, dv, rotary", [
    (False, 3, 16, 16, 16), (False, 2, 24, 40, 12), (False, 1, 64, 128, 0), (False, 2, 40, 8, 40),
    (False, 2, 32, 10, 8), (False, 1, 128, 6, 0), (False, 1, 100, 262, 100),
    (True, 2, 16, 16, 0), (True, 3, 24, 24, 0), (True, 1, 64, 64, 0), (True, 2, 72, 72, 0), (True, 1, 130, 130, 0),
    (True, 2, 20, 20, 0), (True, 1, 6, 6, 0)])
def test_scans_walk_lanes_and_chunks_alike(dtype, delta, H, dk, dv, rotary):
    """Lanes of 1, 2, 15, 16, 17 and 70 tokens from states that are not empty, in slots out of order: the walk from
    end to end and the three passes over chunks of 16 tokens against the reference, outputs and states."""
    want_out, want_state, results = scan_case(delta, H, dk, dv, [70, 1, 17, 2, 16, 15, 33], dtype, rotary, seed=dk + dv)
    for name, (got_out, got_state) in zip(("walk", "chunks"), results):
        scale = max(1.0, float(want_out.abs().max()))
        assert float((got_out - want_out).abs().max()) <= 2e-4 * scale, name
        assert float((got_state - want_state).abs().max()) <= 2e-4 * max(1.0, float(want_state.abs().max())), name


# ------------------------------------------------------------------ the parts alone
def attention_tensors(hidden, H, G, D, V, seed):
    return {"q_proj.weight": rand(H * D, hidden, seed=seed + 1, scale=hidden ** -0.5),
            "k_proj.weight": rand(G * D, hidden, seed=seed + 2, scale=hidden ** -0.5),
            "v_proj.weight": rand(G * V, hidden, seed=seed + 3, scale=hidden ** -0.5),
            "o_proj.weight": rand(hidden, H * V, seed=seed + 4, scale=(H * V) ** -0.5),
            "q_proj.bias": rand(H * D, seed=seed + 5, scale=0.2), "k_proj.bias": rand(G * D, seed=seed + 6, scale=0.2),
            "v_proj.bias": rand(G * V, seed=seed + 7, scale=0.2), "sink": rand(H, seed=seed + 8),
            "r1": rand(H, seed=seed + 9).abs() + 0.05, "r2": rand(H, seed=seed + 10).abs() + 0.05}


def attention_spec(H, G, D, V, window, scale):
    from macllm_infer_amd.config import AttentionSpec, LogDistanceBiasSpec
    return AttentionSpec(num_heads=H, num_kv_heads=G, head_dim=D, scale=scale, position=LogDistanceBiasSpec(num_heads=H),
                         window=window, qkv_bias=True, out_bias=False, value_dim=V, sink=True)


def rounded(tensors, dtype):
    return {name: value.to(dtype).float() if value.dim() >= 2 else value for name, value in tensors.items()}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, G, D, V, window", [(6, 2, 16, 16, 11), (3, 3, 24, 40, 64), (4, 1, 64, 64, 33),
                                                (2, 2, 128, 128, 200), (5, 1, 8, 24, 1)])
def test_attention_with_a_distance_bias_a_window_and_a_sink_alone(dtype, H, G, D, V, window):
    hidden = 40
    tensors = rounded(attention_tensors(hidden, H, G, D, V, seed=window), dtype)
    mixer = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 0.9 / math.sqrt(D), "mask": {"size": window}}
    x = rand(230, hidden, seed=3).to(dtype).float()
    want = mukutar_plain.attention_mixer(x.double(), stored(tensors), mixer)
    make = lambda: PartHarness(attention_spec(H, G, D, V, window, mixer["scale"]), tensors, hidden, dtype, page_size=8)
    feed_every_way(make, x, want, dtype, beside=rand(64, hidden, seed=4))


def crafted_attention(window, distance, length):
    """One query head whose last token's query and the key ``distance`` tokens before it stand out (score 36 against
    less than 1 for every other key, the query's own included: queries, keys and values read columns of their own
    of the input), values that say which token they came from.  Returns the part's tensors, its inputs, the two
    positions and the input's width."""
    hidden, D, V = 24, 8, 8
    block = lambda first: torch.cat([torch.zeros(D, first), torch.eye(D), torch.zeros(D, hidden - first - D)], dim=1)
    tensors = {"q_proj.weight": block(8), "k_proj.weight": block(0), "v_proj.weight": block(16),
               "o_proj.weight": torch.cat([torch.eye(V), torch.zeros(hidden - V, V)], dim=0),
               "q_proj.bias": torch.zeros(D), "k_proj.bias": torch.zeros(D), "v_proj.bias": torch.zeros(V),
               "sink": torch.tensor([-2.0]), "r1": torch.tensor([0.05]), "r2": torch.tensor([0.5])}
    x = rand(length, hidden, seed=distance, scale=0.1)
    query, key = length - 1, length - 1 - distance
    x[query, 8] = 6.0                              # the query's first dim
    x[key, 0] = 6.0                                # the key's first dim
    x[key, 16:] = 5.0                              # the value that shows whether the key was seen
    return tensors, x, query, key, hidden


@pytest.mark.parametrize("feed", ["whole", "decoded", "cut"])
@pytest.mark.parametrize("window, distance", [(21, 20), (21, 21), (16, 15), (16, 16), (300, 299), (300, 300), (24, 1)])
def test_a_key_just_inside_the_window_is_seen_and_the_next_one_is_not(window, distance, feed):
    """A key that decides the output when it is seen: at the window's last place, and one beyond; in a prompt, in
    decoding, and with the portion cut between the key and the query; pages of 8 tokens, so the windows' edges fall
    on page borders (16, 24) and inside pages (21, 300)."""
    length = distance + 27
    tensors, x, query, key, hidden = crafted_attention(window, distance, length)
    mixer = {"heads": 1, "kv_heads": 1, "dim": 8, "vdim": 8, "scale": 1.0, "mask": {"size": window}}
    want = mukutar_plain.attention_mixer(x.double(), stored(tensors), mixer)
    seen = distance < window
    assert (float(want[query, :8].min()) > 4.0) == seen          # the plain model itself shows the edge
    harness = PartHarness(attention_spec(1, 1, 8, 8, window, 1.0), tensors, hidden, torch.float32, page_size=8,
                          capacity=1024)
    if feed == "whole":
        got = harness.run([("r", x)])[0]
    elif feed == "decoded":
        got = torch.cat([harness.run([("r", x[:key + 1])])[0]] +
                        [harness.run([("r", x[t:t + 1])])[0] for t in range(key + 1, length)])
    else:
        middle = key + max(1, distance // 2)
        got = torch.cat([harness.run([("r", x[:middle])])[0], harness.run([("r", x[middle:query - 1])])[0]
                         if query - 1 > middle else x.new_zeros(0, hidden),
                         harness.run([("r", x[max(middle, query - 1):])])[0]])
    close(got, want, torch.float32, f"window {window}, distance {distance}, {feed}")
    assert (float(got[query, :8].min()) > 4.0) == seen


def test_a_large_sink_takes_the_weight_from_every_key():
    H, G, D, V, hidden = 2, 1, 16, 16, 24
    tensors = attention_tensors(hidden, H, G, D, V, seed=5)
    tensors["sink"] = torch.tensor([9.0, -9.0])
    mixer = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 0.25, "mask": {"size": 12}}
    x = rand(40, hidden, seed=6)
    want = mukutar_plain.attention_mixer(x.double(), stored(tensors), mixer)
    without = mukutar_plain.attention_mixer(x.double(), stored(dict(tensors, sink=torch.tensor([-9.0, -9.0]))), mixer)
    assert float((want - without).abs().max()) > 0.05            # the sink shows in the plain model
    harness = PartHarness(attention_spec(H, G, D, V, 12, 0.25), tensors, hidden, torch.float32, page_size=4)
    got = torch.cat([harness.run([("r", x[:25])])[0]] + [harness.run([("r", x[t:t + 1])])[0] for t in range(25, 40)])
    close(got, want, torch.float32, "sink")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, D, V, rot", [(3, 16, 16, 16), (2, 24, 40, 12), (1, 64, 128, 64), (2, 40, 8, 0)])
def test_retention_alone(dtype, H, D, V, rot):
    from macllm_infer_amd.config import NoPositionSpec, RetentionSpec, RopeSpec
    hidden = 48
    decay = [1.0 - 2.0 ** (-3 - 2 * head) for head in range(H)]
    tensors = rounded({"q.weight": rand(H * D, hidden, seed=1, scale=hidden ** -0.5),
                       "k.weight": rand(H * D, hidden, seed=2, scale=hidden ** -0.5),
                       "v.weight": rand(H * V, hidden, seed=3, scale=hidden ** -0.5),
                       "g.weight": rand(H * V, hidden, seed=4, scale=hidden ** -0.5),
                       "o.weight": rand(hidden, H * V, seed=5, scale=(H * V) ** -0.5)}, dtype)
    mixer = {"heads": H, "dim": D, "vdim": V, "decay": decay}
    if rot:
        mixer["rot"] = {"base": 700.0, "dims": rot}
    spec = RetentionSpec(num_heads=H, key_dim=D, value_dim=V, decay=tuple(decay), key_scale=D ** -0.5, norm_eps=2e-6,
                         position=RopeSpec(theta=700.0, rotary_dim=rot) if rot else NoPositionSpec())
    x = rand(300, hidden, seed=7).to(dtype).float()
    want = mukutar_plain.retention_mixer(x.double(), stored(tensors), mixer, 2e-6)
    feed_every_way(lambda: PartHarness(spec, tensors, hidden, dtype, page_size=8), x, want, dtype,
                   beside=rand(64, hidden, seed=8))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, D, rank", [(2, 16, 8), (3, 24, 5), (1, 64, 16), (2, 72, 1)])
def test_the_generalized_delta_rule_alone(dtype, H, D, rank):
    from macllm_infer_amd.config import GeneralDeltaSpec
    hidden, inner = 48, H * D
    tensors = {name: rand(inner, hidden, seed=index, scale=hidden ** -0.5)
               for index, name in enumerate(["r.weight", "k.weight", "v.weight", "g.weight", "a.weight"])}
    tensors.update({"a.bias": rand(inner, seed=11, scale=0.5), "w1.weight": rand(rank, hidden, seed=12, scale=hidden ** -0.5),
                    "w2.weight": rand(inner, rank, seed=13, scale=2.0 * rank ** -0.5), "w0": rand(inner, seed=14),
                    "norm.weight": 1.0 + rand(inner, seed=15, scale=0.2),
                    "o.weight": rand(hidden, inner, seed=16, scale=inner ** -0.5)})
    tensors = rounded(tensors, dtype)
    spec = GeneralDeltaSpec(num_heads=H, head_dim=D, norm_eps=3e-6, decay_rank=rank)
    x = rand(300, hidden, seed=17).to(dtype).float()
    want = mukutar_plain.general_delta_mixer(x.double(), stored(tensors), {"heads": H, "dim": D}, 3e-6)
    feed_every_way(lambda: PartHarness(spec, tensors, hidden, dtype, page_size=8), x, want, dtype,
                   beside=rand(64, hidden, seed=18))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden, inner, T", [(56, 136, 37), (2560, 4104, 9), (8200, 2056, 3)])
def test_the_polynorm_feed_forward_the_offset_norm_and_a_scaled_branch_alone(dtype, hidden, inner, T):
    """Narrow rows, rows wide enough for the kernels' large workgroups, and rows that no longer fit a thread's
    registers."""
    from macllm_infer_amd.config import PolyNormFFNSpec, RmsNormSpec
    from macllm_infer_amd.kernels import build
    from macllm_infer_amd.parts import BuildContext, part_class
    from macllm_infer_amd.parts.base import Residual, ScaledBranch
    context = BuildContext(hidden_size=hidden, dtype=dtype, device=torch.device(DEV), max_context=64)
    build.ensure_modules(("common", "gemm"))
    tensors = rounded({"p.up.weight": rand(inner, hidden, seed=1, scale=hidden ** -0.5),
                       "p.down.weight": rand(hidden, inner, seed=2, scale=inner ** -0.5),
                       "p.act": torch.tensor([0.7, -0.4, 0.25, 0.1])}, dtype)
    spec = PolyNormFFNSpec(intermediate_size=inner, eps=1e-5)
    ffn = part_class(spec)(spec, "p", tensors, context)
    x = rand(T, hidden, seed=3).to(dtype)
    got = ffn.forward(x.to(DEV)).float().cpu()
    want = mukutar_plain.dense_ffn(x.double(), tensors["p.up.weight"].double(), tensors["p.down.weight"].double(),
                                   tensors["p.act"].double(), 1e-5)
    close(got, want, dtype, "feed-forward")
    # h += scale * branch, then the norm with a weight stored around zero
    norm_spec = RmsNormSpec(eps=1e-5, weight_offset=1.0)
    weight = rand(hidden, seed=4, scale=0.2)
    norm = part_class(norm_spec)(norm_spec, "n", {"n.weight": weight}, context)
    h, branch, scale = rand(T, hidden, seed=5), rand(T, hidden, seed=6).to(dtype), 1.0 + rand(hidden, seed=7, scale=0.3)
    residual = Residual(h.clone().to(DEV))
    residual.pending = [ScaledBranch(branch.to(DEV), scale.to(DEV))]
    normed = norm.forward(residual).float().cpu()
    summed = h.double() + branch.double() * scale.double()
    assert float((residual.h.cpu().double() - summed).abs().max()) < 1e-5       # the stream itself stays in float32
    close(normed, mukutar_plain.offset_norm(summed, weight.double(), 1e-5), dtype, "norm")


# ------------------------------------------------------------------ whole models through the step function
MUK_C = {"architecture": "Mukutar", "width": 96, "vocab": 70, "norm": {"eps": 1e-6}, "layers": [
    mukutar_configs.with_mlp(mukutar_configs.retention(2, 64, 128, 32, base=1e6), 120),
    mukutar_configs.with_mlp(mukutar_configs.general_delta(1, 64, 4), 200),
    mukutar_configs.with_mlp(mukutar_configs.attention(4, 4, 64, 64, 40), 64),
    mukutar_configs.with_mlp(mukutar_configs.general_delta(2, 40, 3), None),
    mukutar_configs.with_mlp(mukutar_configs.attention(2, 1, 24, 8, 150), 96),
    mukutar_configs.with_mlp(mukutar_configs.attention(6, 2, 128, 128, 7), 96)]}
SEEDS = {"A": 11, "B": 12, "C": 13}


def model_dir(name, folder, dtype):
    raw = MUK_C if name == "C" else name
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    return mukutar_configs.make_model_dir(raw, folder, seed=SEEDS[name], dtype=storage)


def engine_for(name, folder, dtype, capacity=512, page=8, requests=4, **more):
    from macllm_infer_amd.engine import Engine
    raw, tensors = model_dir(name, folder, dtype)
    engine = Engine(str(folder), dtype=dtype, device=DEV, kv_cache_block_tokens=page, kv_cache_capacity_tokens=capacity,
                    max_active_sequences=requests, **more)
    return engine, raw, tensors


def tokens_for(raw, count, seed):
    return torch.randint(0, raw["vocab"], (count,), generator=torch.Generator().manual_seed(seed)).tolist()


def same(got, want, dtype, what):
    got, want = got.float().cpu().numpy(), want.float().numpy()
    if dtype == "float32":
        error = np.abs(got - want).max(axis=-1)
        gate = F32_GATE * max(1.0, float(np.abs(want).max()))
        assert error.max() <= gate, f"{what}: max error {error.max():.3e} at row {int(np.argmax(error))}, gate {gate:.3e}"
    else:
        assert bfloat16_close(got, want), f"{what}: max error {np.abs(got - want).max():.3e} of scale {np.abs(want).max():.2f}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_cut_decoded_and_mixed_steps_match_the_plain_model(tmp_path, name, dtype):
    """One request whole (long enough for the scans to run in chunks); the same tokens in portions of many sizes in
    a slot and pages that were used before; its tail token by token; then unequal requests side by side, portions
    beside single tokens, one of them sitting out a step."""
    from macllm_infer_amd.engine import Lane
    engine, raw, tensors = engine_for(name, tmp_path, dtype, capacity=640)
    first, second, third = tokens_for(raw, 300, 1), tokens_for(raw, 41, 2), tokens_for(raw, 150, 3)
    want = {0: mukutar_plain.forward(raw, tensors, first), 1: mukutar_plain.forward(raw, tensors, second),
            2: mukutar_plain.forward(raw, tensors, third)}
    engine.add_request("whole")
    same(engine.step([Lane("whole", first, list(range(300)))]), want[0], dtype, "whole")
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
    same(torch.cat(outputs), want[0], dtype, "portions and single tokens")
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
    same(got, rows, dtype, "mixed steps")
    engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_in_a_small_pool_and_the_first_tokens(tmp_path, dtype):
    """Three tokens of a prompt and 330 decoded one by one: windows of 40, 150 and 7 tokens pass over decoded
    tokens, pages of passed tokens come back to a pool that holds 192, and the states are carried through hundreds
    of steps; beside it requests of one and two tokens come and go in the same slots."""
    from macllm_infer_amd.engine import Lane
    engine, raw, tensors = engine_for("C", tmp_path, dtype, capacity=192, page=8, requests=2)
    tokens = tokens_for(raw, 333, 5)
    want = mukutar_plain.forward(raw, tensors, tokens)
    short = tokens_for(raw, 2, 6)
    want_short = mukutar_plain.forward(raw, tensors, short)
    engine.add_request("long")
    outputs = [engine.step([Lane("long", tokens[:3], [0, 1, 2])])]
    for position in range(3, 333):
        if position % 50 == 10:
            engine.add_request("short")
            both = engine.step([Lane("short", short[:1], [0]), Lane("long", tokens[position:position + 1], [0])])
            same(both[:1], want_short[:1], dtype, "a sequence's first token")
            outputs.append(both[1:])
        elif position % 50 == 11:
            both = engine.step([Lane("long", tokens[position:position + 1], [0]), Lane("short", short[1:], [0])])
            same(both[1:], want_short[1:], dtype, "a sequence's second token")
            outputs.append(both[:1])
            engine.finish("short")
        else:
            outputs.append(engine.step([Lane("long", tokens[position:position + 1], [0])]))
    same(torch.cat(outputs), want, dtype, "long decoding")
    engine.finish("long")
    engine.cache.check()


@pytest.mark.parametrize("name, dtype", [("A", "float32"), ("B", "bfloat16"), ("C", "float32"), ("C", "bfloat16")])
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
        same(torch.from_numpy(got[key]), mukutar_plain.forward(raw, tensors, tokens), dtype, key)


@pytest.mark.parametrize("name", ["B", "C"])
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
        want = mukutar_plain.greedy(raw, tensors, prompt, 8)
        if list(result.token_ids) != want:
            # a near tie between two tokens may fall the other way: then the plain model must show the tie
            place = next(i for i, (a, b) in enumerate(zip(result.token_ids, want)) if a != b)
            logits = mukutar_plain.forward(raw, tensors, prompt + want[:place])[-1]
            top = torch.topk(logits, 2).values
            assert float(top[0] - top[1]) < 1e-3, f"prompt of {len(prompt)}: token {place} differs without a tie"
