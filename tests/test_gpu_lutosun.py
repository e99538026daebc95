"""Lutosun on the GPU: every kernel against its plain PyTorch reference, every mechanism alone against the plain
implementation (tests/lutosun_plain.py), and whole models through the step function, the scheduler and the entry
points: whole prompts, portions down to two tokens, token-by-token decoding, unequal batches, pages and slots that
are used again, far keys, the first tokens of a sequence, long decoding, and sizes of many kinds."""
import numpy as np
import pytest
import torch

import lutosun_configs
import lutosun_plain
import ref_ops
import traces
from gates import bfloat16_close
from part_harness import DEV, PartHarness

pytestmark = pytest.mark.gpu

F32_GATE = 2e-4
DTYPES = [torch.float32, torch.bfloat16]


def rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def close(got, want, dtype, what=""):
    scale = max(1.0, float(want.abs().max()))
    gate = (F32_GATE if dtype == torch.float32 else 4e-2) * scale
    error = (got.double().cpu() - want.double().cpu()).abs()
    assert float(error.max()) <= gate, f"{what}: max error {float(error.max()):.3e}, gate {gate:.3e}"


def ops():
    from macllm_infer_amd.kernels import build, ops as module
    build.ensure_modules(["common", "gemm", "latent", "moe", "attention"])
    return module


def i32(values):
    return torch.tensor(values, dtype=torch.int32)


# ------------------------------------------------------------------ kernels against their references
@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("d, T", [(50, 7), (256, 33), (3000, 5), (9000, 2)])
def test_the_layer_norm_adds_weighted_branches_and_a_vector(out_dtype, d, T):
    h = rand(T, d, seed=1, scale=3.0) + 2.0                       # a mean far from zero: the variance needs its second pass
    branches = [(rand(T, d, seed=2).to(torch.bfloat16), 0.7), (rand(T, d, seed=3), 1.0), (rand(T, d, seed=4), -0.25)]
    vector, weight, bias = rand(d, seed=5), rand(d, seed=6) + 1.0, rand(d, seed=7)
    for count in (0, 1, 3):
        for rows in (None, i32([T - 1, 0, T // 2])):
            for with_vector in (False, True):
                want_h, want_out = h.clone(), torch.empty((T if rows is None else 3, d), dtype=out_dtype)
                ref_ops.add_layernorm(want_h, branches[:count], vector if with_vector else None, weight, bias, 1e-5,
                                      want_out, rows)
                got_h = h.clone().to(DEV)
                got_out = torch.empty(want_out.shape, dtype=out_dtype, device=DEV)
                ops().add_layernorm(got_h, [(tensor.to(DEV), factor) for tensor, factor in branches[:count]],
                                    vector.to(DEV) if with_vector else None, weight.to(DEV), bias.to(DEV), 1e-5, got_out,
                                    None if rows is None else rows.to(DEV))
                close(got_h, want_h, torch.float32, "stream")
                close(got_out, want_out.float(), out_dtype, "normed rows")


def test_the_stream_add_and_the_clamped_activation():
    h, rows, vector = rand(9, 70, seed=1), rand(9, 70, seed=2).to(torch.bfloat16), rand(70, seed=3)
    want = h.clone()
    ref_ops.stream_add(want, rows, 0.3, vector)
    got = h.clone().to(DEV)
    ops().stream_add(got, rows.to(DEV), 0.3, vector.to(DEV))
    close(got, want, torch.float32)
    for dtype in DTYPES:
        gate_up = (rand(11, 2 * 37, seed=4) * 2.0).to(dtype)
        want = torch.empty((11, 37), dtype=dtype)
        ref_ops.clamped_glu(gate_up, 0.8, 1.702, 1.0, want)
        got = torch.empty((11, 37), dtype=dtype, device=DEV)
        ops().clamped_glu(gate_up.to(DEV), 0.8, 1.702, 1.0, got)
        close(got.float(), want.float(), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_bigram_row_comes_from_the_request_s_previous_token(dtype):
    vocab, d, buckets = 90, 40, 23
    table, bigram = rand(vocab, d, seed=1).to(dtype), rand(buckets + 1, d, seed=2).to(dtype)
    # three lanes: a request's first tokens, a portion from the middle of another, one decoded token
    token_ids = i32([5, 17, 3, 80, 81, 2, 44])
    positions = i32([0, 1, 2, 9, 10, 11, 30])
    lane_of_token = i32([0, 0, 0, 1, 1, 1, 2])
    cu_seqlens, slot_ids = i32([0, 3, 6, 7]), i32([2, 0, 3])
    previous = i32([[61], [99], [7], [12], [0]])
    want, want_previous = torch.empty(7, d), previous.clone()
    ref_ops.embed_bigram(token_ids, table, 2.5, bigram, buckets, 37, 11, positions, lane_of_token, cu_seqlens, slot_ids,
                         want_previous, want)
    got, got_previous = torch.empty(7, d, device=DEV), previous.clone().to(DEV)
    ops().embed_bigram(token_ids.to(DEV), table.to(DEV), 2.5, bigram.to(DEV), buckets, 37, 11, positions.to(DEV),
                       lane_of_token.to(DEV), cu_seqlens.to(DEV), slot_ids.to(DEV), got_previous, got)
    close(got, want, torch.float32)
    assert got_previous.cpu().tolist() == want_previous.tolist() == [[2], [99], [3], [44], [0]]
    first = table.float()[5] * 2.5 + bigram.float()[buckets]                       # position 0: the last row
    middle = table.float()[80] * 2.5 + bigram.float()[(61 * 37 + 80 * 11) % buckets]  # the slot's token before it
    assert torch.allclose(got[0].cpu(), first, atol=1e-5) and torch.allclose(got[3].cpu(), middle, atol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("q_rank, kv_rank, rope_dim, rotary, interleaved", [
    (20, 24, 8, 8, True), (64, 40, 16, 12, True), (8, 56, 32, 32, False), (80, 64, 32, 32, True), (16, 16, 0, 0, True)])
def test_the_latent_norms_the_turn_and_the_cache_write(dtype, q_rank, kv_rank, rope_dim, rotary, interleaved):
    T, page, pages = 19, 8, 6
    down = rand(T, q_rank + kv_rank + rope_dim + 3, seed=1).to(dtype)[:, :q_rank + kv_rank + rope_dim + 3]
    q_norm, kv_norm = rand(q_rank, seed=2) + 1.0, rand(kv_rank, seed=3) + 1.0
    positions = torch.arange(100, 100 + T, dtype=torch.int32)
    inv_freq = torch.tensor([1000.0 ** (-2.0 * i / max(rotary, 1)) for i in range(rotary // 2)], dtype=torch.float32)
    cells = torch.randperm(page * pages, generator=torch.Generator().manual_seed(4))[:T].to(torch.int32)
    width = kv_rank + rope_dim
    storage = torch.zeros(pages, page * (width + kv_rank), dtype=dtype)
    def views(tensor):
        return (tensor[:, :page * width].unflatten(-1, (1, page, width)),
                tensor[:, page * width:].unflatten(-1, (1, kv_rank, page)))
    want_store, want_q = storage.clone(), torch.empty(T, q_rank, dtype=dtype)
    ref_ops.latent_prepare(down, q_rank, kv_rank, rope_dim, q_norm, kv_norm, 1e-5, positions, inv_freq if rotary else None,
                           rotary, interleaved, cells, *views(want_store), want_q)
    got_store, got_q = storage.clone().to(DEV), torch.empty(T, q_rank, dtype=dtype, device=DEV)
    ops().latent_prepare(down.to(DEV), q_rank, kv_rank, rope_dim, q_norm.to(DEV), kv_norm.to(DEV), 1e-5, positions.to(DEV),
                         inv_freq.to(DEV) if rotary else None, rotary, interleaved, cells.to(DEV), *views(got_store), got_q)
    close(got_q.float(), want_q.float(), dtype, "query latent")
    close(got_store.float(), want_store.float(), dtype, "cache cells")
    if rope_dim:
        heads = 3
        x = rand(T, heads * (10 + rope_dim) + 1, seed=5).to(dtype)
        want = torch.zeros(T, heads * (kv_rank + rope_dim), dtype=dtype)
        got = want.clone().to(DEV)
        args = (10, 10 + rope_dim, heads, rope_dim, positions, inv_freq if rotary else None, rotary, interleaved)
        ref_ops.rotate_heads(x, *args, want, kv_rank, kv_rank + rope_dim)
        ops().rotate_heads(x.to(DEV), args[0], args[1], heads, rope_dim, positions.to(DEV),
                           inv_freq.to(DEV) if rotary else None, rotary, interleaved, got, kv_rank, kv_rank + rope_dim)
        close(got.float(), want.float(), dtype, "turned heads")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T, heads, N, K, x_col, x_stride, out_col, out_stride", [
    (5, 3, 24, 16, 0, 24, 0, 32), (70, 2, 40, 32, 0, 48, 0, 56), (33, 4, 12, 24, 0, 24, 0, 12), (17, 1, 56, 24, 3, 27, 5, 61),
    (200, 5, 64, 48, 0, 80, 0, 96)])
def test_one_product_per_head(dtype, T, heads, N, K, x_col, x_stride, out_col, out_stride):
    x = rand(T, x_col + (heads - 1) * x_stride + K + 2, seed=1).to(dtype)
    weight = (rand(heads, N, K, seed=2) / K ** 0.5).to(dtype)
    want = torch.zeros(T, out_col + (heads - 1) * out_stride + N + 1, dtype=dtype)
    got = want.clone().to(DEV)
    ref_ops.head_linear(x, x_col, x_stride, weight, want, out_col, out_stride)
    ops().head_linear(x.to(DEV), x_col, x_stride, weight.to(DEV), got, out_col, out_stride)
    close(got.float(), want.float(), dtype)


@pytest.mark.parametrize("T, experts, top", [(1, 5, 2), (37, 12, 3), (300, 70, 8), (9, 3, 3), (64, 130, 1), (700, 6, 2)])
def test_the_router_and_the_grouping_of_rows_by_expert(T, experts, top):
    logits = rand(T, experts + 1, seed=1) * 2.0
    correction = rand(experts, seed=2) * 0.05
    want_ids, want_weights, want_gate = ref_ops.moe_route(logits, experts, top, correction, 1.5, 1e-20, True)
    got_ids, got_weights, got_gate = ops().moe_route(logits.to(DEV), experts, top, correction.to(DEV), 1.5, 1e-20, True)
    assert torch.equal(got_ids.cpu().sort(dim=1).values, want_ids.sort(dim=1).values)
    order = got_ids.cpu().long()
    scores = torch.softmax(logits[:, :experts], dim=-1)
    picked = torch.gather(scores, 1, order)
    close(got_weights, picked / picked.sum(dim=1, keepdim=True) * 1.5, torch.float32, "weights")
    close(got_gate, want_gate, torch.float32, "shared gate")
    plan = ops().moe_plan(got_ids, experts)
    source, place, tile_expert = plan.source.cpu(), plan.place.cpu().long(), plan.tile_expert.cpu()
    assert plan.pad == (64 if T * top >= 64 * experts else 16)
    assert plan.capacity % plan.pad == 0 and plan.capacity >= T * top
    flat = got_ids.cpu().reshape(-1)
    assert sorted(place.tolist()) == sorted(set(place.tolist()))                   # every choice has a place of its own
    for entry in range(T * top):
        assert int(source[place[entry]]) == entry // top
        assert int(tile_expert[place[entry] // plan.pad]) == int(flat[entry])      # in a tile of its expert
    assert int((source >= 0).sum()) == T * top
    used = tile_expert[tile_expert >= 0]
    assert torch.equal(used, used.sort().values)                                   # experts in turn, no tile shared


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T, experts, top, hidden, inner, pad", [
    (1, 4, 2, 32, 16, None), (45, 6, 3, 64, 40, None), (130, 9, 2, 48, 24, None), (7, 3, 1, 20, 12, None),
    (400, 5, 2, 72, 88, None), (300, 3, 2, 36, 20, None), (700, 3, 2, 64, 40, 128), (530, 2, 2, 136, 264, 128)])
def test_the_grouped_products_and_the_weighted_sum(dtype, T, experts, top, hidden, inner, pad):
    from macllm_infer_amd.config import ClampedGLUSpec
    glu = ClampedGLUSpec(limit=0.9)
    x = rand(T, hidden, seed=1).to(dtype)
    gate_up = (rand(experts, 2 * inner, hidden, seed=2) / hidden ** 0.5).to(dtype)
    down_w = (rand(experts, hidden, inner, seed=3) / inner ** 0.5).to(dtype)
    chosen = torch.stack([torch.randperm(experts, generator=torch.Generator().manual_seed(10 + t))[:top] for t in range(T)])
    weights = torch.rand(T, top, generator=torch.Generator().manual_seed(4))
    plan = ops().moe_plan(chosen.to(torch.int32).to(DEV), experts, pad)          # (pad: the widest tiles, by hand)
    host = ref_ops.MoePlan.__new__(ref_ops.MoePlan)
    host.pad, host.tokens, host.top_k, host.capacity = plan.pad, T, top, plan.capacity
    host.source, host.place, host.tile_expert = plan.source.cpu(), plan.place.cpu(), plan.tile_expert.cpu()
    want_inner = torch.zeros(plan.capacity, inner, dtype=dtype)
    ref_ops.moe_expert_gemm(x, host, gate_up, want_inner, True, glu)
    got_inner = torch.empty(plan.capacity, inner, dtype=dtype, device=DEV)
    ops().moe_expert_gemm(x.to(DEV), plan, gate_up.to(DEV), got_inner, gather=True, glu=glu)
    used = (host.tile_expert >= 0).repeat_interleave(plan.pad)          # tiles without an expert are not written
    close(got_inner.float().cpu()[used], want_inner.float()[used], dtype, "gate, up and the activation")
    want_down = torch.zeros(plan.capacity, hidden)
    ref_ops.moe_expert_gemm(want_inner, host, down_w, want_down, False, None)
    got_down = torch.empty(plan.capacity, hidden, device=DEV)
    ops().moe_expert_gemm(want_inner.to(DEV), plan, down_w.to(DEV), got_down, gather=False, glu=None)
    live = host.source >= 0
    close(got_down.cpu()[live], want_down[live], torch.float32 if dtype == torch.float32 else dtype, "down")
    shared, gate = rand(T, hidden, seed=5).to(dtype), torch.rand(T, generator=torch.Generator().manual_seed(6))
    want = torch.empty(T, hidden)
    ref_ops.moe_combine(want_down, host, weights, shared, gate, want)
    got = torch.empty(T, hidden, device=DEV)
    ops().moe_combine(want_down.to(DEV), plan, weights.to(DEV), shared.to(DEV), gate.to(DEV), got)
    close(got, want, torch.float32, "the weighted sum")


# ------------------------------------------------------------------ each mechanism alone against the plain model
def rounded(tensors, dtype):
    return {name: value.to(dtype).to(torch.float32) for name, value in tensors.items()}


def latent_tensors(hidden, spec, seed, sharpen=None):
    heads, dim, rope, rank = spec.num_heads, spec.head_dim, spec.rope_dim, spec.kv_rank
    shapes = {"dq.weight": (spec.q_rank, hidden), "uq.weight": (heads * (dim + rope), spec.q_rank),
              "dkv.weight": (rank + rope, hidden), "uk.weight": (heads * dim, rank), "uv.weight": (heads * spec.value_dim, rank),
              "o.weight": (hidden, heads * spec.value_dim)}
    tensors = {name: rand(*shape, seed=seed + index) / shape[1] ** 0.5 for index, (name, shape) in enumerate(shapes.items())}
    tensors["dq.norm.weight"] = rand(spec.q_rank, seed=seed + 10) * 0.1 + 1.0
    tensors["dkv.norm.weight"] = rand(rank, seed=seed + 11) * 0.1 + 1.0
    return tensors


def plain_names(tensors, prefix):
    out = {}
    for name, value in tensors.items():
        name = name[:-len(".weight")] if name.endswith(".weight") else name
        out[f"{prefix}.{name}"] = value
    return out


def latent_spec(heads, dim, rope, vdim, q_rank, kv_rank, rotary=None, base=10000.0, scale=None):
    from macllm_infer_amd.config import InterleavedRopeSpec, LatentAttentionSpec, NoPositionSpec
    position = InterleavedRopeSpec(theta=base, rotary_dim=rope if rotary is None else rotary) if rope else NoPositionSpec()
    return LatentAttentionSpec(num_heads=heads, head_dim=dim, rope_dim=rope, value_dim=vdim, q_rank=q_rank, kv_rank=kv_rank,
                               scale=(dim + rope) ** -0.5 if scale is None else scale, norm_eps=1e-5, position=position)


def mixer_table(spec, base=10000.0):
    table = {"heads": spec.num_heads, "dim": spec.head_dim, "rot_dim": spec.rope_dim, "vdim": spec.value_dim,
             "kv_rank": spec.kv_rank, "q_rank": spec.q_rank, "scale": spec.scale}
    if spec.rope_dim:
        table["rot"] = {"base": spec.position.theta, "dims": spec.position.rotary_dim}
    else:
        table["rot"] = {"base": 1.0, "dims": 0}
    return table


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


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, dim, rope, vdim, q_rank, kv_rank, rotary", [
    (3, 16, 8, 12, 20, 24, 8), (2, 32, 16, 32, 64, 40, 12), (1, 24, 32, 8, 8, 56, 32), (4, 64, 32, 64, 48, 96, 32),
    (5, 12, 0, 20, 16, 16, 0),
    # widths the matrix-core prompt kernel is built for (bfloat16): heads that fill a set of columns, leave a part
    # of one empty, and need a second pass
    (2, 16, 32, 16, 24, 32, 32), (5, 48, 32, 40, 72, 64, 32), (3, 32, 32, 64, 40, 128, 32), (9, 24, 64, 32, 32, 64, 64),
    (2, 64, 64, 32, 32, 128, 64), (3, 96, 64, 64, 64, 192, 64)])
def test_latent_attention_alone(dtype, heads, dim, rope, vdim, q_rank, kv_rank, rotary):
    hidden, T = 56, 170
    spec = latent_spec(heads, dim, rope, vdim, q_rank, kv_rank, rotary, base=300.0)
    tensors = rounded(latent_tensors(hidden, spec, 30), dtype)
    x = rand(T, hidden, seed=2).to(dtype).float()
    mixer = mixer_table(spec)
    if not rope:
        mixer["rot"] = {"base": 2.0, "dims": 0}
    want = lutosun_plain.latent_attention(x.double(), "p", {k: v.double() for k, v in plain_names(tensors, "p").items()},
                                          mixer, 1e-5, torch.float64).float()
    feed_every_way(lambda: PartHarness(spec, tensors, hidden, dtype, page_size=8, capacity=600), x, want, dtype,
                   beside=rand(40, hidden, seed=3))


def far_key_case(distance, T=700, hidden=32, matrix=False):
    """Inputs and weights of a latent attention layer in which the key ``distance`` tokens behind the last query
    stands out: the turned key part is a plain product of the token's row (no norm), so a row thirty times as large
    gives a key part thirty times as large, and its sign is chosen so that the last query's score for it is the
    largest by far.  Returns (spec, tensors, x, the plain rows, how much of the last row that key accounts for)."""
    if matrix:          # widths the matrix-core kernels are built for, weights and rows as bfloat16 holds them
        spec = latent_spec(3, 16, 32, 16, 16, 32, 32, base=50.0, scale=0.5)
        tensors = rounded(latent_tensors(hidden, spec, 50), torch.bfloat16)
    else:
        spec = latent_spec(2, 16, 8, 16, 16, 16, 8, base=50.0, scale=1.0)
        tensors = latent_tensors(hidden, spec, 50)
    names = {k: v.double() for k, v in plain_names(tensors, "p").items()}
    base = rand(T, hidden, seed=4) * 0.3
    if matrix:
        base = base.to(torch.bfloat16).float()
    target = T - 1 - distance
    best = None
    for sign in (1.0, -1.0):
        x = base.clone()
        x[target] = sign * 30.0 * base[target]
        want = lutosun_plain.latent_attention(x.double(), "p", names, mixer_table(spec), 1e-5, torch.float64).float()
        blind = base.clone()
        blind[target] = 0.0
        without = lutosun_plain.latent_attention(blind.double(), "p", names, mixer_table(spec), 1e-5, torch.float64).float()
        share = float((want[-1] - without[-1]).abs().max() / want[-1].abs().max())
        if best is None or share > best[-1]:
            best = (spec, tensors, x, want, share)
    return best


@pytest.mark.parametrize("matrix", [False, True])
@pytest.mark.parametrize("feed", ["whole", "decoded", "cut"])
@pytest.mark.parametrize("distance", [1, 15, 16, 17, 31, 32, 63, 64, 65, 299, 640])
def test_a_far_key_that_stands_out_is_found(distance, feed, matrix):
    """Among hundreds of keys one, ``distance`` tokens behind the last query, carries most of the last row's weight.
    With pages of 16 tokens that key lies next to the query, at page borders and far away; it is found from a prompt,
    from a decoded token, and from a portion cut right behind the key; by the general kernels in float32 and by the
    matrix-core kernels in bfloat16 (whose waves split the keys in runs of 32 and 64)."""
    spec, tensors, x, want, share = far_key_case(distance, matrix=matrix)
    assert share > 0.3, "the crafted key does not stand out"
    T, hidden = x.shape
    target = T - 1 - distance
    dtype = torch.bfloat16 if matrix else torch.float32
    harness = PartHarness(spec, tensors, hidden, dtype, page_size=16, capacity=720)
    if feed == "whole":
        out, = harness.run([("r", x)])
        got = out[-1]
    elif feed == "decoded":
        harness.run([("r", x[:T - 1])])
        got = harness.run([("r", x[T - 1:])])[0][-1]
    else:
        harness.run([("r", x[:target + 1])])
        got = harness.run([("r", x[target + 1:])])[0][-1]
    close(got, want[-1], dtype, f"distance {distance}")


def experts_spec(experts, top, inner, limit, scale, shared=None):
    from macllm_infer_amd.config import ClampedGLUSpec, RoutedExpertsSpec
    return RoutedExpertsSpec(num_experts=experts, top_k=top, expert_size=inner, activation=ClampedGLUSpec(limit=limit),
                             route_scale=scale, shared_size=None if shared is None else shared[0],
                             shared_activation=None if shared is None else ClampedGLUSpec(limit=shared[1]))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden, experts, top, inner, limit, scale, shared, T", [
    (48, 5, 2, 24, 0.7, 1.3, (16, 0.9), 37), (64, 7, 1, 16, 2.5, 1.0, (40, 1.5), 200), (40, 3, 3, 40, 1.0, 2.0, None, 9),
    (52, 9, 4, 20, 0.5, 1.0, (12, 0.4), 1)])
def test_the_mixture_of_experts_alone(dtype, hidden, experts, top, inner, limit, scale, shared, T):
    from macllm_infer_amd.kernels import build
    from macllm_infer_amd.parts import BuildContext, part_class
    spec = experts_spec(experts, top, inner, limit, scale, shared)
    cls = part_class(spec)
    build.ensure_modules(cls.kernel_modules)
    tensors = {"router.weight": rand(experts, hidden, seed=1) * 0.5, "correction": rand(experts, seed=2) * 0.05}
    for number in range(experts):
        tensors[f"e{number}.gate.weight"] = rand(inner, hidden, seed=10 + 3 * number) / hidden ** 0.5 * 2.0
        tensors[f"e{number}.up.weight"] = rand(inner, hidden, seed=11 + 3 * number) / hidden ** 0.5 * 2.0
        tensors[f"e{number}.down.weight"] = rand(hidden, inner, seed=12 + 3 * number) / inner ** 0.5
    if shared is not None:
        tensors.update({"shared.gate.weight": rand(shared[0], hidden, seed=70) / hidden ** 0.5 * 2.0,
                        "shared.up.weight": rand(shared[0], hidden, seed=71) / hidden ** 0.5 * 2.0,
                        "shared.down.weight": rand(hidden, shared[0], seed=72) / shared[0] ** 0.5,
                        "shared.sg.weight": rand(1, hidden, seed=73) / hidden ** 0.5})
    tensors = rounded(tensors, dtype)
    x = rand(T, hidden, seed=3).to(dtype).float()
    mlp = {"expert": {"ff": inner, "limit": limit}, "router": {"experts": experts, "top": top, "scale": scale}}
    if shared is not None:
        mlp["shared"] = {"ff": shared[0], "limit": shared[1]}
    plain = {k: v.double() for k, v in plain_names(tensors, "p").items()}
    want = lutosun_plain.mixture(x.double(), "p", plain, mlp, torch.float64).float()
    part = cls(spec, "p", {f"p.{name}": value for name, value in tensors.items()},
               BuildContext(hidden_size=hidden, dtype=dtype, device=torch.device(DEV), max_context=4096))
    got = part.forward(x.to(dtype).to(DEV))
    assert got.dtype == torch.float32
    if dtype == torch.bfloat16:
        # a token whose last choice is a near tie may take the other expert when its logits are rounded: compare
        # the rows whose choice is clear
        chosen, _ = lutosun_plain.route(x.double(), "p", plain, mlp["router"], torch.float64)
        scores = torch.softmax(x.double() @ plain["p.router"].T, dim=-1) + plain["p.correction"]
        ranked = scores.sort(dim=-1, descending=True).values
        clear = (ranked[:, top - 1] - ranked[:, top]) > 2e-2 if top < experts else torch.ones(T, dtype=torch.bool)
        assert T < 8 or int(clear.sum()) * 2 >= T, "most tokens' choices are clear"
        if bool(clear.any()):
            close(got.cpu()[clear], want[clear], dtype)
    else:
        close(got, want, dtype)


# ------------------------------------------------------------------ whole models through the engine
SEEDS = {"A": 11, "B": 12, "C": 13}


def model_dir(name, folder, dtype):
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    return lutosun_configs.make_model_dir(name, folder, seed=SEEDS[name], storage_dtype=storage)


def engine_for(name, folder, dtype, capacity=512, page=8, requests=4, **more):
    from macllm_infer_amd.engine import Engine
    raw, tensors = model_dir(name, folder, dtype)
    engine = Engine(str(folder), dtype=dtype, device=DEV, kv_cache_block_tokens=page, kv_cache_capacity_tokens=capacity,
                    max_active_sequences=requests, **more)
    return engine, raw, tensors


def tokens_for(raw, count, seed):
    return torch.randint(0, raw["vocab"], (count,), generator=torch.Generator().manual_seed(seed)).tolist()


CLEAR_MARGIN = 0.01


class Rows(torch.Tensor):
    """The plain model's logits with, per position, whether every choice of experts at that position was clear (no
    expert within ``CLEAR_MARGIN`` of the last chosen one, in any layer): 16-bit rounding may turn a choice that is
    not, and the logits of that position are then another model's.  Slices keep the flags."""

    @staticmethod
    def of(logits, clear):
        rows = logits.as_subclass(Rows)
        rows.clear = clear
        return rows

    def __getitem__(self, index):
        return Rows.of(torch.Tensor.__getitem__(self.as_subclass(torch.Tensor), index), self.clear[index])


def plain(raw, tensors, tokens):
    margins = []
    logits = lutosun_plain.forward(tokens, tensors, raw, margins=margins).to(torch.float32)
    clear = torch.ones(len(tokens), dtype=torch.bool)
    for margin in margins:
        clear &= margin > CLEAR_MARGIN
    return Rows.of(logits, clear)


def cat(pieces):
    return Rows.of(torch.cat([piece.as_subclass(torch.Tensor) for piece in pieces]),
                   torch.cat([piece.clear.reshape(-1) for piece in pieces]))


def same(got, want, dtype, what):
    clear = getattr(want, "clear", None)
    want = want.as_subclass(torch.Tensor) if isinstance(want, Rows) else want
    if dtype != "float32" and clear is not None:
        clear = clear.reshape(-1)
        assert want.shape[0] < 20 or int(clear.sum()) * 2 >= want.shape[0], f"{what}: most positions' choices are clear"
        if not bool(clear.any()):
            return
        got, want = got.float().cpu()[clear], want[clear]
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
    """One request whole; the same tokens in portions of many sizes in a slot and pages that were used before; its tail
    token by token; then unequal requests side by side, portions beside single tokens, one of them sitting out a step."""
    from macllm_infer_amd.engine import Lane
    engine, raw, tensors = engine_for(name, tmp_path, dtype, capacity=640)
    first, second, third = tokens_for(raw, 300, 1), tokens_for(raw, 41, 2), tokens_for(raw, 150, 3)
    want = {0: plain(raw, tensors, first), 1: plain(raw, tensors, second), 2: plain(raw, tensors, third)}
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
    rows = cat([want[0][19:20], want[1][:3], want[2][0:1], want[2][139:140], want[1][3:30], want[0][20:21],
                want[0][21:22], want[2][140:141], want[1][40:41], want[2][149:150], want[0][169:170]])
    same(got, rows, dtype, "mixed steps")
    engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_in_a_small_pool_and_the_first_tokens(tmp_path, dtype):
    """Three tokens of a prompt and 250 decoded one by one, through captured graphs; beside it requests of one and two
    tokens come and go in the same slot and pages (their first token takes the bigram table's last row, their second
    one their own first)."""
    from macllm_infer_amd.engine import Lane
    engine, raw, tensors = engine_for("A", tmp_path, dtype, capacity=272, page=8, requests=2)
    tokens = tokens_for(raw, 253, 5)
    want = plain(raw, tensors, tokens)
    short = tokens_for(raw, 2, 6)
    want_short = plain(raw, tensors, short)
    engine.add_request("long")
    outputs = [engine.step([Lane("long", tokens[:3], [0, 1, 2])])]
    for position in range(3, 253):
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
        same(torch.from_numpy(got[key]), plain(raw, tensors, tokens), dtype, key)


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
        want = list(prompt)
        for _ in range(8):
            want.append(int(plain(raw, tensors, want)[-1].argmax()))
        want = want[len(prompt):]
        if list(result.token_ids) != want:
            # a near tie between two tokens may fall the other way: then the plain model must show the tie
            place = next(i for i, (a, b) in enumerate(zip(result.token_ids, want)) if a != b)
            logits = plain(raw, tensors, prompt + want[:place])[-1]
            top = torch.topk(logits, 2).values
            assert float(top[0] - top[1]) < 1e-3, f"prompt of {len(prompt)}: token {place} differs without a tie"


def drawn_configuration(seed):
    """A configuration with every size and option drawn at random: odd widths and vocabularies, 1 to 7 heads, plain
    widths that are and are not whole 16-byte pieces, turned parts turned wholly and partly, layers in any number with
    and without a feed-forward, experts with and without a shared one, any loop, with and without bigram and cap."""
    rng = np.random.default_rng(seed)
    pick = lambda *values: values[int(rng.integers(len(values)))]
    width = int(pick(40, 56, 72, 100, 128, 136))
    count = int(rng.integers(1, 5))
    kinds = []
    for _ in range(int(rng.integers(1, 3))):
        rot_dim = int(pick(0, 4, 8, 16, 32))
        mixer = lutosun_configs.latent(int(rng.integers(1, 8)), int(pick(8, 12, 16, 24, 32, 40)), rot_dim,
                                       int(pick(8, 12, 16, 32, 48)), int(pick(8, 20, 32, 48)), int(pick(8, 16, 24, 32, 64)),
                                       rot_dims=None if rot_dim < 8 or rng.random() < 0.5 else rot_dim // 2,
                                       base=float(pick(100.0, 10000.0, 3e5)))
        experts = int(rng.integers(1, 10))
        mlp = None
        if rng.random() < 0.85:
            mlp = lutosun_configs.moe(experts, int(rng.integers(1, experts + 1)), int(pick(8, 12, 24, 40, 64)),
                                      float(pick(0.5, 1.0, 3.0)), float(pick(1.0, 1.5, 2.5)),
                                      shared=None if rng.random() < 0.3 else (int(pick(8, 20, 32, 72)), float(pick(0.5, 1.0, 7.0))))
        kinds.append(lutosun_configs.with_mlp(mixer, mlp))
    raw = {"architecture": "Lutosun", "width": width, "vocab": int(pick(61, 97, 256, 301)),
           "norm": {"eps": float(pick(1e-5, 1e-6))}, "residual_mult": float(pick(0.25, 0.6, 1.0, 1.4)),
           "embedding": {"scale": float(pick(1.0, 4.0, 8.0))},
           "layers": [kinds[int(rng.integers(len(kinds)))] for _ in range(count)]}
    if rng.random() < 0.7:
        raw["embedding"]["bigram"] = {"buckets": int(pick(1, 7, 64, 251)), "mul_prev": int(pick(1, 29, 1000003)),
                                      "mul_cur": int(pick(1, 19, 999983))}
    if rng.random() < 0.7:
        start = int(rng.integers(0, count))
        raw["loop"] = {"start": start, "stop": int(rng.integers(start + 1, count + 1)), "times": int(rng.integers(1, 4))}
    if rng.random() < 0.6:
        raw["logit_softcap"] = float(pick(5.0, 12.0, 30.0))
    return raw


DRAWN = [(seed, "float32") for seed in range(4100, 4116)] + [(seed, "bfloat16") for seed in range(4200, 4212)]


@pytest.mark.parametrize("seed, dtype", DRAWN)
def test_randomly_drawn_configurations_whole_cut_and_side_by_side(tmp_path, seed, dtype):
    from macllm_infer_amd.engine import Engine, Lane
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    raw, tensors = lutosun_configs.make_model_dir(drawn_configuration(seed), tmp_path, seed=seed, storage_dtype=storage)
    engine = Engine(str(tmp_path), dtype=dtype, device=DEV, kv_cache_block_tokens=int(np.random.default_rng(seed).choice([4, 8, 16])),
                    kv_cache_capacity_tokens=512, max_active_sequences=3)
    first, second = tokens_for(raw, 83, seed), tokens_for(raw, 21, seed + 1)
    want_first, want_second = plain(raw, tensors, first), plain(raw, tensors, second)
    engine.add_request("whole")
    same(engine.step([Lane("whole", first, list(range(83)))]), want_first, dtype, f"seed {seed}, whole")
    engine.finish("whole")
    engine.add_request("a")
    engine.add_request("b")
    rows_a, rows_b, at_a, at_b = [], [], 0, 0
    for size_a, size_b in ((5, 1), (2, 1), (40, 3), (1, 1), (1, 15), (34, 0)):
        lanes = [Lane("a", first[at_a:at_a + size_a], list(range(size_a)))]
        if size_b:
            lanes.append(Lane("b", second[at_b:at_b + size_b], list(range(size_b))))
        rows = engine.step(lanes)
        rows_a.append(rows[:size_a])
        rows_b.append(rows[size_a:])
        at_a, at_b = at_a + size_a, at_b + size_b
    same(torch.cat(rows_a), want_first, dtype, f"seed {seed}, portions beside another request")
    same(torch.cat(rows_b), want_second, dtype, f"seed {seed}, the other request")
    engine.cache.check()
