"""A plain, slow Lutosun: whole sequences, no cache, one function per mechanism, written from the design's
equations with the checkpoint's own tensor names.  It shares no code with the package and is the oracle of the
Lutosun tests.  Everything runs in the dtype of ``compute`` (float64 by default) on the CPU.

The design: a decoder whose embedding adds a hashed bigram row, whose first layers may run several times (each
pass with a cache of its own, the embedding output and a learned vector added before a pass), whose layers are
pre-norm with a layer norm (weight and bias), a latent attention mixer (queries and keys/values through
low-rank latents, one rotated key part shared by all heads, interleaved rotation) and a routed mixture of small
clamped-GLU experts beside a gated shared expert; a capped output.
"""
from __future__ import annotations

import torch


def gelu_free_glu(gate: torch.Tensor, up: torch.Tensor, limit: float) -> torch.Tensor:
    """y = g * sigmoid(1.702 g) * (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit)."""
    g = torch.clamp(gate, max=limit)
    u = torch.clamp(up, min=-limit, max=limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1.0)


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float) -> torch.Tensor:
    mean = x.mean(dim=-1, keepdim=True)
    centred = x - mean
    variance = (centred * centred).mean(dim=-1, keepdim=True)
    return centred / torch.sqrt(variance + eps) * weight + bias


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * weight


def rotate_interleaved(x: torch.Tensor, positions: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """x [T, ..., D]: the first ``dims`` dimensions in pairs (2i, 2i + 1) turned by position * base^(-2i/dims)."""
    out = x.clone()
    if dims == 0:
        return out
    half = dims // 2
    frequency = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=x.dtype)
    angle = positions.to(x.dtype).reshape(-1, *([1] * (x.dim() - 1))) * frequency
    cos, sin = torch.cos(angle), torch.sin(angle)
    even, odd = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = even * cos - odd * sin
    out[..., 1:dims:2] = odd * cos + even * sin
    return out


def embedding(tokens, tensors, config, compute) -> torch.Tensor:
    """embed[token] * scale + bigram[(previous * mul_prev + token * mul_cur) mod buckets]; the first token of a
    sequence takes the table's last row."""
    table = tensors["embed"].to(compute)
    ids = torch.tensor(tokens, dtype=torch.long)
    hashed = config["embedding"].get("bigram")
    if hashed is None:
        return table[ids] * config["embedding"]["scale"]
    bigram = tensors["bigram"].to(compute)
    buckets = hashed["buckets"]
    rows = []
    for index, token in enumerate(tokens):
        if index == 0:
            rows.append(buckets)
        else:
            rows.append((tokens[index - 1] * hashed["mul_prev"] + token * hashed["mul_cur"]) % buckets)
    return table[ids] * config["embedding"]["scale"] + bigram[torch.tensor(rows, dtype=torch.long)]


def latent_attention(h: torch.Tensor, prefix: str, tensors, mixer: dict, eps: float, compute) -> torch.Tensor:
    get = lambda name: tensors[f"{prefix}.{name}"].to(compute)
    tokens = h.shape[0]
    heads, dim, rot_dim, vdim, rank = mixer["heads"], mixer["dim"], mixer["rot_dim"], mixer["vdim"], mixer["kv_rank"]
    positions = torch.arange(tokens)
    rot = mixer.get("rot") or {"base": 1.0, "dims": 0}
    base, rot_dims = rot["base"], rot["dims"]
    query_latent = rms_norm(h @ get("dq").T, get("dq.norm"), eps)
    q = (query_latent @ get("uq").T).reshape(tokens, heads, dim + rot_dim)
    q_plain, q_turned = q[..., :dim], rotate_interleaved(q[..., dim:], positions, base, rot_dims)
    down = h @ get("dkv").T
    latent = rms_norm(down[:, :rank], get("dkv.norm"), eps)
    k_turned = rotate_interleaved(down[:, rank:], positions, base, rot_dims)          # [T, rot_dim], all heads
    k_plain = (latent @ get("uk").T).reshape(tokens, heads, dim)
    values = (latent @ get("uv").T).reshape(tokens, heads, vdim)
    scores = (torch.einsum("qhd,khd->hqk", q_plain, k_plain) + torch.einsum("qhd,kd->hqk", q_turned, k_turned))
    scores = scores * mixer["scale"]
    visible = positions.reshape(-1, 1) >= positions.reshape(1, -1)
    scores = scores.masked_fill(~visible, float("-inf"))
    weights = torch.softmax(scores, dim=-1)
    attended = torch.einsum("hqk,khd->qhd", weights, values).reshape(tokens, heads * vdim)
    return attended @ get("o").T


def expert(h: torch.Tensor, prefix: str, tensors, limit: float, compute) -> torch.Tensor:
    get = lambda name: tensors[f"{prefix}.{name}"].to(compute)
    return gelu_free_glu(h @ get("gate").T, h @ get("up").T, limit) @ get("down").T


def route(h: torch.Tensor, prefix: str, tensors, router: dict, compute):
    """(chosen experts [T, top], their weights [T, top])."""
    scores = torch.softmax(h @ tensors[f"{prefix}.router"].to(compute).T, dim=-1)
    choice = scores + tensors[f"{prefix}.correction"].to(compute)
    chosen = torch.topk(choice, router["top"], dim=-1).indices
    picked = torch.gather(scores, 1, chosen)
    weights = picked / (picked.sum(dim=-1, keepdim=True) + 1e-20) * router["scale"]
    return chosen, weights


def choice_margin(h: torch.Tensor, prefix: str, tensors, router: dict, compute) -> torch.Tensor:
    """Per token, how far the last chosen expert's choice score lies above the best one not chosen (infinite when
    every expert is chosen): a small margin is a choice that rounding may turn."""
    scores = torch.softmax(h @ tensors[f"{prefix}.router"].to(compute).T, dim=-1)
    ranked = (scores + tensors[f"{prefix}.correction"].to(compute)).sort(dim=-1, descending=True).values
    if router["top"] >= router["experts"]:
        return torch.full((h.shape[0],), float("inf"), dtype=compute)
    return ranked[:, router["top"] - 1] - ranked[:, router["top"]]


def mixture(h: torch.Tensor, prefix: str, tensors, mlp: dict, compute, margins=None) -> torch.Tensor:
    chosen, weights = route(h, prefix, tensors, mlp["router"], compute)
    if margins is not None:
        margins.append(choice_margin(h, prefix, tensors, mlp["router"], compute))
    out = torch.zeros_like(h)
    for number in range(mlp["router"]["experts"]):
        rows, places = torch.nonzero(chosen == number, as_tuple=True)
        if rows.numel():
            result = expert(h[rows], f"{prefix}.e{number}", tensors, mlp["expert"]["limit"], compute)
            out[rows] += result * weights[rows, places].reshape(-1, 1)
    if mlp.get("shared") is not None:
        gate = torch.sigmoid(h @ tensors[f"{prefix}.shared.sg"].to(compute).T)          # [T, 1]
        out = out + gate * expert(h, f"{prefix}.shared", tensors, mlp["shared"]["limit"], compute)
    return out


def run_order(config: dict):
    """[(layer, number of the pass or None, first of its pass)] in the order the layers run."""
    count = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(index, None, False) for index in range(count)]
    order = [(index, None, False) for index in range(loop["start"])]
    for turn in range(loop["times"]):
        for index in range(loop["start"], loop["stop"]):
            order.append((index, turn, index == loop["start"]))
    order += [(index, None, False) for index in range(loop["stop"], count)]
    return order


def forward(tokens, tensors, config, compute=torch.float64, streams=None, margins=None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  ``streams``: a list that receives the residual stream after
    every run of a layer.  ``margins``: a list that receives, for every run of a mixture of experts, each token's
    ``choice_margin``."""
    eps = config["norm"]["eps"]
    mult = config["residual_mult"]
    x = embedding(tokens, tensors, config, compute)
    embedded = x.clone()
    for index, turn, first in run_order(config):
        if first:
            if turn > 0:
                x = x + embedded
            x = x + tensors["loop.step"].to(compute)[turn]
        layer = config["layers"][index]
        prefix = f"l{index}"
        normed = layer_norm(x, tensors[f"{prefix}.norm1"].to(compute), tensors[f"{prefix}.norm1.b"].to(compute), eps)
        assert layer["type"] == "latent_attention"
        x = x + mult * latent_attention(normed, f"{prefix}.mix", tensors, layer["mixer"], eps, compute)
        if layer.get("mlp") is not None:
            normed = layer_norm(x, tensors[f"{prefix}.norm2"].to(compute), tensors[f"{prefix}.norm2.b"].to(compute), eps)
            x = x + mult * mixture(normed, f"{prefix}.mlp", tensors, layer["mlp"], compute, margins)
        if streams is not None:
            streams.append(x.clone())
    x = layer_norm(x, tensors["final.norm"].to(compute), tensors["final.norm.b"].to(compute), eps)
    logits = x @ tensors["head"].to(compute).T
    cap = config.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return logits
