"""A plain, slow Mukutar: whole sequences, no cache, one function per mechanism, in float64 on the CPU.

The oracle of the Mukutar tests.  It shares no code with the package: it reads a configuration as a plain
dictionary (the keys of the design's ``config.json``) and weights as a name -> tensor mapping under the
checkpoint's own names (``l<i>.mix.q``, ``l<i>.mix.q.b``, ``l<i>.norm1``, ...).

Notation: x [T, d] the residual stream of one sequence; positions 0 .. T-1.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def rms(values: torch.Tensor, eps: float) -> torch.Tensor:
    """values / sqrt(mean(values^2) + eps) over the last dimension."""
    return values / torch.sqrt((values * values).mean(dim=-1, keepdim=True) + eps)


def offset_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """Root-mean-square norm whose stored weight is the distance from one."""
    return rms(x, eps) * (1.0 + weight)


def poly_norm(z: torch.Tensor, coefficients: torch.Tensor, eps: float) -> torch.Tensor:
    """c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3 with N = division of a token's row by its root mean square."""
    c = coefficients.to(F)
    return c[0] * rms(z, eps) + c[1] * rms(z * z, eps) + c[2] * rms(z * z * z, eps) + c[3]


def dense_ffn(x: torch.Tensor, up: torch.Tensor, down: torch.Tensor, act: torch.Tensor, eps: float) -> torch.Tensor:
    return poly_norm(x @ up.T, act, eps) @ down.T


def rotate_half(x: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """x [T, H, D]: the first ``dims`` dimensions of every head turned by position * base^(-2i/dims), dimension i
    paired with i + dims/2."""
    T = x.shape[0]
    half = dims // 2
    frequency = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    angle = torch.arange(T, dtype=F)[:, None] * frequency[None, :]               # [T, half]
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    first, second = x[..., :half], x[..., half:dims]
    return torch.cat([first * cos - second * sin, second * cos + first * sin, x[..., dims:]], dim=-1)


def attention_mixer(h: torch.Tensor, w: dict, m: dict) -> torch.Tensor:
    """Windowed grouped-query attention whose scores lose r1 * ln(1 + r2 * distance) and whose softmax has one
    more term, exp(sink), in the denominator."""
    T = h.shape[0]
    H, G, D = m["heads"], m.get("kv_heads", m["heads"]), m["dim"]
    V = m.get("vdim", D)
    q = (h @ w["q"].T + w["q.b"]).view(T, H, D)
    k = (h @ w["k"].T + w["k.b"]).view(T, G, D)
    v = (h @ w["v"].T + w["v.b"]).view(T, G, V)
    window = (m.get("mask") or {}).get("size")
    out = torch.zeros(T, H, V, dtype=F)
    for head in range(H):
        group = head // (H // G)
        for i in range(T):
            first = 0 if window is None else max(0, i - window + 1)
            keys = torch.arange(first, i + 1)
            score = (k[first:i + 1, group] @ q[i, head]) * m["scale"]
            distance = (i - keys).to(F)
            score = score - w["r1"][head] * torch.log(1.0 + w["r2"][head] * distance)
            top = torch.maximum(score.max(), w["sink"][head])
            weight = torch.exp(score - top)
            denominator = weight.sum() + torch.exp(w["sink"][head] - top)
            out[i, head] = (weight / denominator) @ v[first:i + 1, group]
    return out.reshape(T, H * V) @ w["o"].T


def retention_mixer(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    """Linear attention with one fixed decay a head: S <- decay S + k v^T, o = S^T q; no softmax, no denominator."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    V = m.get("vdim", D)
    q = (h @ w["q"].T).view(T, H, D)
    k = (h @ w["k"].T).view(T, H, D)
    v = (h @ w["v"].T).view(T, H, V)
    rot = m.get("rot")
    if rot:
        q, k = rotate_half(q, rot["base"], rot["dims"]), rotate_half(k, rot["base"], rot["dims"])
    k = k * D ** -0.5
    out = torch.zeros(T, H, V, dtype=F)
    for head in range(H):
        state = torch.zeros(D, V, dtype=F)
        for t in range(T):
            state = m["decay"][head] * state + torch.outer(k[t, head], v[t, head])
            out[t, head] = state.T @ q[t, head]
    out = rms(out, eps).reshape(T, H * V)
    gate = h @ w["g"].T
    return (out * gate * torch.sigmoid(gate)) @ w["o"].T


def general_delta_mixer(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    """S <- diag(decay) S - (a u)(u^T S) + k v^T with u the unit key; both of the first terms read the old state."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    r = (h @ w["r"].T).view(T, H, D)
    k = (h @ w["k"].T).view(T, H, D)
    v = (h @ w["v"].T).view(T, H, D)
    decay = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(h @ w["w1"].T) @ w["w2"].T + w["w0"])).view(T, H, D)
    a = torch.sigmoid(h @ w["a"].T + w["a.b"]).view(T, H, D)
    unit = k / torch.sqrt((k * k).sum(dim=-1, keepdim=True) + 1e-6)
    out = torch.zeros(T, H, D, dtype=F)
    for head in range(H):
        state = torch.zeros(D, D, dtype=F)
        for t in range(T):
            u = unit[t, head]
            state = (decay[t, head][:, None] * state - torch.outer(a[t, head] * u, u @ state)
                     + torch.outer(k[t, head], v[t, head]))
            out[t, head] = state.T @ r[t, head]
    out = rms(out, eps).reshape(T, H * D) * w["norm"]
    return (out * torch.sigmoid(h @ w["g"].T)) @ w["o"].T


def forward(config: dict, tensors: dict, tokens, keep_layers: bool = False):
    """Logits [T, vocab] of one sequence (float64); with ``keep_layers`` also the stream after every layer."""
    weights = {name: tensor.to(F) for name, tensor in tensors.items()}
    eps = config["norm"]["eps"]
    x = weights["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    after = []
    for index, layer in enumerate(config["layers"]):
        prefix = f"l{index}."
        mix = {name[len(prefix) + 4:]: tensor for name, tensor in weights.items() if name.startswith(prefix + "mix.")}
        h = offset_norm(x, weights[prefix + "norm1"], eps)
        if layer["type"] == "attention":
            y = attention_mixer(h, mix, layer["mixer"])
        elif layer["type"] == "retention":
            y = retention_mixer(h, mix, layer["mixer"], eps)
        elif layer["type"] == "general_delta":
            y = general_delta_mixer(h, mix, layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + y * weights[prefix + "ls1"]
        if layer.get("mlp"):
            h = offset_norm(x, weights[prefix + "norm2"], eps)
            y = dense_ffn(h, weights[prefix + "mlp.up"], weights[prefix + "mlp.down"], weights[prefix + "mlp.act"], eps)
            x = x + y * weights[prefix + "ls2"]
        after.append(x)
    logits = offset_norm(x, weights["final.norm"], eps) @ weights["head"].T
    return (logits, torch.stack(after)) if keep_layers else logits


def greedy(config: dict, tensors: dict, prompt, count: int):
    tokens = list(prompt)
    for _ in range(count):
        tokens.append(int(forward(config, tensors, tokens)[-1].argmax()))
    return tokens[len(prompt):]
