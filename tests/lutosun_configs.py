"""Small Lutosun configurations of the tests, and helpers that write them as model folders.

They differ from each other in every size: width, vocabulary, heads, plain / turned / value widths, latent ranks,
turned dimensions (the whole turned part, and a part of it), experts and how many a token uses, a layer without a
feed-forward, a feed-forward without a shared expert, the looped layers (the middle ones three times, the first one
once, none), branch multipliers (one of them 1), the bigram table (one model without) and the cap on the logits.
"""
import json
import os

import torch

from macllm_infer_amd.config import LutosunConfig
from macllm_infer_amd.weights.random_init import write_random_model
from macllm_infer_amd.weights.safetensors_io import SafetensorsFile


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, rot_dims=None, base=10000.0, scale=None):
    mixer = {"dim": dim, "heads": heads, "kv_rank": kv_rank, "q_rank": q_rank, "rot_dim": rot_dim,
             "scale": (dim + rot_dim) ** -0.5 if scale is None else scale, "vdim": vdim}
    if rot_dim:
        mixer["rot"] = {"base": base, "dims": rot_dim if rot_dims is None else rot_dims}
    return {"type": "latent_attention", "mixer": mixer}


def moe(experts, top, ff, limit, scale=1.0, shared=None):
    mlp = {"expert": {"ff": ff, "limit": limit}, "kind": "moe", "router": {"experts": experts, "scale": scale, "top": top}}
    if shared is not None:
        mlp["shared"] = {"ff": shared[0], "limit": shared[1]}
    return mlp


def with_mlp(layer, mlp):
    return dict(layer, mlp=mlp)


LUT_A = {
    "architecture": "Lutosun", "width": 48, "vocab": 97, "norm": {"eps": 1e-5}, "residual_mult": 0.7,
    "embedding": {"scale": 3.0, "bigram": {"buckets": 53, "mul_cur": 7, "mul_prev": 13}},
    "logit_softcap": 9.0, "loop": {"start": 1, "stop": 3, "times": 3},
    "layers": [with_mlp(latent(3, 16, 8, 12, 20, 24), moe(5, 2, 24, 0.7, 1.3, shared=(16, 0.9))),
               with_mlp(latent(3, 16, 8, 12, 20, 24), moe(5, 2, 24, 0.7, 1.3, shared=(16, 0.9))),
               with_mlp(latent(3, 16, 8, 12, 20, 24), moe(5, 2, 24, 0.7, 1.3, shared=(16, 0.9))),
               with_mlp(latent(3, 16, 8, 12, 20, 24), moe(5, 2, 24, 0.7, 1.3, shared=(16, 0.9)))],
}

LUT_B = {
    "architecture": "Lutosun", "width": 64, "vocab": 131, "norm": {"eps": 1e-6}, "residual_mult": 1.0,
    "embedding": {"scale": 1.0, "bigram": {"buckets": 17, "mul_cur": 1, "mul_prev": 1}},
    "loop": {"start": 0, "stop": 1, "times": 1},
    "layers": [with_mlp(latent(2, 32, 16, 32, 64, 40, rot_dims=12, base=500.0), moe(7, 1, 16, 2.5, shared=(40, 1.5))),
               with_mlp(latent(4, 8, 4, 24, 16, 16, base=100.0), None),
               with_mlp(latent(1, 24, 32, 8, 8, 56, rot_dims=32), moe(3, 3, 40, 1.0, 2.0)),
               with_mlp(latent(2, 32, 16, 32, 64, 40, rot_dims=12, base=500.0), moe(7, 4, 16, 2.5, shared=(8, 0.5)))],
}

# sizes the matrix-core kernels take (multiples of 32 for keys, of 16 for values), no bigram, no loop
LUT_C = {
    "architecture": "Lutosun", "width": 128, "vocab": 211, "norm": {"eps": 1e-5}, "residual_mult": 0.25,
    "embedding": {"scale": 5.0}, "logit_softcap": 30.0,
    "layers": [with_mlp(latent(4, 32, 32, 32, 48, 96, base=1000.0), moe(9, 3, 64, 1.2, 2.5, shared=(96, 1.2))),
               with_mlp(latent(8, 64, 64, 16, 32, 64, base=1000.0), moe(4, 2, 32, 1.2, 1.0, shared=(32, 1.2)))],
}

CONFIGS = {"A": LUT_A, "B": LUT_B, "C": LUT_C}


def config_of(name: str) -> LutosunConfig:
    return LutosunConfig.from_dict(json.loads(json.dumps(CONFIGS[name])))


def make_model_dir(name: str, folder, seed: int = 11, storage_dtype=torch.bfloat16, preset: str = "unit"):
    """Write the configuration ``name`` with random weights into ``folder``; returns (raw config, tensors by their
    stored names, in float32)."""
    config = config_of(name) if isinstance(name, str) else LutosunConfig.from_dict(name)
    write_random_model(config, seed, str(folder), storage_dtype, preset)
    with open(os.path.join(str(folder), "config.json")) as handle:
        raw = json.load(handle)
    handle = SafetensorsFile(os.path.join(str(folder), "model.safetensors"))
    tensors = {stored: handle.tensor(stored).to(torch.float32) for stored in handle.names()}
    handle.close()
    return raw, tensors
