"""Small Mukutar configurations of the tests, and helpers that write them as model folders.

They differ from each other in every size: width, vocabulary, heads and key/value heads, key and value widths
(equal in one, different in the other), windows, rotary dims (whole head and part of it), decay rank, layer
order, and a layer without a feed-forward.
"""
import json
import os

import torch

from macllm_infer_amd.config import MukutarConfig
from macllm_infer_amd.weights.random_init import write_random_model
from macllm_infer_amd.weights.safetensors_io import SafetensorsFile


def attention(heads, kv_heads, dim, vdim, window, scale=None):
    mixer = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "scale": dim ** -0.5 if scale is None else scale,
             "vdim": vdim}
    if window is not None:
        mixer["mask"] = {"size": window}
    return {"type": "attention", "mixer": mixer}


def retention(heads, dim, vdim, rot_dims, base=10000.0, decay=None):
    decay = decay or [1.0 - 2.0 ** (-3 - head) for head in range(heads)]
    mixer = {"decay": decay, "dim": dim, "heads": heads, "vdim": vdim}
    if rot_dims:
        mixer["rot"] = {"base": base, "dims": rot_dims}
    return {"type": "retention", "mixer": mixer}


def general_delta(heads, dim, rank):
    return {"type": "general_delta", "mixer": {"dim": dim, "heads": heads, "decay_rank": rank}}


def with_mlp(layer, ff):
    return dict(layer, mlp=None if ff is None else {"ff": ff, "kind": "dense"})


MUK_A = {"architecture": "Mukutar", "width": 64, "vocab": 96, "norm": {"eps": 1e-5}, "layers": [
    with_mlp(general_delta(2, 16, 8), 80),
    with_mlp(attention(4, 2, 16, 16, 9), 80),
    with_mlp(retention(2, 16, 16, 16), 80)]}

MUK_B = {"architecture": "Mukutar", "width": 48, "vocab": 131, "norm": {"eps": 3e-6}, "layers": [
    with_mlp(attention(3, 1, 32, 16, 21, scale=0.3), 56),
    with_mlp(retention(3, 24, 40, 12, base=500.0), None),
    with_mlp(general_delta(3, 24, 5), 72),
    with_mlp(attention(2, 2, 16, 48, 5), 40),
    with_mlp(retention(1, 32, 8, 0), 64)]}

CONFIGS = {"A": (MUK_A, 11), "B": (MUK_B, 12)}


def make_model_dir(raw, folder, seed=0, dtype=torch.float32):
    """Write a random model of the configuration ``raw`` (a name of CONFIGS or a dictionary); returns
    (raw configuration as read back, tensors by their stored names in float32)."""
    if isinstance(raw, str):
        raw, seed = CONFIGS[raw]
    write_random_model(MukutarConfig.from_dict(raw), seed, str(folder), dtype, "unit")
    return load_model_dir(folder)


def load_model_dir(folder):
    with open(os.path.join(str(folder), "config.json")) as handle:
        raw = json.load(handle)
    handle = SafetensorsFile(os.path.join(str(folder), "model.safetensors"))
    tensors = {name: handle.tensor(name).to(torch.float32) for name in handle.names()}
    handle.close()
    return raw, tensors
