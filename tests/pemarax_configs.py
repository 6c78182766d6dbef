"""Small Pemarax configurations of the tests, and helpers that write them as model folders.

They differ from each other in every size and in the order of their layers: width, vocabulary, query and key/value
heads (one, several, as many as query heads), key and value widths, windows (shorter than a cache page, longer than
a prompt), kept first tokens (none, a few, more than a page), taps of the convolutions (two to four, and none),
rotated dimensions (all of a head, a part), ramp scaling (with and without), latent ranks and turned parts
(a part of the turned part, no turned part at all), state-space heads, groups and norm groups (values that are 1 in
one model are not in another), experts and how many a token uses, a layer without a feed-forward, and the
multiplier of the branches (one model has 1).
"""
import json
import os

import torch

from macllm_infer_amd.config import PemaraxConfig
from macllm_infer_amd.weights.random_init import write_random_model
from macllm_infer_amd.weights.safetensors_io import SafetensorsFile


def attention(heads, kv_heads, dim, vdim, window, keep_first=0, conv=3, rot_dims=None, scaling=None, base=10000.0,
              scale=None):
    mixer = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim, "scale": dim ** -0.5 if scale is None else scale,
             "mask": {"size": window}}
    if keep_first:
        mixer["mask"]["keep_first"] = keep_first
    if conv:
        mixer["conv"] = conv
    if rot_dims:
        mixer["rot"] = {"base": base, "dims": rot_dims}
        if scaling is not None:
            mixer["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return {"type": "attention", "mixer": mixer}


def latent(heads, dim, rot_dim, vdim, kv_rank, window, rot_dims=None, base=10000.0, scale=None):
    mixer = {"dim": dim, "heads": heads, "kv_rank": kv_rank, "rot_dim": rot_dim, "vdim": vdim,
             "scale": (dim + rot_dim) ** -0.5 if scale is None else scale, "mask": {"size": window}}
    if rot_dim:
        mixer["rot"] = {"base": base, "dims": rot_dim if rot_dims is None else rot_dims}
    return {"type": "latent_attention", "mixer": mixer}


def parallel(left, right):
    heads, kv_heads, dim, vdim, window = left
    ssm_heads, ssm_vdim, state, groups, norm_groups, conv = right
    return {"type": "parallel", "mixer": {
        "left": {"dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim, "scale": dim ** -0.5, "mask": {"size": window}},
        "right": {"conv": conv, "groups": groups, "heads": ssm_heads, "norm_groups": norm_groups, "state": state,
                  "vdim": ssm_vdim}}}


def moe(experts, top, ff):
    return {"expert": {"ff": ff}, "kind": "moe", "router": {"experts": experts, "top": top}}


def with_mlp(layer, mlp):
    return dict(layer, mlp=mlp)


PEM_A = {
    "architecture": "Pemarax", "width": 48, "vocab": 101, "norm": {"eps": 1e-5}, "residual_mult": 0.6,
    "layers": [
        with_mlp(parallel((4, 2, 8, 12, 9), (3, 8, 12, 1, 1, 4)), moe(5, 2, 24)),
        with_mlp(attention(4, 2, 16, 8, window=11, keep_first=3, conv=3, rot_dims=16, scaling=(4.0, 64, 8.0, 1.0)), moe(5, 2, 24)),
        with_mlp(latent(3, 8, 8, 12, 16, window=13), None),
        with_mlp(attention(2, 2, 8, 8, window=40, keep_first=10, conv=2, rot_dims=4), moe(6, 1, 16)),
    ],
}

PEM_B = {
    "architecture": "Pemarax", "width": 40, "vocab": 67, "norm": {"eps": 1e-6}, "residual_mult": 1.0,
    "layers": [
        with_mlp(latent(2, 12, 4, 6, 20, window=7, rot_dims=2, base=500.0), moe(4, 4, 12)),
        with_mlp(attention(3, 1, 12, 20, window=6, keep_first=0, conv=4, rot_dims=12, scaling=(8.0, 32, 4.0, 0.5), base=777.0),
                 moe(3, 2, 20)),
        with_mlp(parallel((2, 1, 12, 4, 30), (4, 6, 8, 2, 2, 2)), None),
        with_mlp(latent(1, 16, 0, 16, 12, window=100), moe(7, 3, 8)),
        with_mlp(attention(2, 1, 8, 8, window=5, keep_first=2, conv=0), None),
    ],
}

# the head and state sizes that the matrix-core kernels take, so that bfloat16 steps run through them
PEM_C = {
    "architecture": "Pemarax", "width": 128, "vocab": 211, "norm": {"eps": 1e-5}, "residual_mult": 0.8,
    "layers": [
        with_mlp(attention(4, 2, 64, 64, window=80, keep_first=5, conv=3, rot_dims=64, scaling=(4.0, 128, 16.0, 1.0)), moe(8, 2, 64)),
        with_mlp(latent(4, 32, 32, 48, 64, window=70), moe(8, 2, 64)),
        with_mlp(parallel((4, 1, 64, 64, 48), (4, 32, 32, 1, 2, 3)), moe(8, 3, 32)),
        with_mlp(attention(2, 1, 128, 128, window=33, keep_first=1, conv=2, rot_dims=32), None),
    ],
}

CONFIGS = {"A": PEM_A, "B": PEM_B, "C": PEM_C}


def config_of(name: str) -> PemaraxConfig:
    return PemaraxConfig.from_dict(CONFIGS[name])


def make_model_dir(name, folder, seed: int = 23, storage_dtype=torch.bfloat16, preset: str = "unit"):
    """Write the configuration ``name`` (or a raw configuration) with random weights into ``folder``; returns
    (raw config, tensors by their stored names, in float32)."""
    config = config_of(name) if isinstance(name, str) else PemaraxConfig.from_dict(name)
    write_random_model(config, seed, str(folder), storage_dtype, preset)
    with open(os.path.join(str(folder), "config.json")) as handle:
        raw = json.load(handle)
    handle = SafetensorsFile(os.path.join(str(folder), "model.safetensors"))
    tensors = {stored: handle.tensor(stored).to(torch.float32) for stored in handle.names()}
    handle.close()
    return raw, tensors
