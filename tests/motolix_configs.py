"""Small Motolix configurations of the tests, and helpers that write them as model folders.

They differ from each other in every size: width, vocabulary, heads and key/value heads (one group, several, as many
as heads), key and value widths (equal, narrower, wider), rotary dims (whole head, part of it), frequency stretching
(with, without, on either kind of attention), the decay's temperature and inner width, scales of the two sides, the
order of layers, layers without a feed-forward, and the loop (none, from the first layer, to the last, three passes,
one pass).
"""
import json
import os

import torch

from macllm_infer_amd.config import MotolixConfig
from macllm_infer_amd.weights.random_init import write_random_model
from macllm_infer_amd.weights.safetensors_io import SafetensorsFile


def rot(base, dims, scaling=None):
    out = {"base": base, "dims": dims}
    if scaling is not None:
        out["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return out


def attention(heads, kv_heads, dim, scale, rotation):
    return {"type": "attention", "mixer": {"dim": dim, "heads": heads, "kv_heads": kv_heads, "rot": rotation,
                                           "scale": scale, "vdim": dim}}


def parallel(left, right, left_scale, right_scale):
    heads, kv_heads, dim, vdim, scale, rotation = left
    glu_heads, glu_dim, glu_vdim, tau = right
    return {"type": "parallel", "mixer": {
        "left": {"dim": dim, "heads": heads, "kv_heads": kv_heads, "rot": rotation, "scale": scale, "vdim": vdim},
        "left_scale": left_scale,
        "right": {"dim": glu_dim, "heads": glu_heads, "tau": tau, "vdim": glu_vdim},
        "right_scale": right_scale}}


def with_mlp(layer, ff):
    return dict(layer, mlp=None if ff is None else {"ff": ff, "kind": "dense"})


def model(width, vocab, eps, layers, loop=None, embedding_scale=1.0, logit_scale=1.0):
    raw = {"architecture": "Motolix", "embedding": {"scale": embedding_scale}, "layers": layers,
           "logit_scale": logit_scale, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if loop is not None:
        raw["loop"] = dict(zip(("start", "stop", "times"), loop))
    return raw


# the loop opens the model; two groups of keys; values narrower than keys; rotation of a part of the head
MOT_A = model(64, 96, 1e-5, [
    with_mlp(parallel((4, 2, 16, 8, 0.3, rot(10000.0, 8)), (2, 16, 16, 8.0), 0.8, 1.3), 80),
    with_mlp(attention(4, 2, 16, 0.25, rot(10000.0, 16, (8.0, 1.0, 4.0, 64))), 72),
    with_mlp(parallel((2, 1, 32, 32, 0.2, rot(300.0, 32, (2.0, 1.0, 2.0, 32))), (1, 24, 40, 4.0), 1.0, 1.0), None)],
    loop=(0, 2, 3), embedding_scale=8.0, logit_scale=0.5)

# no loop at all; as many key heads as query heads; an attention layer without a feed-forward, first in the model
MOT_B = model(48, 131, 3e-6, [
    with_mlp(attention(3, 3, 24, 0.3, rot(500.0, 12)), None),
    with_mlp(parallel((3, 3, 16, 24, 0.25, rot(500.0, 16)), (3, 8, 24, 1.0), 1.5, 0.5), 56),
    with_mlp(attention(2, 1, 40, 0.15, rot(1e6, 40)), 40)],
    embedding_scale=1.0, logit_scale=1.0)

# the loop closes the model and runs once; heads of 128 and of 64; wide values
MOT_C = model(96, 70, 1e-6, [
    with_mlp(attention(2, 2, 128, 0.09, rot(1e5, 64, (4.0, 1.0, 4.0, 256))), 120),
    with_mlp(parallel((6, 2, 64, 128, 0.125, rot(1e5, 64)), (2, 64, 128, 12.0), 1.4, 0.6), 200),
    with_mlp(parallel((5, 1, 24, 12, 0.2, rot(1e4, 24)), (4, 12, 20, 2.5), 0.7, 0.9), 64),
    with_mlp(attention(6, 3, 32, 0.18, rot(1e4, 8)), 96)],
    loop=(2, 4, 1), embedding_scale=3.0, logit_scale=0.3)

# two passes over the middle
MOT_D = model(80, 57, 2e-5, [
    with_mlp(attention(5, 1, 16, 0.25, rot(2e4, 16)), 48),
    with_mlp(parallel((2, 2, 48, 16, 0.14, rot(2e4, 24)), (5, 16, 8, 32.0), 1.0, 2.0), 96),
    with_mlp(attention(1, 1, 80, 0.11, rot(2e4, 80, (16.0, 2.0, 8.0, 128))), None),
    with_mlp(parallel((8, 4, 8, 10, 0.35, rot(50.0, 8)), (1, 80, 80, 6.0), 0.5, 1.0), 88)],
    loop=(1, 3, 2), embedding_scale=5.0, logit_scale=2.0)

CONFIGS = {"A": (MOT_A, 11), "B": (MOT_B, 12), "C": (MOT_C, 13), "D": (MOT_D, 14)}


def make_model_dir(raw, folder, seed=0, dtype=torch.float32):
    """Write a random model of the configuration ``raw`` (a name of CONFIGS or a dictionary); returns
    (raw configuration as read back, tensors by their stored names in float32)."""
    if isinstance(raw, str):
        raw, seed = CONFIGS[raw]
    write_random_model(MotolixConfig.from_dict(raw), seed, str(folder), dtype, "unit")
    return load_model_dir(folder)


def load_model_dir(folder):
    with open(os.path.join(str(folder), "config.json")) as handle:
        raw = json.load(handle)
    handle = SafetensorsFile(os.path.join(str(folder), "model.safetensors"))
    tensors = {name: handle.tensor(name).to(torch.float32) for name in handle.names()}
    handle.close()
    return raw, tensors
