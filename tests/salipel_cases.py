"""Shared by the Salipel tests: small configurations, model folders with seeded random weights, ways of cutting a run."""

from __future__ import annotations

import copy
import json
import os
import random
import tempfile
from functools import lru_cache

import numpy as np
import torch

import plain_salipel

_TMP = tempfile.TemporaryDirectory(prefix="llmx_amd_salipel_")


def rot(base, dims, scaling=None):
    out = {"base": base, "dims": dims}
    if scaling:
        out["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return out


def chunked(heads, kv_heads, dim, vdim, scale, size):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": size}}}


def two_maps(heads, kv_heads, dim, vdim, scale, softcap, diff, rotation):
    return {"type": "attention_2", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                                             "softcap": softcap, "diff": diff, "rot": rotation}}


def side_by_side(left, right, left_scale, right_scale):
    heads, kv_heads, dim, scale, size, keep_first, rotation = left
    mask = {"size": size} if keep_first is None else {"size": size, "keep_first": keep_first}
    rh, rd, rv, cap = right
    return {"type": "parallel", "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale, "mask": mask,
                                                   "rot": rotation},
                                          "right": {"heads": rh, "dim": rd, "vdim": rv, "gate_cap": cap},
                                          "left_scale": left_scale, "right_scale": right_scale}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, scale):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale}}


def layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


# A: sizes the matrix-core products take, pages of 16; every mixer and every feed-forward, a layer without one; a window
#    and a chunk that end inside pages; the memory's key width below a wave.
CONFIG_A = {
    "architecture": "Salipel", "vocab": 320, "width": 128, "norm": {"eps": 1e-6}, "residual_mult": 0.6,
    "layers": [
        layer(two_maps(4, 2, 32, 64, 0.2, 30.0, 0.25, rot(10000.0, 16, (4.0, 1.0, 4.0, 64))), dense(192)),
        layer(side_by_side((4, 2, 32, 0.18, 24, 3, rot(500.0, 32)), (2, 16, 24, 8.0), 1.3, 0.4), moe(6, 2, 32, 1.5)),
        layer(chunked(4, 1, 16, 32, 0.3, 40), None),
        layer(two_maps(2, 2, 16, 16, 0.25, 8.0, 0.6, rot(300.0, 0)), moe(4, 1, 48, 0.7)),
    ],
}
# B: sizes no kernel tiles evenly (the universal products run), pages of 4; all of three experts picked; a window of 5
#    without kept tokens, chunks of 7, a memory with one head of 7 x 9; a soft cap small enough to bend the scores.
CONFIG_B = {
    "architecture": "Salipel", "vocab": 97, "width": 54, "norm": {"eps": 1e-5}, "residual_mult": 1.0,
    "layers": [
        layer(chunked(3, 3, 10, 6, 0.5, 7), moe(3, 3, 10, 1.0)),
        layer(side_by_side((3, 1, 10, 0.45, 5, None, rot(77.0, 6, (4.0, 1.0, 4.0, 32))), (1, 7, 9, 5.0), 0.8, 1.1), dense(21)),
        layer(two_maps(3, 1, 10, 14, 0.4, 1.5, 0.5, rot(77.0, 10)), dense(30)),
    ],
}
# C: edges: a window wider than any prompt here with more kept tokens than some prompts have; a window of one key beside
#    five kept ones; chunks of one position (a row sees itself and the sink); a memory as wide as a wave and one above it.
CONFIG_C = {
    "architecture": "Salipel", "vocab": 128, "width": 64, "norm": {"eps": 1e-6}, "residual_mult": 0.25,
    "layers": [
        layer(side_by_side((2, 2, 16, 0.3, 300, 8, rot(5000.0, 16, (8.0, 2.0, 16.0, 32))), (4, 64, 16, 15.0), 1.0, 1.0), None),
        layer(chunked(8, 2, 16, 16, 0.25, 1), dense(64)),
        layer(side_by_side((4, 1, 32, 0.2, 1, 5, rot(100.0, 8)), (1, 80, 40, 3.0), 0.5, 2.0), moe(5, 3, 16, 2.5)),
        layer(chunked(2, 1, 48, 8, 0.15, 16), moe(2, 1, 24, 1.0)),
    ],
}
# D: heads of 128 and a memory of 128 x 128 (two key channels a lane) beside one of 200 x 33; chunks that end on page
#    borders; one key head for six query heads.
CONFIG_D = {
    "architecture": "Salipel", "vocab": 512, "width": 256, "norm": {"eps": 1e-6}, "residual_mult": 0.8,
    "layers": [
        layer(side_by_side((4, 2, 128, 0.09, 100, 2, rot(500000.0, 64, (8.0, 1.0, 4.0, 128))), (2, 128, 128, 12.0), 1.1, 0.6), dense(384)),
        layer(chunked(6, 1, 64, 64, 0.125, 64), moe(8, 2, 64, 2.0)),
        layer(two_maps(4, 2, 64, 128, 0.125, 50.0, 0.3, rot(10000.0, 64)), moe(8, 8, 32, 1.0)),
        layer(side_by_side((2, 1, 64, 0.125, 33, 1, rot(1000.0, 16)), (1, 200, 33, 20.0), 0.7, 0.9), None),
    ],
}
CONFIGS = {"A": CONFIG_A, "B": CONFIG_B, "C": CONFIG_C, "D": CONFIG_D}
PAGES = {"A": 16, "B": 4, "C": 16, "D": 16}
SEEDS = {"A": 31, "B": 32, "C": 33, "D": 34}


def write_folder(config: dict, seed: int, folder: str, edit=None) -> str:
    """A model folder of `config` with the framework's seeded random weights; `edit(tensors)` may change them first."""
    from llmx_amd import RandomInit
    from llmx_amd.models import read_config
    from llmx_amd.weights.folder import random_tensors
    from llmx_amd.weights.safetensors_io import write_safetensors
    cfg = read_config(copy.deepcopy(config))
    tensors = random_tensors(cfg, RandomInit(seed=seed, std=0.08, norm_std=0.2, bias_range=0.5, storage="bfloat16"))
    if edit is not None:
        edit(tensors)
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config, f)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors, metadata={"format": "pt"})
    return folder


@lru_cache(maxsize=None)
def model_folder(name: str) -> str:
    return write_folder(CONFIGS[name], SEEDS[name], os.path.join(_TMP.name, name))


def load_plain(folder: str):
    """(config dict, {name: float64 numpy array}) of a model folder, read with the safetensors package."""
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as f:
        config = json.load(f)
    tensors = {k: v.to(torch.float64).numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    return config, tensors


@lru_cache(maxsize=None)
def plain(name: str):
    return load_plain(model_folder(name))


def tokens_for(name: str, length: int, seed: int):
    rng = random.Random(6131 * seed + length)
    return [rng.randrange(CONFIGS[name]["vocab"]) for _ in range(length)]


@lru_cache(maxsize=None)
def plain_logits(name: str, length: int, seed: int):
    config, tensors = plain(name)
    return torch.from_numpy(plain_salipel.forward(config, tensors, tokens_for(name, length, seed)))


def routed_layers(config: dict):
    return [i for i, entry in enumerate(config["layers"]) if (entry.get("mlp") or {}).get("kind") == "moe"]


def greedy(config, tensors, prompt, n):
    """n tokens, each the largest logit after everything before it (the whole sequence is run again for each)."""
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(np.argmax(plain_salipel.forward(config, tensors, seq)[-1])))
    return seq[len(prompt):]


def portions(length: int, seed: int, smallest: int = 2):
    """Cuts [0, length) into portions of changing size, several of them of `smallest` tokens."""
    rng = random.Random(seed)
    cuts, at = [], 0
    sizes = [smallest, 7, smallest, 16, 3, 33, smallest, 64, 5]
    while at < length:
        n = min(length - at, sizes[len(cuts) % len(sizes)] if rng.random() < 0.7 else rng.randrange(1, 40))
        cuts.append((at, at + n))
        at += n
    return cuts
