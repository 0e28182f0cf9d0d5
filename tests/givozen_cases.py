"""Shared by the Givozen tests: small configurations, model folders with seeded random weights, ways of cutting a run."""

from __future__ import annotations

import copy
import json
import os
import random
import tempfile
from functools import lru_cache

import numpy as np
import torch

import plain_givozen

_TMP = tempfile.TemporaryDirectory(prefix="llmx_amd_givozen_")


def _mixer(heads, kv_heads, dim, vdim, scale, base, dims, scaling=None):
    rot = {"base": base, "dims": dims}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot}


def _moe(experts, top, ff, limit, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}
    if shared:
        out["shared"] = {"ff": shared[0], "limit": shared[1]}
    return out


def _layer(mixer, mlp):
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


# A: sizes the matrix-core products and (keys as wide as values, pages of 16) the matrix-core attention take; a run of two
#    layers in the middle repeated three times; two picks of six experts with a shared expert of another width and clamp,
#    one pick without a shared expert, a dense layer and a layer without a feed-forward; two mixers of different sizes.
_A_WIDE = _mixer(4, 2, 32, 32, 0.2, 10000.0, 16, (4.0, 1.0, 4.0, 64))
_A_NARROW = _mixer(8, 2, 16, 16, 0.31, 500.0, 8, (2.0, 0.5, 3.0, 48))
CONFIG_A = {
    "architecture": "Givozen", "vocab": 320, "width": 128, "norm": {"eps": 1e-6},
    "layers": [
        _layer(_A_WIDE, {"kind": "dense", "ff": 192}),
        _layer(_A_NARROW, _moe(6, 2, 64, 1.5, (48, 2.5))),
        _layer(_A_WIDE, _moe(4, 1, 32, 3.0)),
        _layer(_A_WIDE, None),
    ],
    "loop": {"start": 1, "stop": 3, "times": 3},
}
# B: sizes no kernel tiles evenly (the universal products and attention run), values narrower than keys, one key head, all
#    three of three experts picked, no frequency scaling, no loop, pages of 4.
CONFIG_B = {
    "architecture": "Givozen", "vocab": 97, "width": 54, "norm": {"eps": 1e-5},
    "layers": [
        _layer(_mixer(3, 1, 10, 6, 0.5, 77.0, 6), _moe(3, 3, 10, 0.7, (5, 1.1))),
        _layer(_mixer(3, 3, 10, 14, 0.25, 77.0, 10), {"kind": "dense", "ff": 21}),
    ],
}
# C: as many key heads as query heads, values wider than keys, every dim of a head rotated in one layer and none in another,
#    the whole model repeated twice, three picks of five experts.
CONFIG_C = {
    "architecture": "Givozen", "vocab": 128, "width": 64, "norm": {"eps": 1e-6},
    "layers": [
        _layer(_mixer(6, 6, 16, 48, 0.4, 5000.0, 16, (8.0, 2.0, 16.0, 32)), _moe(5, 3, 32, 2.0, (16, 2.0))),
        _layer(_mixer(2, 1, 48, 16, 0.1, 1000.0, 0), {"kind": "dense", "ff": 64}),
    ],
    "loop": {"start": 0, "stop": 2, "times": 2},
}
# D: a loop of one pass over the last layer only (its vector is added once, the embedding rows never), one head.
CONFIG_D = {
    "architecture": "Givozen", "vocab": 80, "width": 48, "norm": {"eps": 1e-6},
    "layers": [
        _layer(_mixer(1, 1, 64, 64, 0.09, 100.0, 32, (3.0, 1.0, 2.0, 16)), {"kind": "dense", "ff": 72}),
        _layer(_mixer(2, 2, 32, 32, 0.3, 100.0, 4), _moe(2, 1, 24, 5.0, (8, 0.5))),
    ],
    "loop": {"start": 1, "stop": 2, "times": 1},
}
# E: the repeated run reaches the model's end and holds a layer without feed-forward; one pick of sixteen experts beside a
#    shared expert wider than they are; grouped heads with values twice as wide as keys beside a mixer with one key head.
_E_WIDE = _mixer(6, 3, 32, 64, 0.21, 20000.0, 32, (4.0, 1.0, 8.0, 256))
_E_ONE = _mixer(4, 1, 48, 48, 0.17, 3000.0, 24)
CONFIG_E = {
    "architecture": "Givozen", "vocab": 700, "width": 192, "norm": {"eps": 1e-5},
    "layers": [
        _layer(_E_WIDE, _moe(4, 2, 80, 1.2)),
        _layer(_E_ONE, {"kind": "dense", "ff": 320}),
        _layer(_E_WIDE, None),
        _layer(_E_ONE, _moe(16, 1, 48, 4.0, (112, 0.9))),
    ],
    "loop": {"start": 2, "stop": 4, "times": 3},
}
# F: heads of 128 and of 64 (the matrix-core attention's widest kernels, prompt tiles and split contexts), the first layer
#    alone repeated, every one of six experts picked in the last layer.
_F_WIDE = _mixer(4, 2, 128, 128, 0.088, 500000.0, 64, (8.0, 1.0, 4.0, 512))
CONFIG_F = {
    "architecture": "Givozen", "vocab": 512, "width": 384, "norm": {"eps": 1e-6},
    "layers": [
        _layer(_F_WIDE, _moe(6, 2, 96, 3.0, (160, 1.5))),
        _layer(_mixer(6, 3, 64, 64, 0.125, 10000.0, 32, (2.0, 1.0, 2.0, 128)), {"kind": "dense", "ff": 640}),
        _layer(_F_WIDE, _moe(6, 6, 96, 2.0)),
    ],
    "loop": {"start": 0, "stop": 1, "times": 2},
}
CONFIGS = {"A": CONFIG_A, "B": CONFIG_B, "C": CONFIG_C, "D": CONFIG_D, "E": CONFIG_E, "F": CONFIG_F}
PAGES = {"A": 16, "B": 4, "C": 16, "D": 16, "E": 16, "F": 16}
SEEDS = {"A": 21, "B": 22, "C": 23, "D": 24, "E": 25, "F": 26}


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
    rng = random.Random(7919 * seed + length)
    return [rng.randrange(CONFIGS[name]["vocab"]) for _ in range(length)]


@lru_cache(maxsize=None)
def plain_logits(name: str, length: int, seed: int):
    config, tensors = plain(name)
    return torch.from_numpy(plain_givozen.forward(config, tensors, tokens_for(name, length, seed)))


def routed_runs(config: dict):
    """The places in the run order at which a routed feed-forward runs."""
    return [at for at, (i, _, _) in enumerate(plain_givozen.run_order(config)) if (config["layers"][i].get("mlp") or {}).get("kind") == "moe"]


def greedy(config, tensors, prompt, n):
    """n tokens, each the largest logit after everything before it (the whole sequence is run again for each)."""
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(np.argmax(plain_givozen.forward(config, tensors, seq)[-1])))
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
