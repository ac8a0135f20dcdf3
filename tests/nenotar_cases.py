"""Shared by the Nenotar tests: small configurations, model folders with seeded random weights, ways of cutting a run."""

from __future__ import annotations

import copy
import json
import os
import random
import tempfile
from functools import lru_cache

import torch

import plain_nenotar

_TMP = tempfile.TemporaryDirectory(prefix="llmx_amd_nenotar_")


def _latent(heads, dim, rot_dim, vdim, rank, scale, base, dims, scaling=None):
    rot = {"base": base, "dims": dims}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale, "rot": rot}


def _layer(kind, mixer, ff):
    return {"type": kind, "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


# P: every size differs from every other, sizes the matrix-core products take; both mixers, with and without a
#    feed-forward; rotated dims equal to and below the rotated part; with and without frequency scaling.
CONFIG_P = {
    "architecture": "Nenotar", "vocab": 304, "width": 80, "embedding": {"scale": 7.5}, "norm": {"eps": 1e-5}, "token_side": {"dim": 16},
    "layers": [
        _layer("mingru", {"width": 72}, 112),
        _layer("latent_attention", _latent(3, 24, 16, 40, 48, 0.21, 10000.0, 16, (8.0, 64, 16.0, 2.0)), 96),
        _layer("latent_attention", _latent(2, 8, 8, 16, 32, 0.35, 500.0, 4), None),
        _layer("mingru", {"width": 40}, None),
        _layer("latent_attention", _latent(5, 16, 8, 8, 24, 0.17, 250000.0, 8, (3.0, 32, 8.0, 0.5)), 64),
    ],
}
# Q: sizes no kernel tiles evenly (the universal products run), one head, no token input, a recurrent width of 1.
CONFIG_Q = {
    "architecture": "Nenotar", "vocab": 97, "width": 54, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6},
    "layers": [
        _layer("latent_attention", _latent(1, 5, 6, 3, 10, 0.4, 77.0, 6, (2.0, 16, 4.0, 1.5)), 33),
        _layer("mingru", {"width": 1}, 7),
        _layer("mingru", {"width": 67}, 50),
        _layer("latent_attention", _latent(7, 3, 2, 9, 11, 0.5, 1000.0, 2), 21),
    ],
}
# R: attention only (no per-request state), heads above one tile of sixteen, a token input of one dim.
CONFIG_R = {
    "architecture": "Nenotar", "vocab": 128, "width": 64, "embedding": {"scale": 3.0}, "norm": {"eps": 1e-6}, "token_side": {"dim": 1},
    "layers": [
        _layer("latent_attention", _latent(18, 16, 16, 16, 48, 0.18, 10000.0, 16, (4.0, 128, 32.0, 1.0)), 48),
        _layer("latent_attention", _latent(4, 32, 32, 24, 64, 0.125, 50000.0, 32), 48),
    ],
}
# S: recurrent layers only (no pages at all), one of them without a feed-forward.
CONFIG_S = {
    "architecture": "Nenotar", "vocab": 64, "width": 48, "embedding": {"scale": 2.0}, "norm": {"eps": 1e-6}, "token_side": {"dim": 8},
    "layers": [_layer("mingru", {"width": 56}, 40), _layer("mingru", {"width": 24}, None)],
}
CONFIGS = {"P": CONFIG_P, "Q": CONFIG_Q, "R": CONFIG_R, "S": CONFIG_S}
PAGES = {"P": 16, "Q": 4, "R": 16, "S": 16}
SEEDS = {"P": 3, "Q": 4, "R": 5, "S": 6}


def write_folder(config: dict, seed: int, folder: str, edit=None) -> str:
    """A model folder of `config` with the framework's seeded random weights; `edit(tensors)` may change them first."""
    from llmx_amd import RandomInit
    from llmx_amd.models import read_config
    from llmx_amd.weights.folder import random_tensors
    from llmx_amd.weights.safetensors_io import write_safetensors
    cfg = read_config(copy.deepcopy(config))
    tensors = random_tensors(cfg, RandomInit(seed=seed, std=0.06, norm_std=0.2, bias_range=0.5, storage="bfloat16"))
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


@lru_cache(maxsize=None)
def plain(name: str):
    return plain_nenotar.load_folder(model_folder(name))


def tokens_for(name: str, length: int, seed: int):
    rng = random.Random(7919 * seed + length)
    return [rng.randrange(CONFIGS[name]["vocab"]) for _ in range(length)]


@lru_cache(maxsize=None)
def plain_logits(name: str, length: int, seed: int, rounded: bool):
    cfg, w = plain(name)
    return plain_nenotar.forward(cfg, w, tokens_for(name, length, seed), torch.float64, torch.bfloat16 if rounded else None)


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
