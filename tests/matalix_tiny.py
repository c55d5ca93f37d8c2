"""Small Matalix configurations for the tests, with random weights, and helpers around them.

The configurations differ from each other in every size, in the number of layers, in which layers have a feed-forward and in
which layers run again; between them they cover key/value heads shared by two, six and eight query heads and one each,
key sizes and value sizes on both sides of a wave and no power of two, rotations of a part of a head and of all of it and
none, frequencies stretched and plain, windows below and above a page and none at all, one decaying head and several,
decays near zero and near one, value sizes of the recurrence of less than a wave and of several, weights of the two sides
that are equal, one, and far apart, a range of layers that runs twice and three times from the first layer, from a later
one, and over all layers.
"""
from __future__ import annotations

import json
from pathlib import Path

import torch

from palm_infra_amd.config import config_from_dict
from palm_infra_amd.weights import random_tensors, write_safetensors


def _left(heads, kv, dim, vdim, scale, window, rot_dims, base=10000.0, scaling=None):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": window} if window else None,
            "rot": {"dims": rot_dims, "base": base, "scaling": scaling} if rot_dims else None}


def _right(heads, dim, vdim, decay):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}


def _layer(left, right, ls, rs, ff=None, limit=1.0):
    return {"type": "parallel", "mixer": {"left": left, "left_scale": ls, "right": right, "right_scale": rs},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff, "limit": limit}}


_YARN = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}

CONFIGS = {
    "A": {"architecture": "Matalix", "vocab": 211, "width": 64, "norm": {"eps": 1e-5}, "loop": {"start": 0, "stop": 2, "times": 3}, "layers": [
        _layer(_left(4, 2, 24, 40, 0.3, 37, 16, 10000.0, _YARN), _right(3, 16, 24, [0.5, 0.9, 0.99]), 0.7, 1.3, 40, 1.0),
        _layer(_left(4, 2, 24, 40, 0.3, 37, 16, 10000.0, _YARN), _right(3, 16, 24, [0.5, 0.9, 0.99]), 0.7, 1.3),
        _layer(_left(2, 1, 16, 16, 0.25, 5, 16, 500.0), _right(1, 8, 8, [0.95]), 1.0, 1.0, 72, 2.5),
    ]},
    "B": {"architecture": "Matalix", "vocab": 130, "width": 48, "norm": {"eps": 2e-6}, "layers": [
        _layer(_left(3, 3, 40, 72, 0.2, 70, 40, 500.0), _right(1, 40, 72, [0.97]), 1.0, 0.5, 24, 0.75),
        _layer(_left(3, 3, 40, 72, 0.2, 129, 8, 100.0, {"factor": 16.0, "original": 32, "fast": 4.0, "slow": 2.0}), _right(2, 24, 130, [0.2, 0.999]), 0.4, 2.0, 56, 3.0),
    ]},
    "C": {"architecture": "Matalix", "vocab": 97, "width": 40, "norm": {"eps": 1e-6}, "loop": {"start": 1, "stop": 2, "times": 2}, "layers": [
        _layer(_left(6, 1, 8, 12, 0.5, None, None), _right(2, 8, 130, [0.8, 0.6]), 1.5, 1.5, 16, 1.25),
        _layer(_left(6, 1, 8, 12, 0.5, 64, 4, 250000.0), _right(2, 8, 130, [0.8, 0.6]), 1.5, 1.5),
    ]},
    # larger sizes: eight query heads for each key/value head, a key size of two waves' worth for the recurrence, a window of
    # several pages, and all layers run twice
    "D": {"architecture": "Matalix", "vocab": 150, "width": 96, "norm": {"eps": 1e-5}, "loop": {"start": 0, "stop": 2, "times": 2}, "layers": [
        _layer(_left(16, 2, 64, 32, 0.125, 130, 32, 50000.0, {"factor": 8.0, "original": 128, "fast": 16.0, "slow": 1.0}),
               _right(2, 128, 64, [0.9, 0.995]), 1.1, 0.8, 48, 1.5),
        _layer(_left(10, 1, 32, 96, 0.2, 200, 32, 10000.0), _right(4, 32, 16, [0.3, 0.7, 0.9, 0.99]), 0.6, 1.2, 112, 2.0),
    ]},
}
SEEDS = {"A": 51, "B": 52, "C": 53, "D": 54}
# one layer, for the tests of a mechanism alone: a side is switched off by its weight
SINGLE = {
    "left": {"architecture": "Matalix", "vocab": 90, "width": 32, "norm": {"eps": 1e-6},
             "layers": [_layer(_left(4, 2, 12, 20, 0.4, 50, 6, 100.0, _YARN), _right(1, 8, 8, [0.9]), 1.0, 0.0)]},
    "right": {"architecture": "Matalix", "vocab": 90, "width": 32, "norm": {"eps": 1e-6},
              "layers": [_layer(_left(1, 1, 8, 8, 0.4, 9, None), _right(3, 12, 20, [0.4, 0.9, 0.99]), 0.0, 1.0)]},
    "feed_forward": {"architecture": "Matalix", "vocab": 90, "width": 32, "norm": {"eps": 1e-6},
                     "layers": [_layer(_left(1, 1, 8, 8, 0.4, 9, None), _right(1, 8, 8, [0.9]), 0.1, 0.1, 100, 0.5)]},
}


def tensors_of(raw: dict, seed: int, store: str) -> dict:
    """The random-weights mode's numbers (the description makes projections of a scale at which scores spread, gates open and
    close, and the feed-forward's rows reach their cap)."""
    tensors = random_tensors(config_from_dict(raw).spec(), seed, "float32")
    return {k: t.to({"bfloat16": torch.bfloat16, "float32": torch.float32}[store]) for k, t in tensors.items()}


def write_model(raw: dict, seed: int, path, store: str) -> Path:
    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(raw))
    write_safetensors(path / "model.safetensors", tensors_of(raw, seed, store))
    return path


def prompts(raw: dict, lengths, seed: int = 0) -> list:
    g = torch.Generator().manual_seed(4000 + seed)
    return [torch.randint(0, raw["vocab"], (n,), generator=g).tolist() for n in lengths]
