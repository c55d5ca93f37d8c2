"""Small Biguzen configurations for the tests, with random weights, and helpers around them.

The configurations differ from each other in every size, in the number and order of layers and of streams (one, two, three),
and in which layers have a feed-forward and of which kind; between them they cover key/value heads shared by two, three and
eight query heads and one each, key and value sizes on both sides of a wave and no power of two, convolutions of two, three
and four taps and none, rotations of a part of a head, of all of it and none, scaled and plain frequencies, windows below
and above a page and none at all, layers that read another layer's keys and values by a longer window, a shorter one and
none, matrix memories of one head and several with value sizes below a wave and above two, routed experts in groups and
without, with and without a shared expert, one choice a token and several, and a model that begins with a matrix memory.
"""
from __future__ import annotations

import json
from pathlib import Path

import torch

from palm_infra_amd.config import config_from_dict
from palm_infra_amd.weights import random_tensors, write_safetensors


def attention(heads, kv, dim, vdim, scale, conv=None, window=None, rot=None, base=10000.0, factor=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if conv:
        m["conv"] = conv
    if window:
        m["mask"] = {"size": window}
    if rot:
        m["rot"] = {"dims": rot, "base": base}
        if factor:
            m["rot"]["scaling"] = {"factor": factor}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m}


def mlstm(heads, dim, vdim, cap):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, scale, groups=None, shared=None):
    f = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale}}
    if groups:
        f["router"]["groups"] = {"count": groups[0], "keep": groups[1]}
    if shared:
        f["shared"] = {"ff": shared}
    return f


def layer(mixer, mlp=None):
    return dict(mixer, mlp=mlp)


CONFIGS = {
    "A": {"architecture": "Biguzen", "vocab": 211, "width": 64, "streams": 3, "norm": {"eps": 1e-5}, "layers": [
        layer(mlstm(3, 16, 24, 10.0), moe(12, 3, 24, 1.5, groups=(3, 2), shared=40)),
        layer(attention(4, 2, 24, 40, 0.3, conv=4, window=37, rot=16, factor=2.0), dense(40)),
        layer(attention(4, 2, 24, 40, 0.2, conv=2, window=70, rot=16, factor=2.0, kv_from=1)),
        layer(mlstm(2, 24, 70, 6.0), dense(72)),
    ]},
    "B": {"architecture": "Biguzen", "vocab": 130, "width": 48, "streams": 1, "norm": {"eps": 2e-6}, "layers": [
        layer(attention(3, 3, 40, 72, 0.2, rot=40, base=500.0), moe(4, 2, 16, 1.0)),
        layer(mlstm(1, 40, 130, 15.0)),
        layer(attention(2, 1, 16, 16, 0.25, conv=3, window=5), moe(6, 1, 24, 2.0, groups=(2, 1), shared=8)),
        layer(attention(2, 1, 16, 16, 0.4, conv=3, kv_from=2), dense(56)),
    ]},
    # larger sizes: eight query heads for each key/value head, a key size of two waves' worth for the matrix memory, windows
    # of several pages, dense feed-forwards only
    "C": {"architecture": "Biguzen", "vocab": 150, "width": 96, "streams": 2, "norm": {"eps": 1e-5}, "layers": [
        layer(attention(16, 2, 64, 32, 0.125, conv=3, window=130, rot=32, base=50000.0, factor=8.0), dense(48)),
        layer(mlstm(2, 128, 64, 12.0), dense(112)),
        layer(attention(16, 2, 64, 32, 0.2, conv=3, window=200, rot=32, base=50000.0, factor=8.0, kv_from=0)),
        layer(mlstm(4, 32, 16, 8.0), dense(40)),
        layer(attention(6, 2, 32, 96, 0.2, window=64, rot=8, base=100.0), dense(64)),
    ]},
    "D": {"architecture": "Biguzen", "vocab": 97, "width": 40, "streams": 2, "norm": {"eps": 1e-6}, "layers": [
        layer(attention(6, 1, 8, 12, 0.5, conv=2), moe(16, 4, 8, 2.5, groups=(4, 2), shared=24)),
        layer(attention(6, 1, 8, 12, 0.7, conv=2, window=64, rot=4, base=250000.0, kv_from=0), moe(5, 5, 16, 0.5)),
    ]},
}
SEEDS = {"A": 71, "B": 72, "C": 73, "D": 74}
# one layer, for the tests of a mechanism alone
SINGLE = {
    "attention": {"architecture": "Biguzen", "vocab": 90, "width": 32, "streams": 1, "norm": {"eps": 1e-6},
                  "layers": [layer(attention(4, 2, 12, 20, 0.4, conv=3, window=50, rot=6, base=100.0, factor=3.0))]},
    "mlstm": {"architecture": "Biguzen", "vocab": 90, "width": 32, "streams": 1, "norm": {"eps": 1e-6},
              "layers": [layer(mlstm(3, 12, 20, 9.0))]},
    "dense": {"architecture": "Biguzen", "vocab": 90, "width": 32, "streams": 2, "norm": {"eps": 1e-6},
              "layers": [layer(mlstm(1, 8, 8, 9.0), dense(100))]},
    "routed": {"architecture": "Biguzen", "vocab": 90, "width": 32, "streams": 2, "norm": {"eps": 1e-6},
               "layers": [layer(mlstm(1, 8, 8, 9.0), moe(9, 2, 16, 1.7, groups=(3, 2), shared=12))]},
    "streams": {"architecture": "Biguzen", "vocab": 90, "width": 32, "streams": 5, "norm": {"eps": 1e-6},
                "layers": [layer(mlstm(1, 8, 8, 9.0), dense(16)), layer(mlstm(1, 8, 8, 9.0))]},
}


def tensors_of(raw: dict, seed: int, store: str) -> dict:
    """The random-weights mode's numbers (the description makes projections of a scale at which scores spread and gates open
    and close)."""
    tensors = random_tensors(config_from_dict(raw).spec(), seed, "float32")
    return {k: t.to({"bfloat16": torch.bfloat16, "float32": torch.float32}[store]) for k, t in tensors.items()}


def write_model(raw: dict, seed: int, path, store: str) -> Path:
    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(raw))
    write_safetensors(path / "model.safetensors", tensors_of(raw, seed, store))
    return path


def prompts(raw: dict, lengths, seed: int = 0) -> list:
    g = torch.Generator().manual_seed(5000 + seed)
    return [torch.randint(0, raw["vocab"], (n,), generator=g).tolist() for n in lengths]
