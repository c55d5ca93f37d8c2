"""Position encodings that act on q and k as a rotation of pairs.

``rotary``: inv_i = 1 / theta^(2i / rotary_dim), angle = position * inv_i, both in 32-bit
(engine/input_prep.cpp:17-30); pairs are (i, i + rotary_dim/2) for "half_split", the reference's
interleave=false (kernels/rope.cpp:38-48), or (2i, 2i + 1) for "interleaved"; dims beyond rotary_dim
pass unchanged.  ``none`` rotates nothing.

``scaling`` {factor, original, fast, slow} stretches the slow frequencies for sequences longer than ``original``: with
dim(t) = rotary_dim ln(original / (2 pi t)) / (2 ln theta), lo = max(floor(dim(fast)), 0), hi = min(ceil(dim(slow)),
rotary_dim - 1) and ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), pair i turns with inv_i / factor * ramp_i +
inv_i (1 - ramp_i), and cos and sin are both multiplied by 0.1 ln(factor) + 1.

``scaling`` {kind: "linear", factor}: every frequency is divided by ``factor`` (positions count ``factor`` times slower);
cos and sin keep their size.

A position part hands the mixer cos/sin rows for the step's tokens, as the reference feeds its graph
(models/qwen3.py:226-227); they are made once per step and shared by all layers that use the same
part settings.
"""
from __future__ import annotations

import math

import numpy as np
import torch

from ..kernels import ops
from .base import register_part

PAIRINGS = {"half_split": 0, "interleaved": 1}


@register_part("position", "rotary")
class Rotary:
    capturable = True

    def __init__(self, spec, builder):
        self.rotary_dim = int(spec.params["rotary_dim"])
        self.theta = float(spec.params["theta"])
        self.pairing = str(spec.params.get("pairing", "half_split"))
        if self.pairing not in PAIRINGS:
            raise ValueError(f"rotary pairing {self.pairing!r} is not one of {sorted(PAIRINGS)}")
        if self.rotary_dim <= 0 or self.rotary_dim % 2:
            raise ValueError(f"rotary_dim = {self.rotary_dim} must be positive and even")
        half = self.rotary_dim // 2
        i = np.arange(half, dtype=np.float32)
        inv = np.float32(1.0) / np.power(np.float32(self.theta), np.float32(2.0) * i / np.float32(self.rotary_dim))
        self.magnitude = 1.0
        scaling = spec.params.get("scaling")
        if scaling and scaling.get("kind") == "linear":
            inv = (inv.astype(np.float64) / float(scaling["factor"])).astype(np.float32)
        elif scaling:
            factor, original = float(scaling["factor"]), float(scaling["original"])

            def dim_of(turns: float) -> float:
                return self.rotary_dim * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))

            lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
            hi = min(math.ceil(dim_of(float(scaling["slow"]))), self.rotary_dim - 1)
            ramp = np.clip((i.astype(np.float64) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
            inv = (inv.astype(np.float64) / factor * ramp + inv.astype(np.float64) * (1.0 - ramp)).astype(np.float32)
            self.magnitude = 0.1 * math.log(factor) + 1.0
        self.inv_freq = torch.from_numpy(inv.astype(np.float32)).to(builder.device)
        self._key = ("rotary", self.rotary_dim, self.theta, tuple(sorted((k, str(v)) for k, v in scaling.items())) if scaling else None)

    def tables(self, ctx):
        if self._key not in ctx.memo:
            ctx.memo[self._key] = ops.rope_table(ctx.positions, self.inv_freq, self.magnitude)
        return ctx.memo[self._key]


@register_part("position", "none")
class NoPosition:
    capturable = True
    rotary_dim, pairing = 0, "half_split"

    def __init__(self, spec, builder):
        pass

    def tables(self, ctx):
        return None
