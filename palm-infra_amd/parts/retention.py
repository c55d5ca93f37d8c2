"""Retention: linear attention with one fixed decay per head, without softmax or denominator.

Per head, with q_t, k_t of size ``key_dim`` and v_t of size ``value_dim``:

    S_t = decay_h * S_(t-1) + k_t v_t^T,      o_t = S_t^T q_t

q and k are rotated first if the part has a ``position`` (k is multiplied by ``key_scale`` after the rotation); each
head's o_t is divided by its root mean square (``eps`` inside the root, no weight); the heads are joined, multiplied by
silu of a gate projection and projected back.  One joined product makes q | k | v | gate.  S is float32 and is kept
per sequence (``StateNeed``); rotated values and everything in the recurrence are 32-bit whatever the run's type.

Options that make it other linear attentions of the same recurrence: ``input_activation`` "silu" puts q, k and v through
silu first; ``norm`` "joined" norms a token's heads together instead of each alone, o / sqrt(mean over all heads' values
of o^2 + eps) times the weight tensor ``norm`` (float32 [heads * value_dim]); ``gate_activation`` "sigmoid" gates with
the sigmoid of the gate rows instead of their silu.
"""
from __future__ import annotations

import torch

from ..cache import StateNeed
from ..kernels import ops
from .base import register_part
from .linear import Linear


@register_part("mixer", "retention")
class Retention:
    capturable = True

    def __init__(self, spec, builder):
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.nh, self.dk, self.dv = int(p["num_heads"]), int(p["key_dim"]), int(p["value_dim"])
        self.key_scale, self.eps = float(p["key_scale"]), float(p["eps"])
        if len(p["decay"]) != self.nh:
            raise ValueError(f"retention: {len(p['decay'])} decays for {self.nh} heads")
        self.decay = torch.tensor([float(d) for d in p["decay"]], dtype=torch.float32).to(builder.device)
        # the joined product is this part's own, or a wider one that the mixers beside it share (``input`` "shared")
        self.shared_input = p.get("input") == "shared"
        self.qkvg = None if self.shared_input else Linear(builder.tensor(spec, "qkvg"))
        self.out = Linear(builder.tensor(spec, "out"))
        self.in_rows = self.nh * 2 * (self.dk + self.dv)
        if self.qkvg is not None and self.qkvg.weight.shape != (self.in_rows, self.hidden):
            raise ValueError(f"retention: joined q/k/v/gate weight {tuple(self.qkvg.weight.shape)} does not fit {self.nh} heads "
                             f"of key size {self.dk} and value size {self.dv} over hidden {self.hidden}")
        if self.out.weight.shape != (self.hidden, self.nh * self.dv):
            raise ValueError(f"retention: output weight {tuple(self.out.weight.shape)} does not fit")
        self.input_silu = self._choice(p, "input_activation", (None, "silu")) == "silu"
        self.joined = self._choice(p, "norm", ("head_unit", "joined"), "head_unit") == "joined"
        self.gate_sigmoid = self._choice(p, "gate_activation", ("silu", "sigmoid"), "silu") == "sigmoid"
        self.norm_weight = builder.tensor(spec, "norm") if self.joined else None
        if self.gate_sigmoid and not self.joined:
            raise ValueError("retention: the per-head unit norm comes with a silu gate")
        self.position = builder.build(spec.parts["position"]) if "position" in spec.parts else None
        if self.position is not None and (self.position.pairing != "half_split" or self.position.rotary_dim > self.dk):
            raise ValueError("retention: the rotation pairs dimension i with i + rotary_dim/2 within the key size")

    @staticmethod
    def _choice(p, key, allowed, default=None):
        value = p.get(key, default)
        if value not in allowed:
            raise ValueError(f"retention: {key} = {value!r} is not one of {allowed}")
        return value

    @staticmethod
    def cache_needs(spec):
        p = spec.params
        return [StateNeed("retention", (int(p["num_heads"]), int(p["key_dim"]), int(p["value_dim"])))]

    def forward(self, h, ctx):
        if self.qkvg is None:
            raise RuntimeError("retention whose input product is shared gets its rows from the part that makes them")
        return self.forward_rows(self.qkvg(h), 0, ctx)

    def forward_rows(self, rows, col0, ctx):
        """``rows`` [n, >= col0 + in_rows]: q | k | v | gate from column ``col0``."""
        lc = ctx.layer_cache
        if lc is None or not lc.states or "retention" not in lc.states:
            raise RuntimeError("retention needs its state; the step gave it no cache")
        tables = self.position.tables(ctx) if self.position is not None else None
        cos, sin = tables if tables is not None else (None, None)
        o = ops.retention(rows, self.nh, self.dk, self.dv, self.decay, self.key_scale, self.eps, lc.states["retention"], ctx,
                          cos=cos, sin=sin, rot=self.position.rotary_dim if tables is not None else 0,
                          input_silu=self.input_silu, joined_norm=self.norm_weight, gate_sigmoid=self.gate_sigmoid, col0=col0)
        return self.out(o)
