"""Feed-forwards.

``gated_silu``: down( silu(gate(h)) * up(h) ), silu(z) = z / (1 + exp(-z)), with gate and up
joined into one [2I, H] product (models/qwen3.py:276-287; kernels/elementwise.cpp:529-583).

``routed_gated_silu``: ``experts`` gated-silu feed-forwards of which every token goes through ``top``: the router's
logits W_r h + b are 32-bit, the ``top`` largest choose the experts, their weights are the softmax over those logits
alone, and the output is the weighted sum of the chosen experts' outputs.  A step of few rows (a decode step) reads each
(token, choice)'s expert in the kernel, nothing planned on the host (and so it can be recorded); a prompt's (token,
choice) pairs are grouped by expert on the device and all experts' rows go through two grouped products on the matrix
cores (bfloat16); in the float32 mode, and for sizes those do not take, the host groups the pairs and every expert's
rows go through its two products as ``Linear`` makes them.

``capped_gated``: down( g * sigmoid(slope * g) * (u + shift) ) with g = min(gate(h), limit) and u = clamp(up(h), -limit,
limit); gate and up joined into one [2I, H] product.

``dense``: down(act(up(h))) with an activation chosen by name.  ``xielu`` has two learned numbers p, q (tensor
``activation``, float32 [2]): for z > 0, softplus(p) z^2 + z/2; for z <= 0, (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2."""
from __future__ import annotations

import numpy as np
import torch

from ..kernels import ops
from .base import register_part
from .linear import Linear
from .residual import as_tensor


@register_part("feed_forward", "gated_silu")
class GatedSiluFeedForward:
    capturable = True

    def __init__(self, spec, builder):
        self.hidden = int(spec.params["hidden_size"])
        self.inter = int(spec.params["intermediate_size"])
        bias = lambda name: builder.tensor(spec, name) if name in spec.tensors else None
        self.gate_up = Linear(builder.tensor(spec, "gate_up"), bias("gate_up_bias"))
        self.down = Linear(builder.tensor(spec, "down"), bias("down_bias"))
        if self.gate_up.weight.shape != (2 * self.inter, self.hidden) or self.down.weight.shape != (self.hidden, self.inter):
            raise ValueError(f"feed-forward: weights {tuple(self.gate_up.weight.shape)}, {tuple(self.down.weight.shape)} "
                             f"do not fit hidden {self.hidden}, intermediate {self.inter}")

    takes_sink = True

    def forward(self, h, ctx, sink=None):
        return self.down(self.gate_up.gated(h), sink=sink)


@register_part("feed_forward", "capped_gated")
class CappedGatedFeedForward:
    capturable = True

    def __init__(self, spec, builder):
        p = spec.params
        self.hidden, self.inter = int(p["hidden_size"]), int(p["intermediate_size"])
        self.limit, self.slope, self.shift = float(p["limit"]), float(p.get("slope", 1.0)), float(p.get("shift", 0.0))
        if not self.limit > 0:
            raise ValueError(f"feed-forward: limit = {self.limit} must be positive")
        self.gate_up = Linear(builder.tensor(spec, "gate_up"))
        self.down = Linear(builder.tensor(spec, "down"))
        if self.gate_up.weight.shape != (2 * self.inter, self.hidden) or self.down.weight.shape != (self.hidden, self.inter):
            raise ValueError(f"feed-forward: weights {tuple(self.gate_up.weight.shape)}, {tuple(self.down.weight.shape)} "
                             f"do not fit hidden {self.hidden}, intermediate {self.inter}")

    def forward(self, h, ctx):
        return self.down(ops.capped_gate(self.gate_up(as_tensor(h)), self.limit, self.slope, self.shift))


@register_part("feed_forward", "dense")
class DenseFeedForward:
    capturable = True
    ACTIVATIONS = ("xielu",)

    def __init__(self, spec, builder):
        self.hidden = int(spec.params["hidden_size"])
        self.inter = int(spec.params["intermediate_size"])
        self.activation = str(spec.params.get("activation", "xielu"))
        if self.activation not in self.ACTIVATIONS:
            raise ValueError(f"feed-forward: activation {self.activation!r} is not one of {self.ACTIVATIONS}")
        self.up = Linear(builder.tensor(spec, "up"))
        self.down = Linear(builder.tensor(spec, "down"))
        self.act_params = builder.tensor(spec, "activation")
        if self.up.weight.shape != (self.inter, self.hidden) or self.down.weight.shape != (self.hidden, self.inter):
            raise ValueError(f"feed-forward: weights {tuple(self.up.weight.shape)}, {tuple(self.down.weight.shape)} "
                             f"do not fit hidden {self.hidden}, intermediate {self.inter}")
        if self.act_params.shape != (2,):
            raise ValueError(f"feed-forward: xielu takes two numbers, got {tuple(self.act_params.shape)}")

    takes_sink = True

    def forward(self, h, ctx, sink=None):
        return self.down(ops.xielu(self.up(as_tensor(h)), self.act_params), sink=sink)


@register_part("feed_forward", "routed_gated_silu")
class RoutedGatedSiluFeedForward:
    capturable = True            # steps of up to DIRECT_ROWS rows plan nothing on the host; longer ones are never recorded
    DIRECT_ROWS = 128            # as many rows as a recorded step holds at most

    def __init__(self, spec, builder):
        p = spec.params
        self.hidden, self.inter = int(p["hidden_size"]), int(p["intermediate_size"])
        self.experts, self.top = int(p["num_experts"]), int(p["top"])
        if not 1 <= self.top <= self.experts:
            raise ValueError(f"routed feed-forward: {self.top} of {self.experts} experts a token")
        self.router = Linear(builder.tensor(spec, "router"), builder.tensor(spec, "router_bias") if "router_bias" in spec.tensors else None)
        self.gate_up, self.down = builder.tensor(spec, "gate_up"), builder.tensor(spec, "down")
        E, F, W = self.experts, self.inter, self.hidden
        if self.router.weight.shape != (E, W) or self.gate_up.shape != (E * 2 * F, W) or self.down.shape != (E * W, F):
            raise ValueError(f"routed feed-forward: weights {tuple(self.router.weight.shape)}, {tuple(self.gate_up.shape)}, "
                             f"{tuple(self.down.shape)} do not fit {E} experts of inner size {F} over hidden {W}")
        # every expert's two matrices as products of their own, for the rows that a prompt sends it
        self.expert_gate_up = [Linear(self.gate_up[e * 2 * F:(e + 1) * 2 * F]) for e in range(E)]
        self.expert_down = [Linear(self.down[e * W:(e + 1) * W]) for e in range(E)]

    def forward(self, h, ctx):
        h = as_tensor(h)
        chosen, weight = ops.moe_route(self.router(h, out_dtype=torch.float32), self.top)
        if h.shape[0] <= self.DIRECT_ROWS:
            return ops.moe_experts(h, self.gate_up, self.down, chosen, weight, self.inter)
        if ops.moe_grouped_serves(h, self.gate_up, self.inter):
            return ops.moe_grouped(h, self.gate_up, self.down, chosen, weight, self.inter)
        # group the (token, choice) pairs by expert; within an expert in the order of the tokens
        flat = chosen.to("cpu").numpy().reshape(-1)
        order = np.argsort(flat, kind="stable").astype(np.int32)
        counts = np.bincount(flat, minlength=self.experts)
        src = torch.from_numpy(order // self.top).to(h.device)                   # the token of every pair, grouped
        pair_weight = weight.reshape(-1)
        xs = ops.gather_rows(h, src)
        ws = ops.gather_rows(pair_weight.reshape(-1, 1), torch.from_numpy(order).to(h.device)).reshape(-1)
        out = torch.zeros((h.shape[0], self.hidden), dtype=torch.float32, device=h.device)
        at = 0
        for e in range(self.experts):
            n = int(counts[e])
            if n:
                y = self.expert_down[e](self.expert_gate_up[e].gated(xs[at:at + n]))
                ops.scatter_add(out, y, src[at:at + n], ws[at:at + n])
                at += n
        return out
