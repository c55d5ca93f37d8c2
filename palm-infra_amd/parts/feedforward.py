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
``activation``, float32 [2]): for z > 0, softplus(p) z^2 + z/2; for z <= 0, (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2.
``relu_squared`` is max(z, 0)^2, ``gelu_erf`` the exact gelu, ``gelu_tanh`` its tanh form.

``routed_scored``: ``experts`` plain feed-forwards down(gelu(up(h))) (the exact gelu, no biases) of which every token goes
through ``top``.  The router's logits are 32-bit, the scores their sigmoid; the choice is made by score plus the tensor
``correction``, the weights by the scores without it: the chosen experts' scores over their sum (+ 1e-20), times ``scale``.
With ``groups`` the experts lie in that many equal groups of neighbours, a group ranks by the sum of its two largest
corrected scores, and only experts of the best ``keep`` groups can be chosen.  With ``shared_size`` one more expert of that
inner size runs for every token and is added, times the sigmoid of one more router row (the last row of the tensor
``router``), one number per token.  The experts run as those of ``routed_gated_silu`` do."""
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
    ACTIVATIONS = ("xielu", "relu_squared", "gelu_erf", "gelu_tanh")

    def __init__(self, spec, builder):
        self.hidden = int(spec.params["hidden_size"])
        self.inter = int(spec.params["intermediate_size"])
        self.activation = str(spec.params.get("activation", "xielu"))
        if self.activation not in self.ACTIVATIONS:
            raise ValueError(f"feed-forward: activation {self.activation!r} is not one of {self.ACTIVATIONS}")
        self.up = Linear(builder.tensor(spec, "up"))
        self.down = Linear(builder.tensor(spec, "down"))
        self.act_params = builder.tensor(spec, "activation") if self.activation == "xielu" else None
        if self.up.weight.shape != (self.inter, self.hidden) or self.down.weight.shape != (self.hidden, self.inter):
            raise ValueError(f"feed-forward: weights {tuple(self.up.weight.shape)}, {tuple(self.down.weight.shape)} "
                             f"do not fit hidden {self.hidden}, intermediate {self.inter}")
        if self.act_params is not None and self.act_params.shape != (2,):
            raise ValueError(f"feed-forward: xielu takes two numbers, got {tuple(self.act_params.shape)}")

    takes_sink = True

    def forward(self, h, ctx, sink=None):
        z = self.up(as_tensor(h))
        mid = ops.xielu(z, self.act_params) if self.act_params is not None else ops.activation(z, self.activation)
        return self.down(mid, sink=sink)


class RoutedExperts:
    """The experts of a routed feed-forward and how a step's rows go through them, whatever chose them.  ``form``:
    "gated_silu" (an expert's first matrix holds its gate rows, then its up rows) or "gelu" (up rows alone)."""
    DIRECT_ROWS = 128            # as many rows as a recorded step holds at most

    def _set_experts(self, first, down, experts: int, inter: int, hidden: int, form: str):
        self.first, self.down_all, self.form = first, down, form
        self.experts, self.inter, self.hidden = experts, inter, hidden
        per = (2 if form == "gated_silu" else 1) * inter
        if first.shape != (experts * per, hidden) or down.shape != (experts * hidden, inter):
            raise ValueError(f"routed feed-forward: weights {tuple(first.shape)}, {tuple(down.shape)} do not fit {experts} experts of inner "
                             f"size {inter} over hidden {hidden}")
        # every expert's two matrices as products of their own, for the rows that a prompt sends it
        self.expert_first = [Linear(first[e * per:(e + 1) * per]) for e in range(experts)]
        self.expert_down = [Linear(down[e * hidden:(e + 1) * hidden]) for e in range(experts)]

    def _mid(self, e: int, xs):
        return self.expert_first[e].gated(xs) if self.form == "gated_silu" else ops.activation(self.expert_first[e](xs), "gelu_erf")

    def run_experts(self, h, chosen, weight):
        """float32 [n, hidden]: sum_c weight[t, c] * expert chosen[t, c] of h[t]."""
        top = chosen.shape[1]
        if h.shape[0] <= self.DIRECT_ROWS:
            return ops.moe_experts(h, self.first, self.down_all, chosen, weight, self.inter, self.form)
        if ops.moe_grouped_serves(h, self.first, self.inter):
            return ops.moe_grouped(h, self.first, self.down_all, chosen, weight, self.inter, self.form)
        # group the (token, choice) pairs by expert; within an expert in the order of the tokens
        flat = chosen.to("cpu").numpy().reshape(-1)
        order = np.argsort(flat, kind="stable").astype(np.int32)
        counts = np.bincount(flat, minlength=self.experts)
        src = torch.from_numpy(order // top).to(h.device)                        # the token of every pair, grouped
        pair_weight = weight.reshape(-1)
        xs = ops.gather_rows(h, src)
        ws = ops.gather_rows(pair_weight.reshape(-1, 1), torch.from_numpy(order).to(h.device)).reshape(-1)
        out = torch.zeros((h.shape[0], self.hidden), dtype=torch.float32, device=h.device)
        at = 0
        for e in range(self.experts):
            n = int(counts[e])
            if n:
                y = self.expert_down[e](self._mid(e, xs[at:at + n]))
                ops.scatter_add(out, y, src[at:at + n], ws[at:at + n])
                at += n
        return out


@register_part("feed_forward", "routed_gated_silu")
class RoutedGatedSiluFeedForward(RoutedExperts):
    capturable = True            # steps of up to DIRECT_ROWS rows plan nothing on the host; longer ones are never recorded

    def __init__(self, spec, builder):
        p = spec.params
        self.top = int(p["top"])
        E = int(p["num_experts"])
        if not 1 <= self.top <= E:
            raise ValueError(f"routed feed-forward: {self.top} of {E} experts a token")
        self.router = Linear(builder.tensor(spec, "router"), builder.tensor(spec, "router_bias") if "router_bias" in spec.tensors else None)
        if self.router.weight.shape != (E, int(p["hidden_size"])):
            raise ValueError(f"routed feed-forward: router {tuple(self.router.weight.shape)} does not fit {E} experts")
        self._set_experts(builder.tensor(spec, "gate_up"), builder.tensor(spec, "down"), E, int(p["intermediate_size"]), int(p["hidden_size"]),
                          "gated_silu")
        self.gate_up, self.down = self.first, self.down_all
        self.expert_gate_up = self.expert_first

    def forward(self, h, ctx):
        h = as_tensor(h)
        chosen, weight = ops.moe_route(self.router(h, out_dtype=torch.float32), self.top)
        return self.run_experts(h, chosen, weight)


@register_part("feed_forward", "routed_scored")
class RoutedScoredFeedForward(RoutedExperts):
    capturable = True

    def __init__(self, spec, builder):
        p = spec.params
        W, E = int(p["hidden_size"]), int(p["num_experts"])
        self.top, self.scale = int(p["top"]), float(p.get("scale", 1.0))
        self.groups, self.keep = int(p.get("groups") or 1), int(p.get("keep") or 1)
        if not 1 <= self.top <= E or E % self.groups or not 1 <= self.keep <= self.groups or self.keep * (E // self.groups) < self.top:
            raise ValueError(f"routed feed-forward: {self.top} of {E} experts a token, from {self.keep} of {self.groups} groups")
        self.shared = int(p["shared_size"]) if p.get("shared_size") else None
        self.router = Linear(builder.tensor(spec, "router"))          # the experts' rows, then the shared expert's gate row
        if self.router.weight.shape != (E + (1 if self.shared else 0), W):
            raise ValueError(f"routed feed-forward: router {tuple(self.router.weight.shape)} does not fit {E} experts"
                             + (" and a shared expert's gate" if self.shared else ""))
        self.correction = builder.tensor(spec, "correction") if "correction" in spec.tensors else None
        self._set_experts(builder.tensor(spec, "up"), builder.tensor(spec, "down"), E, int(p["intermediate_size"]), W, "gelu")
        if self.shared:
            self.shared_up, self.shared_down = Linear(builder.tensor(spec, "shared_up")), Linear(builder.tensor(spec, "shared_down"))
            if self.shared_up.weight.shape != (self.shared, W) or self.shared_down.weight.shape != (W, self.shared):
                raise ValueError(f"routed feed-forward: the shared expert's weights {tuple(self.shared_up.weight.shape)}, "
                                 f"{tuple(self.shared_down.weight.shape)} do not fit inner size {self.shared} over hidden {W}")

    def forward(self, h, ctx):
        h = as_tensor(h)
        logits = self.router(h, out_dtype=torch.float32)
        chosen, weight = ops.moe_route_scored(logits, self.experts, self.top, self.correction, self.groups, self.keep, self.scale)
        out = self.run_experts(h, chosen, weight)
        if self.shared:
            y = self.shared_down(ops.activation(self.shared_up(h), "gelu_erf"))
            ops.add_gated_rows(out, y, logits, self.experts)
        return out
