"""A matrix memory with an input gate and a forget gate per head and token (the mLSTM of xLSTM).

Per head, with q_t, k_t of size ``key_dim`` (q times ``query_scale``) and v_t of size ``value_dim``, and the two gate rows
a_t, b_t (a projection plus a bias, one number per head each):

    i_t = cap tanh(a_t / cap)                        f_t = logsigmoid(cap tanh(b_t / cap))
    m_t = max(f_t + m_(t-1), i_t)                    (m before the first token is 0)
    S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T,      n_t likewise with k_t alone
    o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)

Each head's o_t is divided by its root mean square (``eps`` inside the root); the joined heads are multiplied by the weight
``norm`` and by the sigmoid of a gate projection, and projected back.  One joined product makes q | k | v | gate; the two
gates' rows come from a product of their own whose result stays 32-bit.  S, n and m are float32 and kept per sequence
(``StateNeed``); everything in the recurrence is 32-bit whatever the run's type.
"""
from __future__ import annotations

import torch

from ..cache import StateNeed
from ..kernels import ops
from .base import register_part
from .linear import Linear


@register_part("mixer", "mlstm")
class MatrixMemory:
    capturable = True

    def __init__(self, spec, builder):
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.nh, self.dk, self.dv = int(p["num_heads"]), int(p["key_dim"]), int(p["value_dim"])
        self.cap, self.eps, self.q_scale = float(p["gate_cap"]), float(p["eps"]), float(p["query_scale"])
        if not self.cap > 0:
            raise ValueError(f"mlstm: the gates' cap {self.cap} must be positive")
        self.qkvg = Linear(builder.tensor(spec, "qkvg"))
        self.gates = Linear(builder.tensor(spec, "gates"))
        self.gate_bias = builder.tensor(spec, "gate_bias") if "gate_bias" in spec.tensors else None
        self.norm_weight = builder.tensor(spec, "norm")
        self.out = Linear(builder.tensor(spec, "out"))
        in_rows = self.nh * 2 * (self.dk + self.dv)
        if self.qkvg.weight.shape != (in_rows, self.hidden) or self.gates.weight.shape != (2 * self.nh, self.hidden):
            raise ValueError(f"mlstm: joined weights {tuple(self.qkvg.weight.shape)} and {tuple(self.gates.weight.shape)} do not fit {self.nh} "
                             f"heads of key size {self.dk} and value size {self.dv} over hidden {self.hidden}")
        if self.out.weight.shape != (self.hidden, self.nh * self.dv):
            raise ValueError(f"mlstm: output weight {tuple(self.out.weight.shape)} does not fit")

    @staticmethod
    def cache_needs(spec):
        p = spec.params
        H, d, dv = int(p["num_heads"]), int(p["key_dim"]), int(p["value_dim"])
        # the memory with the normalizer as one more value column, and the running maximum
        return [StateNeed("mlstm", (H, d, dv + 1)), StateNeed("mlstm_max", (H,))]

    def forward(self, h, ctx):
        lc = ctx.layer_cache
        if lc is None or not lc.states or "mlstm" not in lc.states:
            raise RuntimeError("the matrix memory needs its state; the step gave it no cache")
        rows = self.qkvg(h)
        gates = self.gates(h, out_dtype=torch.float32)
        o = ops.mlstm(rows, gates, self.gate_bias, self.nh, self.dk, self.dv, self.cap, self.q_scale, self.norm_weight, self.eps,
                      lc.states["mlstm"], lc.states["mlstm_max"], ctx)
        return self.out(o)
