"""Softmax attention over the cache with a sink, an optional window and an optional gate, and with key and value sizes
of their own.

One joined product makes q | k | v (| gate).  ``qkv_bias`` (float32 over q | k | v) is added where the sums are still
32-bit.  q and k are normed as ``qk_norm`` says ("projection": one RMS norm over the whole q row, all heads at once, and
one over the whole k row, with plain weights of those sizes; "head": per head with one weight vector of the key size for
all heads; None), then the first ``rotary_dim`` dimensions of every head are rotated.  Query head h reads key/value head
h // (heads / kv_heads); a query at position p sees the keys max(0, p - window + 1) .. p.  With ``sink`` the softmax has
one more term in its denominator, exp(sink_score), that belongs to no value:

    p_j = exp(s_j) / (exp(sink_score) + sum_i exp(s_i)),      s_j = scale * q . k_j

The joined heads are multiplied by sigmoid of the gate rows (``gate`` "sigmoid") before the output projection.  Scores,
weights and sums are 32-bit in both modes.
"""
from __future__ import annotations

from ..cache import KVNeed
from ..kernels import ops
from .base import register_part
from .linear import Linear

QK_NORMS = (None, "projection", "head")
GATES = (None, "sigmoid")


@register_part("mixer", "sink_attention")
class SinkAttention:
    capturable = True

    def __init__(self, spec, builder):
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.nh, self.nkv = int(p["num_heads"]), int(p["num_kv_heads"])
        self.dk, self.dv = int(p["key_dim"]), int(p["value_dim"])
        self.scale, self.eps = float(p["scale"]), float(p.get("eps", 1e-6))
        self.window = int(p["window"]) if p.get("window") else None
        self.sink = float(p.get("sink_score", 0.0)) if p.get("sink") else None
        self.qk_norm, self.gate = p.get("qk_norm"), p.get("gate")
        if self.qk_norm not in QK_NORMS or self.gate not in GATES:
            raise ValueError(f"sink attention: qk_norm {self.qk_norm!r} is one of {QK_NORMS}, gate {self.gate!r} one of {GATES}")
        if self.nh % self.nkv:
            raise ValueError(f"{self.nh} heads are not a multiple of {self.nkv} kv heads")
        # the joined product is this part's own, or a wider one that the mixers beside it share (``input`` "shared")
        self.shared_input = p.get("input") == "shared"
        self.qkvg = None if self.shared_input else Linear(builder.tensor(spec, "qkvg"))
        self.out = Linear(builder.tensor(spec, "out"))
        self.bias = builder.tensor(spec, "qkv_bias") if "qkv_bias" in spec.tensors else None
        self.gate_off = self.nh * self.dk + self.nkv * (self.dk + self.dv)
        self.in_rows = self.gate_off + (self.nh * self.dv if self.gate else 0)
        if self.qkvg is not None and self.qkvg.weight.shape != (self.in_rows, self.hidden):
            raise ValueError(f"sink attention: joined weight {tuple(self.qkvg.weight.shape)} does not fit {self.nh} heads and {self.nkv} kv "
                             f"heads of key size {self.dk} and value size {self.dv} over hidden {self.hidden}")
        if self.out.weight.shape != (self.hidden, self.nh * self.dv):
            raise ValueError(f"sink attention: output weight {tuple(self.out.weight.shape)} does not fit")
        self.q_w = builder.tensor(spec, "q_norm") if self.qk_norm else None
        self.k_w = builder.tensor(spec, "k_norm") if self.qk_norm else None
        self.position = builder.build(spec.parts["position"]) if "position" in spec.parts else None
        if self.position is not None and (self.position.pairing != "half_split" or self.position.rotary_dim > self.dk):
            raise ValueError("sink attention: the rotation pairs dimension i with i + rotary_dim/2 within the key size")
        self.dtype = builder.dtype

    @staticmethod
    def cache_needs(spec):
        p = spec.params
        return [KVNeed(int(p["num_kv_heads"]), int(p["key_dim"]), int(p["window"]) if p.get("window") else None,
                       value_dim=int(p["value_dim"]))]

    def forward(self, h, ctx):
        if self.qkvg is None:
            raise RuntimeError("sink attention whose input product is shared gets its rows from the part that makes them")
        return self.forward_rows(self.qkvg(h), 0, ctx)

    def forward_rows(self, rows, col0, ctx):
        """``rows`` [n, >= col0 + in_rows]: q | k | v (| gate) from column ``col0``."""
        lc = ctx.layer_cache
        if lc is None or lc.kv is None:
            raise RuntimeError("sink attention needs the keys and values of its layer; the step gave it no cache")
        tables = self.position.tables(ctx) if self.position is not None else None
        cos, sin = tables if tables is not None else (None, None)
        rot = self.position.rotary_dim if tables is not None else 0
        table = lc.kv.table_dev
        q = ops.sink_qkv_store(rows, self.nh, self.nkv, self.dk, self.dv, self.bias, self.qk_norm, self.q_w, self.k_w, self.eps,
                               cos, sin, rot, lc.k, lc.v, table, ctx, write_cache=lc.writes, col0=col0)
        o = ops.sink_attention(q, lc.k, lc.v, table, ctx, self.nh, self.nkv, self.dk, self.dv, self.scale, self.window, self.sink,
                               rows if self.gate else None, col0 + self.gate_off)
        return self.out(o)
