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

Further options: ``sink`` "learned": the sink's score is a number per head (tensor ``sink_scores``).  ``gate``
"head_sigmoid": one gate value for each head instead of one for each value.  ``conv_taps`` with the tensor ``conv``
(float32 [channels of q | k | v, taps]): right after the bias every channel of q, k and v goes through a short causal
convolution over time; the last taps - 1 inputs of each sequence are a state of the part.  The position part's ``pairing``
may be "interleaved" (dimension 2i with 2i + 1).  ``kv`` "borrowed": the part has no key and value projections (and no
biases, convolutions or norms of them); its run-order entry reads the keys and values that another entry wrote
(``cache_of``), with its own queries, window, sink and gate, and keeps only its own convolution's state.  ``storage_window``:
the window by which the keys and values are kept if other entries read them with a longer one (None: every position).
"""
from __future__ import annotations

from ..cache import KVNeed, StateNeed
from ..kernels import ops
from .base import register_part
from .linear import Linear

QK_NORMS = (None, "projection", "head")
GATES = (None, "sigmoid", "head_sigmoid")


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
        if p.get("sink") == "learned":
            self.sink = builder.tensor(spec, "sink_scores")
            if self.sink.shape != (self.nh,):
                raise ValueError(f"sink attention: {self.nh} heads have learned sink scores of shape {tuple(self.sink.shape)}")
        self.qk_norm, self.gate = p.get("qk_norm"), p.get("gate")
        self.borrows = p.get("kv", "own") == "borrowed"
        if p.get("kv", "own") not in ("own", "borrowed"):
            raise ValueError(f"sink attention: kv {p.get('kv')!r} is neither 'own' nor 'borrowed'")
        if self.borrows and self.qk_norm == "projection":
            raise ValueError("sink attention: borrowed keys come normed by their own layer; a norm over this layer's k projection has nothing to norm")
        if self.qk_norm not in QK_NORMS or self.gate not in GATES:
            raise ValueError(f"sink attention: qk_norm {self.qk_norm!r} is one of {QK_NORMS}, gate {self.gate!r} one of {GATES}")
        if self.nh % self.nkv:
            raise ValueError(f"{self.nh} heads are not a multiple of {self.nkv} kv heads")
        # the joined product is this part's own, or a wider one that the mixers beside it share (``input`` "shared")
        self.shared_input = p.get("input") == "shared"
        self.qkvg = None if self.shared_input else Linear(builder.tensor(spec, "qkvg"))
        self.out = Linear(builder.tensor(spec, "out"))
        self.bias = builder.tensor(spec, "qkv_bias") if "qkv_bias" in spec.tensors else None
        self.head_gate = self.gate == "head_sigmoid"
        self.channels = self.nh * self.dk + (0 if self.borrows else self.nkv * (self.dk + self.dv))      # of q | k | v
        self.gate_off = self.channels
        self.in_rows = self.gate_off + (0 if not self.gate else self.nh if self.head_gate else self.nh * self.dv)
        self.taps = int(p.get("conv_taps") or 0)
        self.conv = builder.tensor(spec, "conv") if self.taps else None
        if self.conv is not None and self.conv.shape != (self.channels, self.taps):
            raise ValueError(f"sink attention: the convolution {tuple(self.conv.shape)} is not [{self.channels}, {self.taps}]")
        if self.qkvg is not None and self.qkvg.weight.shape != (self.in_rows, self.hidden):
            raise ValueError(f"sink attention: joined weight {tuple(self.qkvg.weight.shape)} does not fit {self.nh} heads and {self.nkv} kv "
                             f"heads of key size {self.dk} and value size {self.dv} over hidden {self.hidden}")
        if self.out.weight.shape != (self.hidden, self.nh * self.dv):
            raise ValueError(f"sink attention: output weight {tuple(self.out.weight.shape)} does not fit")
        self.q_w = builder.tensor(spec, "q_norm") if self.qk_norm else None
        self.k_w = builder.tensor(spec, "k_norm") if self.qk_norm and not self.borrows else self.q_w
        self.position = builder.build(spec.parts["position"]) if "position" in spec.parts else None
        if self.position is not None and self.position.rotary_dim > self.dk:
            raise ValueError("sink attention: the rotation lies within the key size")
        if self.bias is not None and self.bias.shape != (self.channels,):
            raise ValueError(f"sink attention: the bias {tuple(self.bias.shape)} is not [{self.channels}]")
        self.dtype = builder.dtype

    @staticmethod
    def _conv_need(spec):
        p = spec.params
        taps = int(p.get("conv_taps") or 0)
        if taps <= 1:
            return []
        channels = int(p["num_heads"]) * int(p["key_dim"])
        if p.get("kv", "own") != "borrowed":
            channels += int(p["num_kv_heads"]) * (int(p["key_dim"]) + int(p["value_dim"]))
        return [StateNeed("conv", (taps - 1, channels))]

    @staticmethod
    def cache_needs(spec):
        p = spec.params
        if p.get("kv", "own") == "borrowed":
            raise ValueError("sink attention that borrows keys and values runs as an entry that reads another entry's cache")
        window = int(p["window"]) if p.get("window") else None
        if "storage_window" in p:                       # others read these keys, by windows of their own
            window = int(p["storage_window"]) if p["storage_window"] else None
        return [KVNeed(int(p["num_kv_heads"]), int(p["key_dim"]), window, value_dim=int(p["value_dim"]))] + SinkAttention._conv_need(spec)

    @staticmethod
    def cache_needs_beside_shared(spec):
        return SinkAttention._conv_need(spec)

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
        if self.borrows == lc.writes:
            raise RuntimeError("sink attention: a part with key and value projections writes its own cache, one without reads another entry's")
        state = None
        if self.taps > 1:
            if not lc.states or "conv" not in lc.states:
                raise RuntimeError("sink attention with a convolution needs its state; the step gave it none")
            state = lc.states["conv"]
        pairing = self.position.pairing if self.position is not None else "half_split"
        q = ops.sink_qkv_store(rows, self.nh, self.nkv, self.dk, self.dv, self.bias, self.qk_norm, self.q_w, self.k_w, self.eps,
                               cos, sin, rot, lc.k, lc.v, table, ctx, write_cache=not self.borrows, col0=col0, pairing=pairing,
                               conv=self.conv, conv_state=state)
        o = ops.sink_attention(q, lc.k, lc.v, table, ctx, self.nh, self.nkv, self.dk, self.dv, self.scale, self.window, self.sink,
                               rows if self.gate else None, col0 + self.gate_off, gate_per_head=self.head_gate)
        return self.out(o)
