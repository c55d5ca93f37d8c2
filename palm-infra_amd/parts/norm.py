"""RMSNorm: y = x * (1 / sqrt(mean(x^2) + eps)) * w, statistics in 32-bit (kernels/norm.cpp:13-31).
The residual add that precedes a norm in a block is fused into the same pass
(engine/cuda_ops.cu:140-170 has the same fusion).  With ``offset`` c the checkpoint stores w - c (a weight kept around
zero for c = 1): the sum is made once, in 32-bit, when the part is built.

``dyt`` (Dynamic Tanh): y = tanh(alpha x) w + b with one learned slope alpha, a weight and a bias over the width: no mean and
no variance, nothing crosses the columns.

``streams_in``: the reader of a residual stream that runs in several copies [n, S, width]: u = sum_s in[s] x_s (without the
tensor ``in``: the plain sum), then the norm it wraps.  The block that writes the streams hands its write to the reader that
comes next, so one pass writes one sublayer's output and norms the next one's input."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import register_part


@register_part("norm", "rms")
class RMSNorm:
    capturable = True      # launches the same kernels whatever the step holds: may be recorded into a HIP graph
    takes_planes = True    # ``delta`` may be float32 planes [P, n, width], added one after the other
    folds_into_products = True   # y = x * f(row) * weight, f = 1 / sqrt(mean(x^2) + eps): see parts/residual.py

    def __init__(self, spec, builder):
        self.width = int(spec.params["width"])
        self.eps = float(spec.params["eps"])
        self.weight = builder.tensor(spec, "weight")
        offset = float(spec.params.get("offset", 0.0))
        if offset:
            self.weight = self.weight + offset
        self.dtype = builder.dtype
        if self.weight.shape != (self.width,):
            raise ValueError(f"RMSNorm of width {self.width} got a weight of shape {tuple(self.weight.shape)}")

    def __call__(self, x: torch.Tensor, delta: torch.Tensor | None = None, update: bool = False,
                 rows: torch.Tensor | None = None, out_dtype: torch.dtype | None = None) -> torch.Tensor:
        return ops.rmsnorm(x, self.weight, self.eps, out_dtype or self.dtype, delta=delta, update_x=update, rows=rows)

    @property
    def stream_norm(self):
        """How the pass over several streams applies this norm itself: (kind, weight, bias, slope, eps)."""
        return ("rms", self.weight, None, 1.0, self.eps)


@register_part("norm", "dyt")
class DynamicTanh:
    capturable = True

    def __init__(self, spec, builder):
        self.width = int(spec.params["width"])
        self.eps = float(spec.params.get("eps", 0.0))            # kept for whoever asks; the norm itself has no use for it
        self.weight = builder.tensor(spec, "weight")
        self.bias = builder.tensor(spec, "bias") if "bias" in spec.tensors else None
        self.alpha = float(builder.tensor(spec, "alpha").to(torch.float32).reshape(-1)[0].item()) if "alpha" in spec.tensors \
            else float(spec.params.get("alpha", 1.0))
        self.dtype = builder.dtype
        for v in (self.weight, self.bias):
            if v is not None and v.shape != (self.width,):
                raise ValueError(f"a tanh norm of width {self.width} got a vector of shape {tuple(v.shape)}")
        self._one = None

    @property
    def stream_norm(self):
        return ("dyt", self.weight, self.bias, self.alpha, self.eps)

    def __call__(self, x: torch.Tensor, delta: torch.Tensor | None = None, update: bool = False,
                 rows: torch.Tensor | None = None, out_dtype: torch.dtype | None = None) -> torch.Tensor:
        """x float32 [n, width]: one stream.  ``delta`` [n, width] is added first (with ``update`` the sum is written back)."""
        xs = x.view(x.shape[0], 1, x.shape[1])
        y = mix = out_w = None
        if delta is not None:
            if delta.dim() != 2:
                raise ValueError("a tanh norm adds one branch output, not planes of partial sums")
            if rows is None and not update:
                xs = xs.clone()
            if self._one is None:
                self._one = torch.ones((1, 1), dtype=torch.float32, device=x.device)
            y, mix, out_w = delta, self._one, self._one[0]
        return ops.streams_mix_norm(xs, y, mix, out_w, None, "dyt", self.weight, self.bias, self.alpha, self.eps, rows=rows,
                                    out_dtype=out_dtype or self.dtype)


@register_part("norm", "streams_in")
class StreamsReader:
    capturable = True

    def __init__(self, spec, builder):
        self.streams = int(spec.params["streams"])
        self.inner = builder.build(spec.parts["norm"])
        self.in_w = builder.tensor(spec, "in") if "in" in spec.tensors else None
        self.width, self.eps, self.dtype = self.inner.width, self.inner.eps, builder.dtype
        if self.in_w is not None and self.in_w.shape != (self.streams,):
            raise ValueError(f"a reader of {self.streams} streams got weights of shape {tuple(self.in_w.shape)}")
        if not getattr(self.inner, "capturable", False):
            self.capturable = False

    def _streams(self, x: torch.Tensor) -> torch.Tensor:
        xs = x.view(x.shape[0], 1, x.shape[1]) if x.dim() == 2 else x
        if xs.dim() != 3 or xs.shape[1] != self.streams or xs.shape[2] != self.width:
            raise ValueError(f"a reader of {self.streams} streams of width {self.width} got a stream of shape {tuple(x.shape)}")
        return xs

    def read(self, x: torch.Tensor, y=None, mix=None, out_w=None, rows=None, out_dtype=None) -> torch.Tensor:
        """What this reader makes of the streams after the sublayer output ``y`` has been written into them with ``mix`` and
        ``out_w`` (y None: of the streams as they are).  With ``rows`` the streams stay as they are."""
        xs, out_dtype = self._streams(x), out_dtype or self.dtype
        fused = getattr(self.inner, "stream_norm", None)
        if fused is not None:
            kind, w, b, alpha, eps = fused
            return ops.streams_mix_norm(xs, y, mix, out_w, self.in_w, kind, w, b, alpha, eps, rows=rows, out_dtype=out_dtype)
        u = ops.streams_mix_norm(xs, y, mix, out_w, self.in_w, None, rows=rows, out_dtype=torch.float32)
        return self.inner(u, out_dtype=out_dtype)

    def __call__(self, x: torch.Tensor, delta: torch.Tensor | None = None, update: bool = False,
                 rows: torch.Tensor | None = None, out_dtype: torch.dtype | None = None) -> torch.Tensor:
        if delta is not None:
            raise ValueError("a branch output goes into several streams with the weights of its block, not through the reader")
        return self.read(x, rows=rows, out_dtype=out_dtype)


@register_part("norm", "none")
class PassThrough:
    """No norm at all, for blocks whose branches read the residual stream itself: the rows (plus ``delta``) in the
    activation type.  In the float32 mode, without a delta or a row selection, that is the stream itself."""
    capturable = True
    passes_through = True

    def __init__(self, spec=None, builder=None, dtype: torch.dtype | None = None):
        self.dtype = dtype if dtype is not None else builder.dtype

    def __call__(self, x: torch.Tensor, delta: torch.Tensor | None = None, update: bool = False,
                 rows: torch.Tensor | None = None, out_dtype: torch.dtype | None = None) -> torch.Tensor:
        out_dtype = out_dtype or self.dtype
        if delta is not None:
            if delta.dim() == 3:
                delta = delta.sum(0)
            total = x + delta.to(torch.float32)
            if update:
                x.copy_(total)
            x = total
        if rows is not None:
            x = x.index_select(0, rows.long())
        if out_dtype == x.dtype:
            return x
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        ops.convert_into(x, out)
        return out
