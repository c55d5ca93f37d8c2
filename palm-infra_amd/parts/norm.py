"""RMSNorm: y = x * (1 / sqrt(mean(x^2) + eps)) * w, statistics in 32-bit (kernels/norm.cpp:13-31).
The residual add that precedes a norm in a block is fused into the same pass
(engine/cuda_ops.cu:140-170 has the same fusion).  With ``offset`` c the checkpoint stores w - c (a weight kept around
zero for c = 1): the sum is made once, in 32-bit, when the part is built."""
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
