"""Two (or more) mixers side by side: all read the same input, and their outputs are added with one fixed weight each.

The sum is not made here: ``forward`` returns a ``WeightedSum`` (parts/residual.py), and the block adds its terms to the
residual stream in the 32-bit pass that it runs anyway.  Every side keeps what it needs per sequence; together they must
not ask twice for the same kind of storage under one name.
"""
from __future__ import annotations

from .base import cache_needs, register_part
from .residual import WeightedSum, as_tensor


@register_part("mixer", "parallel")
class ParallelMixers:
    def __init__(self, spec, builder):
        self.sides = [builder.build(s) for s in spec.parts.values()]
        self.weights = [float(w) for w in spec.params["weights"]]
        if len(self.weights) != len(self.sides) or not self.sides:
            raise ValueError(f"parallel mixers: {len(self.weights)} weights for {len(self.sides)} sides")

    @property
    def capturable(self) -> bool:
        return all(getattr(s, "capturable", False) for s in self.sides)

    @staticmethod
    def cache_needs(spec):
        out = []
        for side in spec.parts.values():
            out += cache_needs(side)
        return out

    def forward(self, h, ctx):
        h = as_tensor(h)
        return WeightedSum([side.forward(h, ctx) for side in self.sides], list(self.weights))
