"""Two (or more) mixers side by side: all read the same input, and their outputs are added with one fixed weight each.

The sum is not made here: ``forward`` returns a ``WeightedSum`` (parts/residual.py), and the block adds its terms to the
residual stream in the 32-bit pass that it runs anyway.  Every side keeps what it needs per sequence; together they must
not ask twice for the same kind of storage under one name.

With a tensor ``in`` (the sides' input matrices joined along their rows, in the order of the sides) one product serves all
sides: each then takes its columns of the result (its description says ``input`` "shared" and names no input matrix of
its own).
"""
from __future__ import annotations

from .base import cache_needs, register_part
from .linear import Linear
from .residual import WeightedSum, as_tensor


@register_part("mixer", "parallel")
class ParallelMixers:
    def __init__(self, spec, builder):
        self.sides = [builder.build(s) for s in spec.parts.values()]
        self.weights = [float(w) for w in spec.params["weights"]]
        if len(self.weights) != len(self.sides) or not self.sides:
            raise ValueError(f"parallel mixers: {len(self.weights)} weights for {len(self.sides)} sides")
        self.shared = Linear(builder.tensor(spec, "in")) if "in" in spec.tensors else None
        if self.shared is not None:
            if not all(getattr(s, "shared_input", False) for s in self.sides):
                raise ValueError("parallel mixers: a shared input product needs sides that take their rows from it")
            if sum(s.in_rows for s in self.sides) != self.shared.out_features:
                raise ValueError(f"parallel mixers: the shared input product makes {self.shared.out_features} columns, the sides take "
                                 f"{[s.in_rows for s in self.sides]}")

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
        if self.shared is None:
            return WeightedSum([side.forward(h, ctx) for side in self.sides], list(self.weights))
        rows = self.shared(h)
        terms, col0 = [], 0
        for side in self.sides:
            terms.append(side.forward_rows(rows, col0, ctx))
            col0 += side.in_rows
        return WeightedSum(terms, list(self.weights))
