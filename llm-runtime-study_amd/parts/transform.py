"""Parts of the role "transform": they work in place on float32 rows, the residual stream right after the embedding or
the logits (see parts/base.py)."""

from __future__ import annotations

import math

from ..kernels import ops
from .base import Part, TensorSpec, register


class SoftCap(Part):
    """x = cap * tanh(x / cap): keeps every value within (-cap, cap), close to the identity for small ones."""

    graph_safe = True
    plan_safe = True

    def __init__(self, cap: float):
        if not cap > 0:
            raise ValueError(f"cap must be positive, got {cap}")
        self.cap = float(cap)

    def flops(self, tokens, pairs):
        return 0.0

    def forward(self, ctx, x):
        ops.soft_cap(x, self.cap)


register("transform", "soft_cap", SoftCap)


class Scale(Part):
    """x *= factor: logits times a constant of the model."""

    graph_safe = True
    plan_safe = True

    def __init__(self, factor: float):
        if not math.isfinite(factor):
            raise ValueError(f"factor must be finite, got {factor}")
        self.factor = float(factor)

    def flops(self, tokens, pairs):
        return 0.0

    def forward(self, ctx, x):
        ops.scale_values(x, self.factor)


register("transform", "scale", Scale)


class LearnedPositions(Part):
    """x[t] += table[position of t]: a learned vector per position, added to the stream after the embedding (unscaled).  `rows`
    is how many positions the table holds; -1 leaves it to the checkpoint."""

    graph_safe = True
    plan_safe = True

    def __init__(self, rows: int, size: int):
        if size <= 0 or (rows <= 0 and rows != -1):
            raise ValueError(f"rows and size must be positive (rows may be -1: as the checkpoint has it), got {rows} and {size}")
        self.rows, self.size = rows, size
        self.table = None

    def tensors(self):
        return {"weight": TensorSpec((self.rows, self.size), role="embedding")}

    def bind(self, weights, dtype):
        self.table = weights["weight"].to(dtype).contiguous()
        self.rows = self.table.shape[0]

    def flops(self, tokens, pairs):
        return 0.0

    def forward(self, ctx, x):
        ops.add_gathered(x, self.table, ctx.positions)


register("transform", "learned_positions", LearnedPositions)
