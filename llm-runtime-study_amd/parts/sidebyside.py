"""Two mixers side by side: both read the same input and the layer's mixer output is a weighted sum of theirs,
    out = left_scale * left(x) + right_scale * right(x).
Either may keep pages or a state of fixed size; what the pair keeps is both (`BothNeeds` when one keeps pages and the other a
state; the two then find theirs in the one LayerCache the entry owns).  Each mixer stores its output into a float32 buffer of
the step and one kernel adds the two up into the rows the pair was given.  Tensors are named `<left_name>.*` and `<right_name>.*`.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import BothNeeds, PagedKVNeed, Part, PartSpec, StateNeed, create, flops_of, register, under
from .linear import materialize


class SideBySide(Part):
    can_overwrite = True

    def __init__(self, left: PartSpec, right: PartSpec, left_scale: float = 1.0, right_scale: float = 1.0,
                 names: tuple = ("left", "right")):
        self.left, self.right = create("mixer", left), create("mixer", right)
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        self.names = tuple(names)
        for part in (self.left, self.right):
            if not getattr(part, "can_overwrite", False):
                raise ValueError(f"a mixer that runs beside another must store its output (accumulate=False): {type(part).__name__} cannot")
        needs = [part.cache_need() for part in (self.left, self.right)]
        paged = [need for need in needs if isinstance(need, PagedKVNeed)]
        states = [need for need in needs if isinstance(need, StateNeed)]
        if len(paged) > 1 or len(states) > 1 or len(paged) + len(states) != sum(need is not None for need in needs):
            raise ValueError("two mixers side by side may keep one set of pages and one state between them")
        self._need = BothNeeds(paged[0], states[0]) if paged and states else (paged or states or [None])[0]

    def _children(self):
        return list(zip(self.names, (self.left, self.right)))

    def tensors(self):
        return {f"{prefix}.{name}": spec for prefix, part in self._children() for name, spec in part.tensors().items()}

    def bind(self, weights, dtype):
        for prefix, part in self._children():
            part.bind(under(weights, prefix + "."), dtype)

    def weight_bytes(self):
        return sum(part.weight_bytes() for _, part in self._children())

    def flops(self, tokens, pairs):
        return sum(flops_of(part, tokens, pairs) for _, part in self._children())

    def cache_need(self):
        return self._need

    @property
    def graph_safe(self) -> bool:
        return all(getattr(part, "graph_safe", False) for _, part in self._children())

    @property
    def plan_safe(self) -> bool:
        return all(getattr(part, "plan_safe", False) for _, part in self._children())

    @property
    def wants_query_groups(self) -> bool:
        return any(getattr(part, "wants_query_groups", False) for _, part in self._children())

    def forward(self, ctx, x, residual, cache, then_norm=None, accumulate: bool = True):
        x = materialize(ctx, x)
        shape = tuple(residual.shape)
        left = ctx.scratch("side_left_out", shape, torch.float32)
        right = ctx.scratch("side_right_out", shape, torch.float32)
        self.left.forward(ctx, x, left, cache, accumulate=False)
        self.right.forward(ctx, x, right, cache, accumulate=False)
        if accumulate:
            ops.axpby(left, left, self.left_scale, right, self.right_scale)
            ops.axpby(residual, residual, 1.0, left, 1.0)
        else:
            ops.axpby(residual, left, self.left_scale, right, self.right_scale)
        return None


register("mixer", "side_by_side", SideBySide)
