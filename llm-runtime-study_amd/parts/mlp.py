"""Feed-forwards.  SwiGLU: down(silu(gate(x)) * up(x)), three bias-free projections (with `activation="clamped"` the gated
activation is g * sigmoid(alpha g) * (u + 1), g = min(gate(x), limit), u = clamp(up(x), -limit, limit)); DenseMLP (at the end of the file):
down(act(up(x))), two bias-free projections with an activation between them.

Reference mini_llm/nn/mlp.py:80-87.  gate and up are stacked into one [2I, H] matrix when
the weights are bound, so one product feeds the gated activation; the down projection adds
straight into the float32 residual stream (or, with `accumulate=False`, stores into the float32 rows it is given).
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, TensorSpec, register
from .linear import linear, rows_of


class SwiGLU(Part):
    graph_safe = True  # launches only library kernels on arena buffers
    plan_safe = True
    takes_lazy_norm = True
    begins_next_norm = True
    can_overwrite = True        # forward(..., accumulate=False) stores its output

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu", alpha: float = 1.702, limit: float | None = None):
        if hidden_size <= 0 or intermediate_size <= 0:
            raise ValueError("hidden_size and intermediate_size must be positive")
        if activation not in ("silu", "clamped"):
            raise ValueError(f"unknown gated activation {activation!r}; known: silu, clamped")
        if activation == "clamped" and (limit is None or not limit > 0):
            raise ValueError(f"the clamped activation needs a positive limit, got {limit}")
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        # "clamped": down(g * sigmoid(alpha g) * (u + 1)) with g = min(gate(x), limit), u = clamp(up(x), -limit, limit)
        self.clamped = None if activation == "silu" else (float(alpha), float(limit))
        self.gate_up = self.down = None

    def tensors(self):
        h, i = self.hidden_size, self.intermediate_size
        return {
            "gate_proj.weight": TensorSpec((i, h)),
            "up_proj.weight": TensorSpec((i, h)),
            "down_proj.weight": TensorSpec((h, i)),
        }

    def bind(self, weights, dtype):
        gate, up = weights["gate_proj.weight"].to(dtype), weights["up_proj.weight"].to(dtype)
        h, i = self.hidden_size, self.intermediate_size
        # bfloat16: rows interleaved in groups of 8 (8 gate rows, then the 8 up rows of the same
        # features), so that the product's epilogue has both halves of a feature and writes
        # silu(gate) * up itself; otherwise gate rows then up rows and a separate activation kernel
        self.interleaved = dtype == torch.bfloat16 and i % 8 == 0 and h % 8 == 0 and self.clamped is None
        if self.interleaved:
            self.gate_up = torch.stack((gate.view(i // 8, 8, h), up.view(i // 8, 8, h)), 1).reshape(2 * i, h).contiguous()
        else:
            self.gate_up = torch.cat((gate, up), 0).contiguous()
        self.down = weights["down_proj.weight"].to(dtype).contiguous()

    def weight_bytes(self):
        return (self.gate_up.numel() + self.down.numel()) * self.down.element_size()

    def forward(self, ctx, x, residual, then_norm=None, accumulate: bool = True):
        t = rows_of(x)
        act = ctx.scratch("ffn_act", (t, self.intermediate_size), ctx.dtype)
        if self.interleaved:
            linear(ctx, act, x, self.gate_up, swiglu=True)
        else:
            gate_up = ctx.scratch("ffn_gate_up", (t, 2 * self.intermediate_size), ctx.dtype)
            linear(ctx, gate_up, x, self.gate_up)
            if self.clamped is not None:
                ops.gated_clamped(act, gate_up, *self.clamped)
            else:
                ops.silu_mul(act, gate_up)
        return linear(ctx, residual, act, self.down, accumulate=accumulate, then_norm=then_norm)


register("feed_forward", "swiglu", SwiGLU)


class DenseMLP(Part):
    """down(act(up(x))): two bias-free projections, `activation` between them: "gelu" (the exact one, 0.5 z (1 + erf(z / sqrt 2))),
    "gelu_tanh", "silu" or "relu" (kernels/ops.py, ACTIVATIONS).  The down projection adds into the float32 rows it is given, or
    stores into them with `accumulate=False`."""

    graph_safe = True
    plan_safe = True
    can_overwrite = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "gelu"):
        if hidden_size <= 0 or intermediate_size <= 0:
            raise ValueError("hidden_size and intermediate_size must be positive")
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"unknown activation {activation!r}; known: {', '.join(ops.ACTIVATIONS)}")
        self.hidden_size, self.intermediate_size, self.activation = hidden_size, intermediate_size, activation
        self.up = self.down = None

    def tensors(self):
        return {"up_proj.weight": TensorSpec((self.intermediate_size, self.hidden_size)),
                "down_proj.weight": TensorSpec((self.hidden_size, self.intermediate_size))}

    def bind(self, weights, dtype):
        self.up = weights["up_proj.weight"].to(dtype).contiguous()
        self.down = weights["down_proj.weight"].to(dtype).contiguous()

    def weight_bytes(self):
        return (self.up.numel() + self.down.numel()) * self.down.element_size()

    def forward(self, ctx, x, residual, then_norm=None, accumulate: bool = True):
        t = rows_of(x)
        act = ctx.scratch("ffn_act", (t, self.intermediate_size), ctx.dtype)
        linear(ctx, act, x, self.up)
        ops.activation(act, act, self.activation)
        return linear(ctx, residual, act, self.down, accumulate=accumulate, then_norm=then_norm)


register("feed_forward", "dense_mlp", DenseMLP)
