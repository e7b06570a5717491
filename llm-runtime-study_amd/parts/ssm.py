"""Selective state space mixer: a recurrence whose memory is one matrix per head, written by outer products and read by a vector.

For a token with input x, inner = heads * value_dim, N = state_size, per head h (group h // (heads / groups)):
    [z | u | B | C | dt] = W_in x            z, u: inner; B, C: groups * N; dt: heads
    u, B, C = silu(conv([u | B | C]))        a causal convolution over time per channel, a few taps, with a bias, zeros before the start
    dt      = softplus(dt + dt_bias)
    S <- exp(-exp(A_log_h) dt) S + dt B u^T  S [N, value_dim], zero at a sequence's start
    y       = S^T C + D_h u
    out     = W_o (part_rms_norm(y * silu(z)) * norm_weight)      the norm in `norm_parts` equal parts of inner, each by its own
                                                                  root mean square; the gate comes before the norm
Step sizes, decays, the state and the read-out with its gated norm are float32 in every run; the input projection is written
in float32 too.

The recurrence is the scan of the gated delta rule's kernels without its correction (csrc/delta.hip, RULE_PLAIN) with B as the
keys, C as the queries and dt u as the values, so a request's state row has the same form: every head's S in the order the
scan's threads hold it, then the convolution's last taps - 1 inputs of every channel (`StateNeed`).
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, StateNeed, TensorSpec, register
from .linear import linear, materialize, rows_of


class StateSpace(Part):
    graph_safe = True
    plan_safe = True
    can_overwrite = True

    def __init__(self, hidden_size: int, num_heads: int, num_groups: int, state_size: int, value_dim: int, conv_taps: int, norm_parts: int,
                 norm_eps: float, conv_bias: bool = True):
        for name, value in (("hidden_size", hidden_size), ("num_heads", num_heads), ("num_groups", num_groups), ("state_size", state_size),
                            ("value_dim", value_dim), ("conv_taps", conv_taps), ("norm_parts", norm_parts)):
            if value <= 0:
                raise ValueError(f"{name} must be positive, got {value}")
        if num_heads % num_groups != 0:
            raise ValueError(f"num_heads must be divisible by num_groups, got {num_heads} and {num_groups}")
        if (num_heads * value_dim) % norm_parts != 0:
            raise ValueError(f"the {num_heads * value_dim} inner values do not divide into {norm_parts} parts")
        if state_size > 256:
            raise ValueError(f"the scan kernel takes state_size up to 256, got {state_size}")
        if norm_eps <= 0:
            raise ValueError(f"norm_eps must be positive, got {norm_eps}")
        self.hidden_size, self.num_heads, self.num_groups, self.state_size = hidden_size, num_heads, num_groups, state_size
        self.value_dim, self.conv_taps, self.norm_parts, self.norm_eps, self.has_conv_bias = value_dim, conv_taps, norm_parts, norm_eps, conv_bias
        self.inner = num_heads * value_dim
        self.channels = self.inner + 2 * num_groups * state_size           # what passes the convolution: u, B, C
        self.columns = self.inner + self.channels + num_heads               # ... with z in front and dt behind
        self.w_in = self.w_o = self.conv = self.conv_bias = self.a_log = self.dt_bias = self.skip = self.norm = None

    def tensors(self):
        specs = {"in_proj.weight": TensorSpec((self.columns, self.hidden_size)),
                 "conv.weight": TensorSpec((self.channels, self.conv_taps)),
                 "dt_bias": TensorSpec((self.num_heads,), role="bias"),
                 "A_log": TensorSpec((self.num_heads,), role="bias"),
                 "D": TensorSpec((self.num_heads,), role="norm"),
                 "norm.weight": TensorSpec((self.inner,), role="norm"),
                 "o_proj.weight": TensorSpec((self.hidden_size, self.inner))}
        if self.has_conv_bias:
            specs["conv.bias"] = TensorSpec((self.channels,), role="bias")
        return specs

    def bind(self, weights, dtype):
        stacked = weights["in_proj.weight"].to(dtype)
        pad = -stacked.shape[0] % 16          # whole groups of 16 output columns suit every product kernel
        if pad:
            stacked = torch.cat((stacked, stacked.new_zeros(pad, self.hidden_size)), 0)
        self.w_in = stacked.contiguous()
        self.conv = weights["conv.weight"].float().contiguous()
        self.conv_bias = weights["conv.bias"].float().contiguous() if self.has_conv_bias else None
        self.a_log, self.dt_bias = weights["A_log"].float().contiguous(), weights["dt_bias"].float().contiguous()
        self.skip, self.norm = weights["D"].float().contiguous(), weights["norm.weight"].float().contiguous()
        self.w_o = weights["o_proj.weight"].to(dtype).contiguous()

    def weight_bytes(self):
        return (self.w_in.numel() + self.w_o.numel()) * self.w_o.element_size()

    def flops(self, tokens, pairs):
        # the projections, and per token and head the state's update and its read-out
        return super().flops(tokens, pairs) + 4.0 * tokens * self.num_heads * self.state_size * self.value_dim

    def state_floats(self) -> int:
        return ops.delta_state_floats(self.num_heads, self.num_groups, self.state_size, self.value_dim, self.conv_taps)

    def cache_need(self):
        return StateNeed((self.state_floats(),), torch.float32)

    def forward(self, ctx, x, residual, cache, then_norm=None, accumulate: bool = True):
        if cache is None or cache.state is None:
            raise ValueError("the state space mixer needs a state row per request")
        t = rows_of(x)
        x = materialize(ctx, x)
        proj = ctx.scratch("ssm_proj", (t, self.w_in.shape[0]), torch.float32)
        linear(ctx, proj, x, self.w_in)
        out = ctx.scratch("ssm_out", (t, self.inner), ctx.dtype)
        qkv = ctx.scratch("ssm_cbv", (t, self.channels), torch.float32)
        gates = ctx.scratch("ssm_gates", (t, 2 * self.num_heads), torch.float32)
        raw = ctx.scratch("ssm_read_out", (t, self.inner), torch.float32)
        skipped = ctx.scratch("ssm_skip", (t, self.inner), torch.float32)
        ops.state_space(out, proj, cache.state, ctx.token_request, ctx.cu_seqlens_q, ctx.slot_ids, ctx.R, self.conv, self.conv_bias,
                        self.num_groups, self.num_heads, self.state_size, self.value_dim, self.a_log, self.dt_bias, self.skip, self.norm,
                        self.norm_parts, self.norm_eps, qkv, gates, raw, skipped)
        linear(ctx, residual, out, self.w_o, accumulate=accumulate)
        return None


register("mixer", "state_space", StateSpace)
