"""Gated delta rule: a mixer whose memory is one matrix per head, updated token by token.

For a token with input x, per head h (key group h // (heads / kv_heads), as in grouped-query attention):
    q, k  = unit(silu(conv(W_q x))), unit(silu(conv(W_k x)))        q also times head_dim ** -0.5
    v     = silu(conv(W_v x))
    beta  = sigmoid(W_b x)                                           the step size
    g     = exp(-exp(A_log) * softplus(W_a x + dt_bias))             the decay
    S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q     S [head_dim, value_dim], zero at a sequence's start
    out   = W_o (rms_norm(o) * norm_weight * silu(W_g x))            the norm per head over value_dim
`conv` is a causal convolution over time, a few taps per channel, no bias, zeros before the sequence's start;
`unit(z) = z / sqrt(sum(z^2) + 1e-6)`.  The gates, the unit norms, the state and the read-out are float32 in
every run; the projections that feed them are written in float32 too.

`channel_decay` (with `decay_rank`, `gate_rank`): the decay is one number per head and key channel, multiplying the rows of S,
    g = exp(-exp(A_log_h) * softplus(W_a2 (W_a1 x) + dt_bias))  laid out heads x head_dim, dt_bias of that size,
and the output gate is sigmoid(W_g2 (W_g1 x)) laid out heads x value_dim; W_a1 and W_g1 are stacked behind q, k, v and the step
size.  The second matrices are applied in float32: as two products of their own, or, for ranks of at most UPS_IN_KERNEL_RANK (a
handful of multiply-adds an output cost less than two more launches), inside the recurrence's kernels.  A rank of None is read from
the checkpoint's tensors when they are bound.

All six input projections are one stacked product.  What a request keeps between steps is one float32 row: the
matrices of all heads, then the convolution's last taps - 1 inputs of every channel (`StateNeed`); the cache
manager hands out the rows, clears a row at admission and the kernels find a request's row by its slot.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, StateNeed, TensorSpec, register
from .linear import linear, materialize, rows_of

STATE_LANES = 16     # lanes that share a column of a head's matrix in the scan kernel


def state_rows(head_dim: int) -> int:
    """Rows of a head's matrix that one of those lanes holds: head_dim is padded to 16 times 4, 8 or 16."""
    return 4 if head_dim <= 64 else 8 if head_dim <= 128 else 16


class GatedDeltaRule(Part):
    UPS_IN_KERNEL_RANK = 8

    graph_safe = True   # launches only this package's kernels on arena buffers, reads the step's data on the device
    plan_safe = True
    can_overwrite = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, conv_taps: int, norm_eps: float,
                 channel_decay: bool = False, decay_rank: int | None = None, gate_rank: int | None = None):
        for name, value in (("hidden_size", hidden_size), ("num_heads", num_heads), ("num_kv_heads", num_kv_heads), ("head_dim", head_dim),
                            ("value_dim", value_dim), ("conv_taps", conv_taps)):
            if value <= 0:
                raise ValueError(f"{name} must be positive, got {value}")
        if num_heads % num_kv_heads != 0:
            raise ValueError(f"num_heads must be divisible by num_kv_heads, got {num_heads} and {num_kv_heads}")
        if head_dim > 256:
            raise ValueError(f"the scan kernel takes head_dim up to 256, got {head_dim}")
        if norm_eps <= 0:
            raise ValueError(f"norm_eps must be positive, got {norm_eps}")
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.head_dim, self.value_dim, self.conv_taps, self.norm_eps = head_dim, value_dim, conv_taps, norm_eps
        self.channels = 2 * num_kv_heads * head_dim + num_heads * value_dim          # what passes the convolution: q, k, v
        self.columns = self.channels + num_heads * value_dim + 2 * num_heads          # ... and the output gate, step size, decay input
        if not channel_decay and (decay_rank is not None or gate_rank is not None):
            raise ValueError("decay_rank and gate_rank belong to channel_decay")
        for name, value in (("decay_rank", decay_rank), ("gate_rank", gate_rank)):
            if value is not None and value <= 0:
                raise ValueError(f"{name} must be positive when given, got {value}")
        self.channel_decay, self.decay_rank, self.gate_rank = channel_decay, decay_rank, gate_rank
        self.w_in = self.w_o = self.conv = self.a_log = self.dt_bias = self.norm = self.decay_up = self.gate_up = self.decay_w = self.gate_w = None

    def _projections(self):
        qk, v = self.num_kv_heads * self.head_dim, self.num_heads * self.value_dim
        if self.channel_decay:
            # a rank that is not given is whatever the checkpoint holds: -1 in a shape stands for any size
            return (("q_proj", qk), ("k_proj", qk), ("v_proj", v), ("b_proj", self.num_heads), ("a1_proj", self.decay_rank or -1),
                    ("g1_proj", self.gate_rank or -1))
        return (("q_proj", qk), ("k_proj", qk), ("v_proj", v), ("g_proj", v), ("b_proj", self.num_heads), ("a_proj", self.num_heads))

    def tensors(self):
        specs = {f"{name}.weight": TensorSpec((width, self.hidden_size)) for name, width in self._projections()}
        for name, width in self._projections()[:3]:
            specs[f"{name[0]}_conv.weight"] = TensorSpec((width, self.conv_taps))
        specs["A_log"] = TensorSpec((self.num_heads,), role="bias")
        specs["dt_bias"] = TensorSpec((self.num_heads * self.head_dim if self.channel_decay else self.num_heads,), role="bias")
        if self.channel_decay:
            specs["a2_proj.weight"] = TensorSpec((self.num_heads * self.head_dim, self.decay_rank or -1))
            specs["g2_proj.weight"] = TensorSpec((self.num_heads * self.value_dim, self.gate_rank or -1))
        specs["norm.weight"] = TensorSpec((self.value_dim,), role="norm")
        specs["o_proj.weight"] = TensorSpec((self.hidden_size, self.num_heads * self.value_dim))
        return specs

    def bind(self, weights, dtype):
        stacked = torch.cat([weights[f"{name}.weight"] for name, _ in self._projections()], 0).to(dtype)
        pad = -stacked.shape[0] % 16          # whole groups of 16 output columns suit every product kernel
        if pad:
            stacked = torch.cat((stacked, stacked.new_zeros(pad, self.hidden_size)), 0)
        self.w_in = stacked.contiguous()
        self.conv = torch.cat([weights[f"{name}_conv.weight"] for name in "qkv"], 0).float().contiguous()
        self.a_log, self.dt_bias = weights["A_log"].float().contiguous(), weights["dt_bias"].float().contiguous()
        self.norm = weights["norm.weight"].float().contiguous()
        self.w_o = weights["o_proj.weight"].to(dtype).contiguous()
        if self.channel_decay:
            # the second matrices by columns, so that neighbouring lanes read neighbouring values: [rank, outputs] float32
            self.decay_up = weights["a2_proj.weight"].float().t().contiguous()
            self.gate_up = weights["g2_proj.weight"].float().t().contiguous()
            first = {name: weights[f"{name}.weight"].shape[0] for name in ("a1_proj", "g1_proj")}
            if (first["a1_proj"], first["g1_proj"]) != (self.decay_up.shape[0], self.gate_up.shape[0]):
                raise ValueError(f"the two matrices of a low-rank input disagree: {first} against {self.decay_up.shape[0]} and {self.gate_up.shape[0]}")
            self.decay_rank, self.gate_rank = self.decay_up.shape[0], self.gate_up.shape[0]
            # ... and as stored, [outputs, rank], for the products
            self.decay_w, self.gate_w = weights["a2_proj.weight"].float().contiguous(), weights["g2_proj.weight"].float().contiguous()

    def weight_bytes(self):
        ups = (self.decay_w.numel() + self.gate_w.numel()) * 4 if self.channel_decay else 0
        return (self.w_in.numel() + self.w_o.numel()) * self.w_o.element_size() + ups

    def flops(self, tokens, pairs):
        # the projections, and per token and head the two products with the state and its update
        return super().flops(tokens, pairs) + 6.0 * tokens * self.num_heads * self.head_dim * self.value_dim

    def state_floats(self) -> int:
        return self.num_heads * state_rows(self.head_dim) * STATE_LANES * self.value_dim + (self.conv_taps - 1) * self.channels

    def cache_need(self):
        return StateNeed((self.state_floats(),), torch.float32)

    def forward(self, ctx, x, residual, cache, then_norm=None, accumulate: bool = True):
        if cache is None or cache.state is None:
            raise ValueError("the gated delta rule needs a state row per request")
        t = rows_of(x)
        x = materialize(ctx, x)
        proj = ctx.scratch("delta_proj", (t, self.w_in.shape[0]), torch.float32)
        linear(ctx, proj, x, self.w_in)
        out = ctx.scratch("delta_out", (t, self.num_heads * self.value_dim), ctx.dtype)
        qkv = ctx.scratch("delta_qkv", (t, self.channels), torch.float32)
        gates = ctx.scratch("delta_gates", (t, 2 * self.num_heads), torch.float32)
        raw = ctx.scratch("delta_read_out", (t, self.num_heads * self.value_dim), torch.float32)
        if self.channel_decay:
            decays = ctx.scratch("delta_decays", (t, self.num_heads * self.head_dim), torch.float32)
            if max(self.decay_rank, self.gate_rank) <= self.UPS_IN_KERNEL_RANK:
                decay_up, gate_up, gate_in = self.decay_up, self.gate_up, None
            else:
                first = self.channels + self.num_heads
                gate_in = ctx.scratch("delta_gate_in", (t, self.num_heads * self.value_dim), torch.float32)
                linear(ctx, decays, proj[:, first:first + self.decay_rank], self.decay_w)
                linear(ctx, gate_in, proj[:, first + self.decay_rank:first + self.decay_rank + self.gate_rank], self.gate_w)
                decay_up = gate_up = None
            ops.delta_rule_channels(out, proj, cache.state, ctx.token_request, ctx.cu_seqlens_q, ctx.slot_ids, ctx.R, self.conv, self.num_kv_heads,
                                    self.num_heads, self.head_dim, self.value_dim, self.a_log, self.dt_bias, self.norm, self.norm_eps, qkv, gates, raw,
                                    decay_up, decays, gate_up, gate_in)
            linear(ctx, residual, out, self.w_o, accumulate=accumulate)
            return None
        ops.delta_rule(out, proj, cache.state, ctx.token_request, ctx.cu_seqlens_q, ctx.slot_ids, ctx.R, self.conv, self.num_kv_heads,
                       self.num_heads, self.head_dim, self.value_dim, self.a_log, self.dt_bias, self.norm, self.norm_eps, qkv, gates, raw)
        linear(ctx, residual, out, self.w_o, accumulate=accumulate)
        return None


register("mixer", "gated_delta_rule", GatedDeltaRule)
