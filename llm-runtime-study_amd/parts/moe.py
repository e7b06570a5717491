"""Routed experts: a feed-forward made of many small ones, of which every token runs a few.

    z = W_router x                                 float32 (x may be the activation's rounding)
    rule "softmax_chosen":  chosen = the `top` largest z + bias;  p = softmax((z + bias)[chosen])
    rule "sigmoid":         s = sigmoid(z); chosen = the `top` largest s + bias (the bias takes part in the choice only;
                            with groups, among the experts of the `keep` groups whose two largest s + bias sum highest);
                            p = s[chosen] / (sum of s[chosen] + 1e-20) * scale
    rule "sigmoid_scores":  chosen as under "sigmoid"; p = s[chosen] * scale (the scores as they are, not divided by their sum)
    out = sum over chosen e of p_e * expert_e(x), or with `weight_on="input"` the sum of expert_e(p_e * x)
    expert "relu_squared":  W_down relu(W_up x)^2;   "silu_gated":  W_down (silu(W_gate x) * (W_up x))
    expert "clamped_gated": W_down (g * sigmoid(alpha g) * (u + 1)) with g = min(W_gate x, limit), u = clamp(W_up x, -limit, limit)
    `shared`: a feed-forward part that runs for every token; its output is added to the experts' sum (before a layer's norm).

On the device: the router product, the choice per token, one sort of the step's (token, choice) pairs by expert
into runs padded to whole row tiles, two grouped products over the sorted rows (the activation in the first one's
epilogue), and one kernel that adds a token's rows up in the order of its choices, which can also apply the norm
of a layer that normalises outputs and add the result into the stream (`applies_output_norm`), or replace the stream by the
layer norm of its sum with it (`applies_sum_norm`).  Nothing is read
on the host: the launches are sized by the step's shape alone (at most pairs / tile + experts tiles).
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, PartSpec, TensorSpec, create, flops_of, register, under
from .linear import kernels_of, materialize, rows_of, workspace_of

ACTIVATIONS = ("relu_squared", "silu_gated", "clamped_gated")


class RoutedExperts(Part):
    applies_output_norm = True    # forward(..., output_norm=norm): residual += norm(out) instead of residual += out
    applies_sum_norm = True       # forward(..., sum_norm=(norm, alpha)): residual = norm(alpha * residual + out), for a layer norm
    rounds_stream = True          # forward(..., rounded=buffer): the updated stream is left there in bfloat16 as well

    def __init__(self, hidden_size: int, intermediate_size: int, num_experts: int, top: int, router_bias: bool = False,
                 activation: str = "relu_squared", rule: str = "softmax_chosen", groups: int = 0, keep: int = 0, weight_scale: float = 1.0,
                 bias_name: str = "router.bias", weight_on: str = "output", activation_alpha: float = 1.702, activation_limit: float | None = None,
                 shared: PartSpec | None = None):
        if min(hidden_size, intermediate_size, num_experts, top) <= 0:
            raise ValueError("hidden_size, intermediate_size, num_experts and top must be positive")
        if top > num_experts:
            raise ValueError(f"a token cannot run {top} of {num_experts} experts")
        if num_experts > 512:
            raise ValueError(f"the routing kernel takes up to 512 experts, got {num_experts}")
        if activation not in ACTIVATIONS:
            raise ValueError(f"unknown activation {activation!r}; known: {', '.join(ACTIVATIONS)}")
        self.hidden_size, self.intermediate_size, self.num_experts, self.top = hidden_size, intermediate_size, num_experts, top
        self.inner = intermediate_size       # features a grouped product makes per expert (one more where an odd size is padded)
        self.router_bias, self.activation, self.bias_name = router_bias, activation, bias_name
        self.rule = ops.RouteRule(rule, groups, keep, weight_scale)
        if rule not in ops.RouteRule.KINDS:
            raise ValueError(f"unknown routing rule {rule!r}; known: {', '.join(ops.RouteRule.KINDS)}")
        if groups and (rule != "sigmoid" or num_experts % groups or not 0 < keep <= groups or keep * (num_experts // groups) < top):
            raise ValueError(f"{num_experts} experts in {groups} groups of which {keep} are kept cannot give {top} choices under rule {rule!r}")
        if not weight_scale > 0:
            raise ValueError(f"weight_scale must be positive, got {weight_scale}")
        self.gated = activation in ("silu_gated", "clamped_gated")
        self.clamped = None
        if activation == "clamped_gated":
            if activation_limit is None or not activation_limit > 0:
                raise ValueError(f"the clamped activation needs a positive limit, got {activation_limit}")
            self.clamped = (float(activation_alpha), float(activation_limit))
        if weight_on not in ("output", "input"):
            raise ValueError(f"weight_on must be 'output' or 'input', got {weight_on!r}")
        if weight_on == "input" and self.clamped is None:
            raise ValueError("weights on the experts' inputs are served by the clamped gated activation's kernels only")
        self.weight_on = weight_on
        self.shared = None if shared is None else create("feed_forward", shared)
        if self.shared is not None and not getattr(self.shared, "can_overwrite", False):
            raise ValueError("a shared expert must be able to store its output (can_overwrite)")
        self.router = self.bias = self.up = self.down = None

    @property
    def graph_safe(self) -> bool:
        return self.shared is None or getattr(self.shared, "graph_safe", False)

    @property
    def plan_safe(self) -> bool:
        return self.shared is None or getattr(self.shared, "plan_safe", False)

    def tensors(self):
        h, i = self.hidden_size, self.intermediate_size
        specs = {"router.weight": TensorSpec((self.num_experts, h))}
        if self.router_bias:
            specs[self.bias_name] = TensorSpec((self.num_experts,), role="bias")
        for e in range(self.num_experts):
            if self.gated:
                specs[f"experts.{e}.gate.weight"] = TensorSpec((i, h))
            specs[f"experts.{e}.up.weight"] = TensorSpec((i, h))
            specs[f"experts.{e}.down.weight"] = TensorSpec((h, i))
        if self.shared is not None:
            specs.update({f"shared.{name}": spec for name, spec in self.shared.tensors().items()})
        return specs

    def bind(self, weights, dtype):
        router = weights["router.weight"].to(dtype)
        pad = -router.shape[0] % 16           # whole groups of 16 output columns suit every product kernel
        if pad:
            router = torch.cat((router, router.new_zeros(pad, self.hidden_size)), 0)
        self.router = router.contiguous()
        self.bias = weights[self.bias_name].float().contiguous() if self.router_bias else None
        if self.clamped is not None and self.intermediate_size % 2:
            # an odd size: one more feature whose gate, up and down weights are zero; it gives g = u = 0, so 0 * sigmoid(0) * 1 = 0
            self._bind_padded(weights, dtype)
            return
        if self.gated:      # a feature's gate row, then its up row: one product makes both, and its epilogue the gated activation
            self.paired = self.intermediate_size % 2 == 0
            join = (lambda g, u: torch.stack((g, u), 1).reshape(2 * self.intermediate_size, self.hidden_size)) if self.paired else (lambda g, u: torch.cat((g, u), 0))
            self.up = torch.stack([join(weights[f"experts.{e}.gate.weight"], weights[f"experts.{e}.up.weight"]).to(dtype)
                                   for e in range(self.num_experts)]).contiguous()
        else:
            self.up = torch.stack([weights[f"experts.{e}.up.weight"].to(dtype) for e in range(self.num_experts)]).contiguous()
        self.down = torch.stack([weights[f"experts.{e}.down.weight"].to(dtype) for e in range(self.num_experts)]).contiguous()
        if self.shared is not None:
            self.shared.bind(under(weights, "shared."), dtype)

    def _bind_padded(self, weights, dtype):
        h, i = self.hidden_size, self.intermediate_size
        self.paired = True
        rows = []
        for e in range(self.num_experts):
            gate, up = weights[f"experts.{e}.gate.weight"].to(dtype), weights[f"experts.{e}.up.weight"].to(dtype)
            zero = gate.new_zeros(1, h)
            rows.append(torch.stack((torch.cat((gate, zero), 0), torch.cat((up, zero), 0)), 1).reshape(2 * (i + 1), h))
        self.up = torch.stack(rows).contiguous()
        self.down = torch.stack([torch.cat((weights[f"experts.{e}.down.weight"].to(dtype), self.up.new_zeros(h, 1)), 1)
                                 for e in range(self.num_experts)]).contiguous()
        self.inner = i + 1
        if self.shared is not None:
            self.shared.bind(under(weights, "shared."), dtype)

    def weight_bytes(self):
        """What a decode step of one token reads: the router and the chosen experts."""
        chosen = (3 if self.gated else 2) * self.top * self.hidden_size * self.intermediate_size
        return (self.router.numel() + chosen) * self.up.element_size() + (0 if self.shared is None else self.shared.weight_bytes())

    def flops(self, tokens, pairs):
        own = 2.0 * tokens * (self.num_experts * self.hidden_size + (3 if self.gated else 2) * self.top * self.hidden_size * self.intermediate_size)
        return own + (0.0 if self.shared is None else flops_of(self.shared, tokens, pairs))

    def forward(self, ctx, x, residual, then_norm=None, output_norm=None, rounded=None, sum_norm=None):
        t = rows_of(x)
        x = materialize(ctx, x)
        experts, top = self.num_experts, self.top
        logits = ctx.scratch("moe_logits", (t, self.router.shape[0]), torch.float32)
        ops.gemm(logits, x, self.router, choice=kernels_of(ctx), workspace=workspace_of(ctx) if ctx.dtype == torch.bfloat16 else None)
        ids = ctx.scratch("moe_ids", (t, top), torch.int32)
        weights = ctx.scratch("moe_weights", (t, top), torch.float32)
        tile, tiles = ops.moe_tile_rows(t * top, experts), ops.moe_max_tiles(t * top, experts)
        rows = tiles * tile
        sorted_pairs = ctx.scratch("moe_sorted", (rows,), torch.int32)
        place = ctx.scratch("moe_place", (t * top,), torch.int32)
        tile_expert = ctx.scratch("moe_tile_expert", (tiles,), torch.int32)
        if t <= ops.ROUTE_ALIGN_TOKENS:        # few tokens: the choice and the sort in one launch
            ops.moe_route_align(logits[:, :experts], self.bias, ids, weights, sorted_pairs, place, tile_expert, rule=self.rule)
        else:
            ops.moe_route(logits[:, :experts], self.bias, ids, weights, rule=self.rule)
            ops.moe_align(ids, experts, sorted_pairs, place, tile_expert)
        hidden = ctx.scratch("moe_hidden", (rows, self.inner), ctx.dtype)
        on_input = self.weight_on == "input"
        if self.clamped is not None and self.paired:
            ops.moe_experts(hidden, x, self.up, sorted_pairs, tile_expert, tile, top, gather=True, relu_squared=False, clamped_pairs=self.clamped,
                            pair_weights=weights if on_input else None)
        elif self.clamped is not None:
            raise ValueError("the clamped gated activation is made in the grouped product's epilogue, which takes an even expert size")
        elif self.gated and self.paired:
            ops.moe_experts(hidden, x, self.up, sorted_pairs, tile_expert, tile, top, gather=True, relu_squared=False, silu_pairs=True)
        elif self.gated:    # an odd size: gate rows then up rows, and the activation as a kernel of its own
            both = ctx.scratch("moe_gate_up", (rows, 2 * self.intermediate_size), ctx.dtype)
            ops.moe_experts(both, x, self.up, sorted_pairs, tile_expert, tile, top, gather=True, relu_squared=False)
            ops.silu_mul(hidden, both)
        else:
            ops.moe_experts(hidden, x, self.up, sorted_pairs, tile_expert, tile, top, gather=True, relu_squared=True)
        outputs = ctx.scratch("moe_outputs", (rows, self.hidden_size), torch.float32)
        ops.moe_experts(outputs, hidden, self.down, sorted_pairs, tile_expert, tile, top, gather=False, relu_squared=False)
        extra = None
        if self.shared is not None:      # runs for every token; its rows join the experts' sum before any norm
            extra = ctx.scratch("moe_shared_out", (t, self.hidden_size), torch.float32)
            self.shared.forward(ctx, x, extra, accumulate=False)
        more = {"top": top, "extra": extra}
        if on_input:                     # the weights went into the experts with their inputs: every choice counts once
            weights = None
        if sum_norm is not None:
            weight, eps = sum_norm[0].layer_parameters()
            ops.moe_combine(residual[:t], outputs, place, weights, weight, eps, rounded=rounded, layer_norm_alpha=sum_norm[1], **more)
        elif output_norm is None:
            ops.moe_combine(residual[:t], outputs, place, weights, None, rounded=rounded, **more)
        else:
            weight, eps = output_norm.rms_parameters()
            ops.moe_combine(residual[:t], outputs, place, weights, weight, eps, rounded=rounded, **more)
        return None


register("feed_forward", "routed_experts", RoutedExperts)
