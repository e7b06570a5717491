"""Arrangement of norms, mixer and feed-forward in one layer.

PreNormBlock (reference mini_llm/model/qwen.py:58-72):
    h = h + mixer(norm1(h));  h = h + feed_forward(norm2(h))
The two sums happen inside the parts, which add into the float32 residual stream.

OutputNormBlock: the sublayers read the stream itself and the norms are applied to what they give out:
    h = h + norm1(mixer(h));  h = h + norm2(feed_forward(h))      (the feed-forward may be absent)
A sublayer writes its output into a float32 buffer of the step (a part that says `can_overwrite` stores it, any
other adds into the buffer after it has been cleared), and the norm adds the normalised rows into the stream; a
feed-forward that says `applies_output_norm` is given the norm and does both itself, in the kernel that sums up
its output.

PostNormBlock: the sublayers read the stream itself and each norm is applied to the sum, which replaces the stream:
    h = norm1(alpha * h + mixer(h));  h = norm2(alpha * h + feed_forward(h))      (the feed-forward may be absent)
alpha is a constant of the model.  A sublayer writes into a float32 buffer of the step as for OutputNormBlock, and the norm's
`scale_add_normed` does the rest in one kernel; a feed-forward that says `applies_sum_norm` is given norm and alpha and does
it in the kernel that sums its output up.

ParallelBlock: one norm, and both sublayers read its output; their sum, times a constant of the model, is added to the stream:
    x = norm(h);  h = h + multiplier * (mixer(x) + feed_forward(x))      (the feed-forward may be absent)
The mixer stores its output into a float32 buffer of the step, the feed-forward adds into it, and one kernel adds the buffer
into the stream and leaves the next block's norm of the new stream beside it (`axpby` with a norm), which the model hands
to the block that runs next if that is one of this kind.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, PartSpec, create, flops_of, register, under
from .linear import materialize


class PreNormBlock(Part):
    def __init__(self, mixer: PartSpec, feed_forward: PartSpec, mixer_norm: PartSpec, ff_norm: PartSpec,
                 names: dict | None = None):
        self.mixer = create("mixer", mixer)
        self.feed_forward = create("feed_forward", feed_forward)
        self.mixer_norm = create("norm", mixer_norm)
        self.ff_norm = create("norm", ff_norm)
        self.names = {"mixer": "mixer", "feed_forward": "feed_forward", "mixer_norm": "mixer_norm", "ff_norm": "ff_norm"}
        self.names.update(names or {})

    def _children(self):
        return [(self.names[k], getattr(self, k)) for k in ("mixer_norm", "mixer", "ff_norm", "feed_forward")]

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
        return self.mixer.cache_need()

    @property
    def graph_safe(self) -> bool:
        return all(getattr(part, "graph_safe", False) for _, part in self._children())

    @property
    def plan_safe(self) -> bool:
        return all(getattr(part, "plan_safe", False) for _, part in self._children())

    @property
    def wants_query_groups(self) -> bool:
        return getattr(self.mixer, "wants_query_groups", False)

    chains_norms = True

    @property
    def first_norm(self):
        return self.mixer_norm

    def forward(self, ctx, h, cache, normed=None, then_norm=None):
        """Run the layer on the residual stream h.  `normed`: this layer's first norm of h, already
        begun by the product that last updated h; `then_norm`: the norm that follows this layer.
        Returns that norm of the updated h if the last product began it, else None."""
        # a consumer that says `takes_lazy_norm` gets the norm as a description to fold into its
        # first matrix product; any other gets the normalised tensor
        x = self._normed(ctx, self.mixer_norm, self.mixer, h, normed)
        if getattr(self.mixer, "begins_next_norm", False):
            begun = self.mixer.forward(ctx, x, h, cache, then_norm=self.ff_norm)
        else:
            self.mixer.forward(ctx, x, h, cache)
            begun = None
        x = self._normed(ctx, self.ff_norm, self.feed_forward, h, begun)
        if then_norm is not None and getattr(self.feed_forward, "begins_next_norm", False):
            return self.feed_forward.forward(ctx, x, h, then_norm=then_norm)
        self.feed_forward.forward(ctx, x, h)
        return None

    @staticmethod
    def _normed(ctx, norm, consumer, h, begun=None):
        lazy = getattr(consumer, "takes_lazy_norm", False)
        if begun is not None:
            return begun if lazy else materialize(ctx, begun)
        if lazy and getattr(norm, "has_lazy_form", False):
            return norm.forward(ctx, h, lazy=True)
        return norm.forward(ctx, h)


register("block", "prenorm", PreNormBlock)


class OutputNormBlock(Part):
    def __init__(self, mixer: PartSpec, mixer_norm: PartSpec, feed_forward: PartSpec | None = None, ff_norm: PartSpec | None = None,
                 names: dict | None = None):
        if (feed_forward is None) != (ff_norm is None):
            raise ValueError("a feed-forward and its norm come together")
        self.mixer = create("mixer", mixer)
        self.mixer_norm = create("norm", mixer_norm)
        self.feed_forward = None if feed_forward is None else create("feed_forward", feed_forward)
        self.ff_norm = None if ff_norm is None else create("norm", ff_norm)
        for norm in (self.mixer_norm, self.ff_norm):
            if norm is not None and not callable(getattr(norm, "add_normed", None)):
                raise ValueError("a norm of a sublayer's output must offer add_normed(ctx, residual, y)")
        self.names = {"mixer": "mixer", "feed_forward": "feed_forward", "mixer_norm": "mixer_norm", "ff_norm": "ff_norm"}
        self.names.update(names or {})

    def _children(self):
        return [(self.names[k], getattr(self, k)) for k in ("mixer_norm", "mixer", "ff_norm", "feed_forward") if getattr(self, k) is not None]

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
        return self.mixer.cache_need()

    @property
    def graph_safe(self) -> bool:
        return all(getattr(part, "graph_safe", False) for _, part in self._children())

    @property
    def plan_safe(self) -> bool:
        return all(getattr(part, "plan_safe", False) for _, part in self._children())

    @property
    def wants_query_groups(self) -> bool:
        return getattr(self.mixer, "wants_query_groups", False)

    # What a block of this kind hands the next one of its kind (models/decoder.py passes it on as `given`): the stream
    # rounded to bfloat16, left by the kernel that last added into it, so that no kernel of its own rounds it again.
    handover_kind = "rounded_stream"

    @staticmethod
    def _input(ctx, h):
        """The stream as the activation a sublayer reads: itself in float32 runs, else rounded once."""
        if ctx.dtype == torch.float32:
            return h
        x = ctx.scratch("stream_rounded", tuple(h.shape), ctx.dtype)
        ops.round_rows(x, h)
        return x

    @staticmethod
    def _cleared(ctx, h):
        y = ctx.scratch("sublayer_out", tuple(h.shape), torch.float32)
        ops.fill_i32(y.view(torch.int32), 0)
        return y

    def _add_normed(self, ctx, norm, h, y, name):
        """h += norm(y); returns the updated stream as the next reader's activation if the norm's kernel left it (bfloat16
        runs with a norm that can), else None."""
        if ctx.dtype == torch.bfloat16 and getattr(norm, "rounds_stream", False):
            rounded = ctx.scratch(name, tuple(h.shape), torch.bfloat16)
            norm.add_normed(ctx, h, y, rounded=rounded)
            return rounded
        norm.add_normed(ctx, h, y)
        return None

    def forward(self, ctx, h, cache, given=None):
        x = given if given is not None else self._input(ctx, h)
        if getattr(self.mixer, "can_overwrite", False):
            y = ctx.scratch("sublayer_out", tuple(h.shape), torch.float32)
            self.mixer.forward(ctx, x, y, cache, accumulate=False)
        else:
            y = self._cleared(ctx, h)
            self.mixer.forward(ctx, x, y, cache)
        if self.feed_forward is None:
            return self._add_normed(ctx, self.mixer_norm, h, y, "stream_rounded_next")
        x = self._add_normed(ctx, self.mixer_norm, h, y, "stream_rounded_mid")
        if x is None:
            x = self._input(ctx, h)
        if getattr(self.feed_forward, "applies_output_norm", False) and getattr(self.ff_norm, "rms_parameters", None) is not None:
            if ctx.dtype == torch.bfloat16 and getattr(self.feed_forward, "rounds_stream", False):
                rounded = ctx.scratch("stream_rounded_next", tuple(h.shape), torch.bfloat16)
                self.feed_forward.forward(ctx, x, h, output_norm=self.ff_norm, rounded=rounded)
                return rounded
            self.feed_forward.forward(ctx, x, h, output_norm=self.ff_norm)
            return None
        y = self._cleared(ctx, h)
        self.feed_forward.forward(ctx, x, y)
        return self._add_normed(ctx, self.ff_norm, h, y, "stream_rounded_next")


register("block", "outnorm", OutputNormBlock)


class PostNormBlock(OutputNormBlock):
    """h = norm1(alpha * h + mixer(h)); h = norm2(alpha * h + feed_forward(h)).  Everything around the two sums (which
    buffer a sublayer writes, what is handed to the next block) is OutputNormBlock's."""

    def __init__(self, mixer: PartSpec, mixer_norm: PartSpec, feed_forward: PartSpec | None = None, ff_norm: PartSpec | None = None,
                 alpha: float = 1.0, names: dict | None = None, norm_without_ff: PartSpec | None = None):
        if (feed_forward is None) != (ff_norm is None):
            raise ValueError("a feed-forward and its norm come together")
        if norm_without_ff is not None and feed_forward is not None:
            raise ValueError("norm_without_ff is for a layer that has no feed-forward")
        # A layer without feed-forward has no second update.  Checkpoints that carry the second norm's weight for such a
        # layer all the same mean h = norm2(alpha * h) by it: the tensor is asked for as optional, and the update is made
        # exactly when it was there.
        self.norm_without_ff = None if norm_without_ff is None else create("norm", norm_without_ff)
        self.norm_without_ff_bound = False
        self.alpha = float(alpha)
        self.mixer = create("mixer", mixer)
        self.mixer_norm = create("norm", mixer_norm)
        self.feed_forward = None if feed_forward is None else create("feed_forward", feed_forward)
        self.ff_norm = None if ff_norm is None else create("norm", ff_norm)
        for norm in (self.mixer_norm, self.ff_norm):
            if norm is not None and not callable(getattr(norm, "scale_add_normed", None)):
                raise ValueError("a norm of the sum of stream and sublayer must offer scale_add_normed(ctx, residual, y, alpha)")
        self.names = {"mixer": "mixer", "feed_forward": "feed_forward", "mixer_norm": "mixer_norm", "ff_norm": "ff_norm"}
        self.names.update(names or {})

    def tensors(self):
        out = super().tensors()
        if self.norm_without_ff is not None:
            from dataclasses import replace

            out.update({f"{self.names['ff_norm']}.{name}": replace(spec, optional=True) for name, spec in self.norm_without_ff.tensors().items()})
        return out

    def bind(self, weights, dtype):
        super().bind(weights, dtype)
        if self.norm_without_ff is not None:
            prefix = self.names["ff_norm"] + "."
            wanted = list(self.norm_without_ff.tensors())
            self.norm_without_ff_bound = bool(wanted) and all(prefix + name in weights for name in wanted)
            if self.norm_without_ff_bound:
                self.norm_without_ff.bind(under(weights, prefix), dtype)

    def _add_normed(self, ctx, norm, h, y, name):
        """h = norm(alpha * h + y); returns the new stream as the next reader's activation if the norm's kernel left it."""
        if ctx.dtype == torch.bfloat16 and getattr(norm, "rounds_stream", False):
            rounded = ctx.scratch(name, tuple(h.shape), torch.bfloat16)
            norm.scale_add_normed(ctx, h, y, self.alpha, rounded=rounded)
            return rounded
        norm.scale_add_normed(ctx, h, y, self.alpha)
        return None

    def forward(self, ctx, h, cache, given=None):
        x = given if given is not None else self._input(ctx, h)
        y = self._sublayer(ctx, self.mixer, x, h, cache)
        if self.feed_forward is None and not self.norm_without_ff_bound:
            return self._add_normed(ctx, self.mixer_norm, h, y, "stream_rounded_next")
        x = self._add_normed(ctx, self.mixer_norm, h, y, "stream_rounded_mid")
        if self.feed_forward is None:       # the second norm's weight was there: h = norm2(alpha * h + 0)
            return self._add_normed(ctx, self.norm_without_ff, h, self._cleared(ctx, h), "stream_rounded_next")
        if x is None:
            x = self._input(ctx, h)
        if getattr(self.feed_forward, "applies_sum_norm", False) and getattr(self.ff_norm, "layer_parameters", None) is not None:
            # the kernel that sums the feed-forward's output up takes the stream's share and the norm with it
            rounded = ctx.scratch("stream_rounded_next", tuple(h.shape), torch.bfloat16) if ctx.dtype == torch.bfloat16 else None
            self.feed_forward.forward(ctx, x, h, sum_norm=(self.ff_norm, self.alpha), rounded=rounded)
            return rounded
        y = self._sublayer(ctx, self.feed_forward, x, h)
        return self._add_normed(ctx, self.ff_norm, h, y, "stream_rounded_next")

    def _sublayer(self, ctx, part, x, h, *cache):
        """What `part` gives out for the input x, in the step's float32 buffer for sublayer outputs."""
        if getattr(part, "can_overwrite", False):
            y = ctx.scratch("sublayer_out", tuple(h.shape), torch.float32)
            part.forward(ctx, x, y, *cache, accumulate=False)
        else:
            y = self._cleared(ctx, h)
            part.forward(ctx, x, y, *cache)
        return y


register("block", "postnorm", PostNormBlock)


class ParallelBlock(Part):
    def __init__(self, mixer: PartSpec, norm: PartSpec, feed_forward: PartSpec | None = None, multiplier: float = 1.0, names: dict | None = None):
        self.mixer = create("mixer", mixer)
        self.norm = create("norm", norm)
        self.feed_forward = None if feed_forward is None else create("feed_forward", feed_forward)
        self.multiplier = float(multiplier)
        if not getattr(self.mixer, "can_overwrite", False):
            raise ValueError(f"the mixer of a parallel block must store its output (accumulate=False): {type(self.mixer).__name__} cannot")
        self.names = {"mixer": "mixer", "feed_forward": "feed_forward", "norm": "norm"}
        self.names.update(names or {})

    def _children(self):
        return [(self.names[k], getattr(self, k)) for k in ("norm", "mixer", "feed_forward") if getattr(self, k) is not None]

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
        return self.mixer.cache_need()

    @property
    def graph_safe(self) -> bool:
        return all(getattr(part, "graph_safe", False) for _, part in self._children())

    @property
    def plan_safe(self) -> bool:
        return all(getattr(part, "plan_safe", False) for _, part in self._children())

    @property
    def wants_query_groups(self) -> bool:
        return getattr(self.mixer, "wants_query_groups", False)

    # What a block of this kind hands the next one of its kind: (norm part, its normalised rows of the stream), made by the
    # kernel that added this block's output into the stream; the next block uses them if its norm is the one named.
    handover_kind = "normed_stream"
    takes_next_norm = True

    @property
    def first_norm(self):
        return self.norm

    def forward(self, ctx, h, cache, given=None, next_norm=None):
        if given is not None and given[0] is self.norm:
            x = given[1]
        else:
            x = self.norm.forward(ctx, h)
        y = ctx.scratch("sublayer_out", tuple(h.shape), torch.float32)
        self.mixer.forward(ctx, x, y, cache, accumulate=False)
        if self.feed_forward is not None:
            self.feed_forward.forward(ctx, x, y)
        parameters = getattr(next_norm, "rms_parameters", None)
        if parameters is None:
            ops.axpby(h, h, 1.0, y, self.multiplier)
            return None
        weight, eps = parameters()
        turn = ctx.memo["normed_stream_turn"] = 1 - ctx.memo.get("normed_stream_turn", 0)     # not the buffer this block's x lies in
        normed = ctx.scratch(f"stream_normed{turn}", tuple(h.shape), ctx.dtype)
        ops.axpby(h, h, 1.0, y, self.multiplier, weight if weight.dtype == torch.float32 else self._weight_f32(next_norm, weight), eps, normed)
        return (next_norm, normed)

    @staticmethod
    def _weight_f32(norm, weight):
        """The norm's weight in float32 (made once and kept on the norm part)."""
        kept = getattr(norm, "_weight_f32", None)
        if kept is None or kept.device != weight.device:
            kept = norm._weight_f32 = weight.float().contiguous()
        return kept


register("block", "parallel", ParallelBlock)
