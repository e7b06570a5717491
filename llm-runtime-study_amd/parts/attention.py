"""Grouped-query causal attention over the paged cache.

Reference mini_llm/nn/attention.py:141-254: q/k/v projections of the normed input, head
split (head h owns columns h*d..(h+1)*d), optional per-head RMSNorm of q and k over head_dim
with one weight for all q heads and one for all k heads (Qwen3, 291-302), rotation of q and k
by the token's absolute position, write of k and v into the cache, softmax(q k^T * scale) v
over cached positions j <= p (mask rule 231-235; scale 1/sqrt(d) unless given, 95-99), kv head
h // (nq/nkv) for query head h (18-33), then the output projection without bias.

q, k and v come from one stacked [nq*d + 2*nkv*d, H] product.  When `kv_shared` is set the
layer owns no keys or values: it projects queries only and attends to the cache of the layer
it is told to read.  `window` keeps keys with p - window < j <= p.  With `values_from_keys` there is no
value projection: a position's value is its key as projected, before the per-head norm and the rotation; the
key matrix is stacked a second time where the value matrix would be, so that every kernel after the product sees
the usual row of q, k and v heads (the product makes those columns twice, from the same weights and inputs).
`forward(..., accumulate=False)` stores the output projection into the float32 rows it is given instead of adding to them.

Further forms, each a parameter: `norm_over="projection"` normalises q and k over the whole projection (all heads of a token
at once, a weight per column) instead of per head; `value_dim` gives the values a size of their own; `keep_first` keeps the
first positions of a sequence visible behind a window (token i sees j <= i with i - j < window or j < keep_first; the kept
keys keep their positions); `output_gate` multiplies the heads' outputs by sigmoid(W_g x) before the output projection (the
gate's matrix is stacked behind q, k and v).  A layer with any of them prepares its heads with `qkv_norm_prep`; its attention
runs on the matrix cores where the shape allows (bfloat16, values as wide as keys; the kept positions' keys are then one more
partial result beside those of the window's splits, which the merge of the splits adds in) and in the any-shape kernel otherwise.

And these, served by the same path: `unit_norm_after_rotation` divides every q and k head by its own root mean square (no
weight, `qk_norm_eps`) after the rotation instead of a weighted norm before it (`rotate_unit_prep` prepares the heads; the
position part says whether a pair is (i, i + rot/2) or (2i, 2i + 1)); `sink` adds a learned term exp(sink_h) per head to the
softmax's denominator, which has no key and no value; `score_cap` passes the scaled scores through cap * tanh(score / cap);
`output_gate="head"` gates with one number a head, sigmoid(W_g x)_h, in the attention kernel that finishes a query or the merge
of its partial results, where `True` gates every value by a kernel of its own; `bias` with any of these
adds the stacked biases to q, k and v: in the product's epilogue, or, where `rotate_unit_prep` prepares the heads, in that kernel
as it reads the rows (in float32; the product then runs without a bias, through the vendor's library for many rows).
"""

from __future__ import annotations

import math

import torch

from ..kernels import ops
from .base import PagedKVNeed, Part, PartSpec, TensorSpec, create, length_class, register
from .linear import ScaledRows, kernels_of, linear, materialize, rows_of, workspace_of


class GQAAttention(Part):
    graph_safe = True  # launches only library kernels on arena buffers
    plan_safe = True   # ... and nothing but this package's kernels, with arguments that follow the step's shape alone
    takes_lazy_norm = True
    begins_next_norm = True
    wants_query_groups = True   # ragged steps go to a kernel that walks groups of a request's consecutive tokens
    can_overwrite = True        # forward(..., accumulate=False) stores its output

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, *,
                 position: PartSpec = PartSpec("none"), qk_norm: bool = False, qk_norm_eps: float = 1e-6,
                 bias: bool = False, scale: float | None = None, window: int | None = None,
                 kv_shared: bool = False, values_from_keys: bool = False, norm_over: str = "head", value_dim: int | None = None,
                 keep_first: int = 0, output_gate: bool | str = False, unit_norm_after_rotation: bool = False, sink: bool = False,
                 score_cap: float | None = None):
        for name, value in (("hidden_size", hidden_size), ("num_heads", num_heads), ("num_kv_heads", num_kv_heads), ("head_dim", head_dim)):
            if value <= 0:
                raise ValueError(f"{name} must be positive, got {value}")
        if num_heads % num_kv_heads != 0:
            raise ValueError(f"num_heads must be divisible by num_kv_heads, got {num_heads} and {num_kv_heads}")
        if scale is not None and (not math.isfinite(scale) or scale <= 0):
            raise ValueError(f"scale must be finite and positive, got {scale}")
        if window is not None and window <= 0:
            raise ValueError(f"window must be positive when given, got {window}")
        if qk_norm and qk_norm_eps <= 0:
            raise ValueError(f"qk_norm_eps must be positive, got {qk_norm_eps}")
        self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim = hidden_size, num_heads, num_kv_heads, head_dim
        self.position = create("position", position)
        self.qk_norm, self.qk_norm_eps, self.bias = qk_norm, qk_norm_eps, bias
        self.scale = 1.0 / math.sqrt(head_dim) if scale is None else scale
        if values_from_keys and kv_shared:
            raise ValueError("a layer that owns no keys has no values to take from them")
        self.window, self.kv_shared, self.values_from_keys = window, kv_shared, values_from_keys
        if norm_over not in ("head", "projection"):
            raise ValueError(f"norm_over must be 'head' or 'projection', got {norm_over!r}")
        if value_dim is not None and value_dim <= 0:
            raise ValueError(f"value_dim must be positive when given, got {value_dim}")
        if keep_first < 0 or (keep_first and window is None):
            raise ValueError(f"keep_first must not be negative and needs a window, got {keep_first}")
        if output_gate not in (False, True, "head"):
            raise ValueError(f"output_gate must be False, True (a gate a value) or 'head' (a gate a head), got {output_gate!r}")
        if score_cap is not None and (not math.isfinite(score_cap) or score_cap <= 0):
            raise ValueError(f"score_cap must be finite and positive when given, got {score_cap}")
        if unit_norm_after_rotation and qk_norm:
            raise ValueError("heads are normalised before the rotation with a weight (qk_norm) or after it without one, not both")
        if unit_norm_after_rotation and qk_norm_eps <= 0:
            raise ValueError(f"qk_norm_eps must be positive, got {qk_norm_eps}")
        self.norm_over, self.value_dim, self.keep_first, self.output_gate = norm_over, value_dim or head_dim, keep_first, output_gate
        self.unit_after, self.has_sink, self.score_cap = unit_norm_after_rotation, sink, score_cap
        self.neighbours = getattr(self.position, "pairing", "halves") == "interleaved"
        # the forms that the kernels preparing whole rows serve (see the module's text)
        self.whole_rows = bool((qk_norm and norm_over == "projection") or self.value_dim != head_dim or keep_first > 0 or output_gate
                               or unit_norm_after_rotation or sink or score_cap is not None or self.neighbours)
        if self.whole_rows and (kv_shared or values_from_keys or (qk_norm and norm_over == "head")):
            raise ValueError("a norm over the projection or after the rotation, values of their own size, kept first positions, a sink, "
                             "capped scores and an output gate come without shared or key-made values and per-head norms before the rotation")
        if self.neighbours and qk_norm:
            raise ValueError("neighbouring pairs are rotated by the kernel that normalises after the rotation or not at all")
        self.b_late = None
        self.gate_width = 0 if not output_gate else num_heads if output_gate == "head" else num_heads * self.value_dim
        self.sinks = None
        self.w_qkv = self.b_qkv = self.w_o = self.q_norm = self.k_norm = None

    # ------------------------------------------------------------------ weights
    def tensors(self):
        h, d = self.hidden_size, self.head_dim
        names = ("q_proj",) if self.kv_shared else ("q_proj", "k_proj") if self.values_from_keys else ("q_proj", "k_proj", "v_proj")
        widths = {"q_proj": self.num_heads * d, "k_proj": self.num_kv_heads * d, "v_proj": self.num_kv_heads * self.value_dim}
        specs = {f"{n}.weight": TensorSpec((widths[n], h)) for n in names}
        if self.bias:
            specs.update({f"{n}.bias": TensorSpec((widths[n],), role="bias") for n in names})
        if self.output_gate:
            specs["g_proj.weight"] = TensorSpec((self.gate_width, h))
        if self.has_sink:
            specs["sink"] = TensorSpec((self.num_heads,), role="bias")
        specs["o_proj.weight"] = TensorSpec((h, self.num_heads * self.value_dim))
        if self.qk_norm:
            over = d if self.norm_over == "head" else None
            specs["q_norm.weight"] = TensorSpec((over or widths["q_proj"],), role="norm")
            if not self.kv_shared:
                specs["k_norm.weight"] = TensorSpec((over or widths["k_proj"],), role="norm")
        return specs

    def bind(self, weights, dtype):
        names = ("q_proj",) if self.kv_shared else ("q_proj", "k_proj", "k_proj") if self.values_from_keys else ("q_proj", "k_proj", "v_proj")
        if self.output_gate:
            names += ("g_proj",)
        stacked = [weights[f"{n}.weight"] for n in names]
        biases = [weights[f"{n}.bias"] if n != "g_proj" else weights["g_proj.weight"].new_zeros(self.gate_width) for n in names] if self.bias else None
        pad = -sum(w.shape[0] for w in stacked) % 16 if self.whole_rows else 0     # rows of whole groups of 16 columns suit every product kernel
        if pad:
            stacked.append(stacked[0].new_zeros(pad, self.hidden_size))
            if biases is not None:
                biases.append(biases[0].new_zeros(pad))
        self.w_qkv = torch.cat(stacked, 0).to(dtype).contiguous()
        self.b_qkv = torch.cat(biases, 0).to(dtype).contiguous() if self.bias else None
        # the kernel that rotates and then normalises the heads adds the biases itself, in float32, as it reads the rows
        self.b_late = torch.cat(biases, 0).float().contiguous() if self.bias and (self.unit_after or self.neighbours) else None
        if self.has_sink:
            self.sinks = weights["sink"].float().contiguous()
        self.w_o = weights["o_proj.weight"].to(dtype).contiguous()
        if self.qk_norm:
            self.q_norm = weights["q_norm.weight"]
            self.k_norm = weights["k_norm.weight"] if not self.kv_shared else self.q_norm
            if self.whole_rows:
                self.q_norm, self.k_norm = self.q_norm.float().contiguous(), self.k_norm.float().contiguous()

    def weight_bytes(self):
        return (self.w_qkv.numel() + self.w_o.numel()) * self.w_o.element_size()

    def flops(self, tokens, pairs):
        if self.window is not None:
            pairs = min(pairs, tokens * self.window)
        # the projections, then scores and weighted values: two products of head_dim per pair and query head
        return super().flops(tokens, pairs) + 2.0 * pairs * self.num_heads * (self.head_dim + self.value_dim)

    def cache_need(self):
        if self.kv_shared:
            return None
        if self.value_dim != self.head_dim or self.keep_first:
            return PagedKVNeed(self.num_kv_heads, self.head_dim, self.window, value_dim=None if self.value_dim == self.head_dim else self.value_dim,
                               keep_first=self.keep_first)
        return PagedKVNeed(self.num_kv_heads, self.head_dim, self.window)

    @staticmethod
    def _decode_splits(workgroups: int, longest: int, bound: int, page_size: int) -> int:
        """Into how many workgroups the keys of one decode token are divided: enough to give every
        compute unit two when the batch alone does not (measured on MI355X inside the 8-request
        decode step at 2,048 tokens of context: 8 splits 4.58 ms, 4 splits 4.61 ms), but at least
        256 keys each (a power of two that follows the length's class, not the length); and enough
        that the block table entries of one workgroup (at most 4,096) fit its LDS for contexts up
        to `bound`."""
        units = ops.compute_units()
        # from five workgroups for every eight units on, the batch alone does as well or better, and there is nothing
        # to merge (2,048 tokens of context, batch 20 / 24 / 32: 37.8 / 42.0 / 52.7 us undivided against 40.1 / 45 /
        # 54.4 us with the 4 / 3 / 2 parts that two workgroups a unit would ask for; the same at 8,192 tokens)
        wanted = 1 if 8 * workgroups >= 5 * units else -(-2 * units // workgroups)
        # between one and one and a half workgroups a unit some units have two where the others have one, and with
        # contexts of 2,048 tokens and more the second round costs more than a merge: two parts (40 query heads on 8:
        # batch 33 / 40 / 44 / 48 at 2,048 tokens 72.6 / 75.1 / 77.9 / 79.7 us undivided, 66.5 / 71.5 / 73.3 / 78.2 in two parts;
        # at 4,096 tokens 140 / 144 / 148 / 151 against 122 / 129 / 134 / 144; at 1,024 tokens and from batch 52 on nothing
        # is gained; four parts are better still up to batch 40 and worse from 44 on, and a graph serves both)
        if units < workgroups <= units + units // 2 and length_class(longest) >= 2048:
            wanted = 2
        return max(1, min(wanted, length_class(longest) // 256, 64), -(-bound // (4096 * page_size)))

    @staticmethod
    def _prefill_splits(workgroups: int, longest: int, outputs: int, heads_per_group: int = 4, tokens: int = 0) -> int:
        """Into how many workgroups the keys of every query group of a ragged step are divided: one, unless
        the groups alone leave compute units idle (a last portion of a prompt, a short portion after a long
        context), and never from two workgroups a unit on.  Partial results (float32, `outputs` values per split)
        stay within 256 MB.  Measured on
        MI355X, 32 query heads on 8 kv heads:
          * contexts of 16,384 tokens and more: towards eight workgroups a unit, at least 1,024 keys each
            (32,768 tokens of context: 1 token 1,161 -> 57 us with 32 splits, 64 tokens 1,165 -> 105 us with
            16, 512 tokens 1,186 -> 576 us with 8);
          * shorter contexts: towards two workgroups a unit, at least 256 keys each (2,048 tokens of context: 64 tokens 42.5 -> 18.6 us with 8 splits, 256 tokens 43.2 -> 32.4 with
            4, 512 tokens 87.5 -> 76.4 with 2, but 1,024 tokens 96.8 -> 127 and 2,032 tokens 111 -> 173 with 2:
            what the merge reads and writes grows with the tokens, what a split saves with the context).  So under
            16,384 tokens of context the keys are divided only where the longest context is at least four times the
            step's `tokens` (undivided against 2 splits with their merge: 512 tokens after 0 / 512 / 1,024 / 1,536:
            16.9 / 26.6 / 36.2 / 45.8 against 24.4 / 30.5 / 36.9 / 42.9 us; 256 tokens after 256 / 512 / 768 / 1,024:
            16.5 / 21.1 / 25.7 / 30.2 against 18.8 / 20.3 / 23.1 / 25.6 us; 128 tokens after 0 / 256 / 512: 14.4 / 14.1 /
            18.5 against 16.2 / 16.8 / 17.1 us).
        A kv group of five to eight heads walks the keys once with a wave for every head while the launch is at
        most two workgroups a unit; that walk is short enough that one workgroup a unit is the aim (40 heads on
        8: 512 tokens after 1,536 54 us undivided against 72 with 2; 256 tokens 51 -> 43 with 2, 128 tokens
        after 8,064 177 -> 59 with 4, 64 tokens after 2,000 50 -> 22 with 8); from 16,384 tokens of context on the rule
        for long contexts holds for them too (512 tokens after 32,256: 697 us undivided, 617 with 8)."""
        units = ops.compute_units()
        within = (64 << 20) // max(outputs, 1)
        if workgroups >= 2 * units:      # (2,048 tokens in groups of 32 after 30,720: 1,071 us undivided, 1,115 with 2)
            return 1
        if longest < 16384 and longest < 4 * tokens:
            return 1
        if heads_per_group > 4 and workgroups <= units and longest < 16384:
            return max(1, min(-(-units // workgroups), longest // 256, 32, within))
        if longest >= 16384:
            return max(1, min(-(-8 * units // workgroups), longest // 1024, 32, within))
        return max(1, min(-(-2 * units // workgroups), longest // 256, 32, within))

    PREPARE_INSIDE_ROWS = 16     # rows of a decode step up to which the attention kernel prepares q, k and v itself

    # ------------------------------------------------------------------ forward
    def forward(self, ctx, x, residual, cache, then_norm=None, accumulate: bool = True):
        if cache is None:
            raise ValueError("attention needs a paged cache (its own, or the one it is told to read)")
        t, d, nq = rows_of(x), self.head_dim, self.num_heads
        nkv = 0 if self.kv_shared else self.num_kv_heads
        group = ctx.group(cache.group)
        tables = self.position.tables(ctx)
        cos, sin = tables if tables is not None else (None, None)
        if self.whole_rows:
            return self._forward_whole_rows(ctx, x, residual, cache, group, cos, sin, then_norm, accumulate)
        qkv = ctx.scratch("attn_qkv", (t, (nq + 2 * nkv) * d), ctx.dtype)
        # 17..128 rows of a decode step: the q/k/v product and the preparation of its heads as two kernels, the
        # second adding up the sums of the product's K splits (no kernel of its own for that)
        together = (ctx.all_decode and self.b_qkv is None and ctx.dtype == torch.bfloat16 and t > self.PREPARE_INSIDE_ROWS
                    and ops.gemm_mid_qk_prep_takes(self.w_qkv.dtype, t, nq, nkv, d, self.w_qkv.shape[1], 0 if cos is None else cos.shape[1],
                                                   kernels_of(ctx)))
        begun = plain = None
        if together:
            begun = x if isinstance(x, ScaledRows) else None          # a norm that the product before began
            plain = begun.x if begun is not None else materialize(ctx, x)
            together = plain.dtype == torch.bfloat16 and plain.is_contiguous()
        if together:
            ops.gemm_mid_qk_prep(qkv, plain, self.w_qkv, None if begun is None else begun.sumsq, 0.0 if begun is None else begun.eps,
                                 nq, nkv, d, self.q_norm, self.k_norm, self.qk_norm_eps, cos, sin, cache.k_pages, cache.v_pages,
                                 group.slots, group.page_size, choice=kernels_of(ctx), workspace=workspace_of(ctx))
        else:
            linear(ctx, qkv, x if plain is None or begun is not None else plain, self.w_qkv, self.b_qkv)
        out = ctx.scratch("attn_out", (t, nq * d), ctx.dtype)
        kv_heads = cache.k_pages.shape[1]
        decode = ctx.all_decode and ops.attention_decode_supported(ctx.dtype, nq, kv_heads, d, group.page_size)
        # a decode step's attention kernel normalises and rotates q and k and writes the new key and
        # value itself, when the rotation covers the whole head or there is none; beyond 16 rows a kernel
        # before it does that once a token (measured: 98 against 108 us for the attention kernel at 64 rows)
        whole_head = cos is None or cos.shape[1] * 2 == d
        prepare = queries_raw = None
        if together:
            pass
        elif decode and whole_head and ops.decode_prepare_supported(d, cos is not None) and t <= self.PREPARE_INSIDE_ROWS:
            prepare = ops.DecodePrepare(self.q_norm, self.k_norm, self.qk_norm_eps, cos, sin, nkv)
        else:
            # a ragged step of heads of 128: the attention kernel normalises and rotates the q heads on their way into its
            # registers, so that only the k and v heads pass through a kernel before it (a third of the rows' bytes;
            # measured at 2,048 tokens, 32 q heads on 8: 19-22 -> 10.4 us for the kernel before attention, 66 -> 68 us
            # for attention itself)
            if (not decode and nkv > 0 and whole_head and ops.attention_prefill_prepares(d)
                    and ops.attention_decode_supported(ctx.dtype, nq, kv_heads, d, group.page_size)):
                queries_raw = ops.DecodePrepare(self.q_norm, None, self.qk_norm_eps, cos, sin, 0)
            ops.qk_prep(qkv, nq, nkv, d, self.q_norm, self.k_norm, self.qk_norm_eps, cos, sin,
                        cache.k_pages, cache.v_pages, group.slots, group.page_size, skip_q=queries_raw is not None)
        if decode:
            longest, bound = ctx.max_k, ctx.max_k_bound
            if self.window is not None:
                longest, bound = min(longest, self.window + 32), min(bound, self.window + 64)
            splits = self._decode_splits(t * kv_heads, longest, bound, group.page_size)
            part_o = part_ml = None
            if splits > 1:
                part_o = ctx.scratch("attn_part_o", (t, nq * splits * d), torch.float32)
                part_ml = ctx.scratch("attn_part_ml", (t, nq * splits * 2), torch.float32)
            ops.attention_decode(out, qkv, cache.k_pages, cache.v_pages, group.block_table, ctx.token_slot, ctx.positions,
                                 nq, self.scale, self.window or 0, splits, part_o, part_ml, ctx.max_k_bound, prepare,
                                 form=1)   # the next tile on its way while one is worked on, the first one before the query is prepared (measured: 0.6 % of a step)
        elif ops.attention_decode_supported(ctx.dtype, nq, kv_heads, d, group.page_size):
            # sized by the step's coarse bound of the longest context, the same for every step of one shape
            longest = ctx.max_k_bound if self.window is None else min(ctx.max_k_bound, self.window + 64)
            singles = ctx.single_rows
            if singles:
                # the single tokens at the head of a mixed step (decoding requests beside a prompt portion) go to the
                # kernel of decode steps, which divides one token's keys between waves and workgroups; as rows of
                # the other kernel each would walk its whole context in one workgroup
                splits = self._decode_splits(singles * kv_heads, longest, ctx.max_k_bound, group.page_size)
                part_o = part_ml = None
                if splits > 1:
                    part_o = ctx.scratch("attn_single_part_o", (singles, nq * splits * d), torch.float32)
                    part_ml = ctx.scratch("attn_single_part_ml", (singles, nq * splits * 2), torch.float32)
                first = None
                if queries_raw is not None:      # the decode kernel prepares the q heads of its rows likewise
                    parted = None
                    if cos is not None:          # the tables' rows of the single tokens and of the rest, cut once a step
                        parted = ctx.memo.get(("rotation_rows", id(cos)))
                        if parted is None:
                            parted = ctx.memo[("rotation_rows", id(cos))] = (cos[:singles], sin[:singles], cos[singles:], sin[singles:])
                    first = ops.DecodePrepare(self.q_norm, self.k_norm, self.qk_norm_eps, None if parted is None else parted[0],
                                              None if parted is None else parted[1], 0)
                ops.attention_decode(out[:singles], qkv[:singles], cache.k_pages, cache.v_pages, group.block_table, ctx.token_slot,
                                     ctx.positions, nq, self.scale, self.window or 0, splits, part_o, part_ml, ctx.max_k_bound, first, form=1)
            rest = ctx.memo.get("rows_after_singles")
            if rest is None:
                rest = ctx.memo["rows_after_singles"] = (ctx.token_slot[singles:], ctx.positions[singles:])
            if queries_raw is not None and singles and cos is not None:
                queries_raw = ops.DecodePrepare(self.q_norm, None, self.qk_norm_eps, parted[2], parted[3], 0)
            splits = self._prefill_splits(ctx.num_qblocks * kv_heads, longest, (t - singles) * nq * d, nq // kv_heads, t - singles)
            part_o = part_ml = None
            if splits > 1:
                part_o = ctx.scratch("attn_part_o", (t - singles, nq * splits * d), torch.float32)
                part_ml = ctx.scratch("attn_part_ml", (t - singles, nq * splits * 2), torch.float32)
            ops.attention_prefill(out[singles:], qkv[singles:], cache.k_pages, cache.v_pages, group.block_table, rest[0], rest[1],
                                  ctx.qblock_token0, ctx.qblock_count, nq, self.scale, self.window or 0, ctx.max_qblock, ctx.max_k_bound,
                                  splits, part_o, part_ml, queries_raw)
        else:
            ops.attention(out, qkv, cache.k_pages, cache.v_pages, group.block_table, ctx.token_slot, ctx.positions,
                          nq, self.scale, self.window or 0)
        return linear(ctx, residual, out, self.w_o, accumulate=accumulate, then_norm=then_norm)

    def _forward_whole_rows(self, ctx, x, residual, cache, group, cos, sin, then_norm, accumulate):
        """The forms whose heads `qkv_norm_prep` prepares: one product for q, k, v (and the gate), the norms over the whole
        projection, rotation and the write into the pages in one kernel, attention, the gate, the output projection."""
        t, d, dv, nq, nkv = rows_of(x), self.head_dim, self.value_dim, self.num_heads, self.num_kv_heads
        gate_at = (nq + nkv) * d + nkv * dv
        qkv = ctx.scratch("attn_qkvg", (t, self.w_qkv.shape[0]), ctx.dtype)
        linear(ctx, qkv, x, self.w_qkv, None if self.b_late is not None else self.b_qkv)
        if self.unit_after or self.neighbours:
            ops.rotate_unit_prep(qkv, nq, nkv, d, dv, self.qk_norm_eps, self.unit_after, cos, sin, self.neighbours, cache.k_pages, cache.v_pages,
                                 group.slots, group.page_size, bias=self.b_late)
        else:
            ops.qkv_norm_prep(qkv, nq, nkv, d, dv, self.q_norm, self.k_norm, self.qk_norm_eps, cos, sin, cache.k_pages, cache.v_pages,
                              group.slots, group.page_size)
        more = {"sinks": self.sinks, "softcap": self.score_cap or 0.0}
        # a gate a head is applied by the attention kernel that finishes a query (or by the merge of its partial results); a
        # gate a value by a kernel of its own behind them
        gates = qkv[:, gate_at:gate_at + nq] if self.output_gate == "head" else None
        out = ctx.scratch("attn_out", (t, nq * dv), ctx.dtype)
        cores = dv == d and ops.attention_decode_supported(ctx.dtype, nq, nkv, d, group.page_size)
        extra = 1 if self.keep_first else 0      # the kept first positions' share is one more partial result for the merge
        if cores and ctx.all_decode:
            longest, bound = ctx.max_k, ctx.max_k_bound
            if self.window is not None:
                longest, bound = min(longest, self.window + 32), min(bound, self.window + 64)
            splits = self._decode_splits(t * nkv, longest, bound, group.page_size)
            part_o = part_ml = None
            if splits + extra > 1:
                part_o = ctx.scratch("attn_part_o", (t, nq * (splits + extra) * d), torch.float32)
                part_ml = ctx.scratch("attn_part_ml", (t, nq * (splits + extra) * 2), torch.float32)
            ops.attention_decode(out, qkv, cache.k_pages, cache.v_pages, group.block_table, ctx.token_slot, ctx.positions,
                                 nq, self.scale, self.window or 0, splits, part_o, part_ml, ctx.max_k_bound, None, form=1,
                                 keep_first=self.keep_first, gates=gates, **more)
        elif cores:
            longest = ctx.max_k_bound if self.window is None else min(ctx.max_k_bound, self.window + 64)
            singles = ctx.single_rows
            if singles:
                splits = self._decode_splits(singles * nkv, longest, ctx.max_k_bound, group.page_size)
                part_o = part_ml = None
                if splits + extra > 1:
                    part_o = ctx.scratch("attn_single_part_o", (singles, nq * (splits + extra) * d), torch.float32)
                    part_ml = ctx.scratch("attn_single_part_ml", (singles, nq * (splits + extra) * 2), torch.float32)
                ops.attention_decode(out[:singles], qkv[:singles], cache.k_pages, cache.v_pages, group.block_table, ctx.token_slot,
                                     ctx.positions, nq, self.scale, self.window or 0, splits, part_o, part_ml, ctx.max_k_bound, None, form=1,
                                     keep_first=self.keep_first, gates=None if gates is None else gates[:singles], **more)
            rest = ctx.memo.get("rows_after_singles")
            if rest is None:
                rest = ctx.memo["rows_after_singles"] = (ctx.token_slot[singles:], ctx.positions[singles:])
            splits = self._prefill_splits(ctx.num_qblocks * nkv, longest, (t - singles) * nq * d, nq // nkv, t - singles)
            part_o = part_ml = None
            if splits + extra > 1:
                part_o = ctx.scratch("attn_part_o", (t - singles, nq * (splits + extra) * d), torch.float32)
                part_ml = ctx.scratch("attn_part_ml", (t - singles, nq * (splits + extra) * 2), torch.float32)
            ops.attention_prefill(out[singles:], qkv[singles:], cache.k_pages, cache.v_pages, group.block_table, rest[0], rest[1],
                                  ctx.qblock_token0, ctx.qblock_count, nq, self.scale, self.window or 0, ctx.max_qblock, ctx.max_k_bound,
                                  splits, part_o, part_ml, None, keep_first=self.keep_first, gates=None if gates is None else gates[singles:], **more)
        else:
            ops.attention(out, qkv, cache.k_pages, cache.v_pages, group.block_table, ctx.token_slot, ctx.positions, nq, self.scale,
                          self.window or 0, self.keep_first, gates=gates, **more)
        if self.output_gate is True:
            ops.sigmoid_gate(out, qkv[:, gate_at:gate_at + self.gate_width])
        return linear(ctx, residual, out, self.w_o, accumulate=accumulate, then_norm=then_norm)


register("mixer", "gqa_attention", GQAAttention)
