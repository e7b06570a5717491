"""Python face of the gfx950 kernel library.

Every function checks on the host that the operand shapes, dtypes and strides are what
its kernel assumes, then launches on the current torch stream.  Nothing here computes
with torch: tensors are only containers of device memory.  Loading fails loudly when
the library is missing or cannot be built; there is no fallback.
"""

from __future__ import annotations

import functools
import threading

from dataclasses import dataclass
import ctypes
import struct
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p, POINTER, byref

import torch

from ..errors import KernelError
from . import build as _build

_lib = None
_lib_path = ""

F32, BF16 = 0, 1
OUT_STORE, OUT_STORE_F32, OUT_ADD_F32 = 0, 1, 2


@dataclass(frozen=True)
class KernelChoice:
    """Which matrix-product kernels a caller wants where there is a choice.  A step carries its runner's
    (`ctx.kernels`); measurements and tests make their own.  Nothing of it is kept in the kernel library:
    the parts that concern a kernel travel with every call.

    few_rows_max   rows up to which the few-rows kernels (and the norms folded into them) are used: 16 in
                   steps, since from 17 rows on other kernels are faster; the kernels themselves take 64
    mid            the kernel for 17..128 rows may be used
    mid_waves, mid_splits   its workgroup shape (4, 5, 6 or 8 waves) and number of K splits (0: its own choice)
    mid_even       its weight rows dealt out evenly over a whole multiple of the compute units, some workgroups with
                   16 rows more than the others: 0 where it pays (its own choice), 1 never, 2 wherever the shape allows
    whole_lines    the few-rows kernel loads its weights as whole 128-byte lines where the shape allows
    library        bfloat16 products of more rows than these kernels are made for go to the vendor's matrix
                   library (as the reference leaves them to nn.Linear); else to this package's own kernel"""

    few_rows_max: int = 16
    mid: bool = True
    mid_waves: int = 0
    mid_splits: int = 0
    mid_even: int = 0
    whole_lines: bool = True
    library: bool = True

    def __post_init__(self):
        if not 1 <= self.few_rows_max <= 64:
            raise KernelError(f"the few-rows kernel takes 1..64 rows, got few_rows_max={self.few_rows_max}")
        if self.mid_waves not in (0, 4, 5, 6, 8) or not 0 <= self.mid_splits <= 16:
            raise KernelError(f"the kernel for 17..128 rows has 4, 5, 6 or 8 waves and 1..16 K splits (0: its own choice), got {self.mid_waves} and {self.mid_splits}")
        if self.mid_even not in (0, 1, 2):
            raise KernelError(f"mid_even is 0 (where it pays), 1 (never) or 2 (wherever the shape allows), got {self.mid_even}")

    @property
    def word(self) -> int:
        """The choices a kernel launch needs, as the one integer the entry points take."""
        return int(self.mid) | int(self.whole_lines) << 1 | self.mid_waves << 4 | self.mid_splits << 8 | self.mid_even << 13


DEFAULT_CHOICE = KernelChoice()

_SIGNATURES = {
    "lrs_last_error": (c_char_p, []),
    "lrs_plan_run": (c_int, [c_void_p, c_int64, c_int, c_void_p]),
    "lrs_device_arch": (c_int, [c_int, c_char_p, c_int, POINTER(c_int)]),
    "lrs_graph_begin": (c_int, [c_void_p]),
    "lrs_graph_end": (c_int, [c_void_p, POINTER(c_void_p)]),
    "lrs_graph_launch": (c_int, [c_void_p, c_void_p]),
    "lrs_graph_destroy": (c_int, [c_void_p]),
    "lrs_copy_h2d": (c_int, [c_void_p, c_void_p, c_int64, c_void_p]),
    "lrs_copy_h2d_scatter": (c_int, [c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_int, c_void_p]),
    "lrs_embed": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_float, c_void_p]),
    "lrs_rmsnorm": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_float, c_void_p]),
    "lrs_add_rmsnorm": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_void_p]),
    "lrs_rope_table": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_void_p]),
    "lrs_qk_prep": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_float,
                            c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "lrs_gemm_mid_qk_prep": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_float, c_int, c_int, c_int,
                                     c_void_p, c_void_p, c_int, c_float, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                     c_void_p, c_int64, c_void_p]),
    "lrs_silu_mul": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "lrs_add_into": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_void_p]),
    "lrs_fill_i32": (c_int, [c_void_p, c_int, c_int64, c_void_p]),
    "lrs_step_prepare": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                 c_int, c_void_p, c_int, c_int, c_int, c_void_p]),
    "lrs_step_prepare_summary_size": (c_int, []),
    "lrs_scatter_i32": (c_int, [c_void_p, c_void_p, c_int, c_void_p]),
    "lrs_gather_rows": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "lrs_gemm": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p,
                         c_int, c_float, c_int, c_int, c_void_p, c_int64, c_void_p]),
    "lrs_gemm_workspace_bytes": (c_int64, []),
    "lrs_gemm_lines_add_rmsnorm": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_int, c_float, c_void_p, c_int,
                                           c_void_p, c_int64, c_void_p]),
    "lrs_gemm_norm_chain": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                    c_void_p, c_int, c_float, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "lrs_gemm_norm_chain_parts": (c_int, [c_int]),
    "lrs_scale_rows": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_void_p]),
    "lrs_gemm_skinny_capacity": (c_int, []),
    "lrs_advance_decode": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
    "lrs_advance_slots": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_void_p]),
    "lrs_copy_to_pinned": (c_int, [c_void_p, c_void_p, c_int64, c_void_p]),
    "lrs_stream_read": (c_int, [c_void_p, c_int64, c_void_p, c_int, c_void_p]),
    "lrs_probe_lds": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p]),
    "lrs_probe_mfma": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "lrs_probe_lines": (c_int, [c_void_p, c_size_t, c_void_p, c_int, c_int, c_size_t, c_int, c_void_p]),
    "lrs_gemm_prepare": (c_int, []),
    "lrs_library_gemm_prepare": (c_int, []),
    "lrs_library_gemm": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "lrs_host_device_pointer": (c_int, [c_void_p, POINTER(c_void_p)]),
    "lrs_gemm_mid_shape": (c_int, [c_int, c_int, c_int, c_void_p, c_void_p]),
    "lrs_gemm_mid_deal": (c_int, [c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "lrs_gemm_mid_scaled": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int, c_float, c_int,
                                    c_void_p, c_int64, c_void_p]),
    "lrs_gemm_mid_add_norm_begin": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                            c_void_p, c_int64, c_void_p]),
    "lrs_norm_begin_parts": (c_int, [c_int]),
    "lrs_attention": (c_int, [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                              c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_void_p, c_float, c_void_p, c_int, c_void_p]),
    "lrs_qkv_norm_prep": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_float, c_void_p, c_void_p,
                                  c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
    "lrs_sigmoid_gate": (c_int, [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "lrs_rotate_unit_prep": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p, c_void_p, c_int, c_int,
                                     c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p]),
    "lrs_gated_clamped": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_float, c_void_p]),
    "lrs_add_gathered": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p]),
    "lrs_scale_values": (c_int, [c_void_p, c_int64, c_float, c_void_p]),
    "lrs_axpby": (c_int, [c_void_p, c_void_p, c_float, c_void_p, c_float, c_int, c_int, c_void_p, c_float, c_void_p, c_int, c_void_p]),
    "lrs_activation": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_int, c_void_p]),
    "lrs_delta_rule_channels": (c_int, [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                                        c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p,
                                        c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p]),
    "lrs_ssm": (c_int, [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                        c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_float,
                        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "lrs_attention_decode": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                     c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_int, c_int,
                                     c_void_p, c_void_p, c_int, c_float, c_void_p, c_void_p, c_int, c_void_p, c_float, c_void_p, c_int, c_void_p]),
    "lrs_attention_prefill": (c_int, [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                      c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int,
                                      c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_float, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_int, c_void_p]),
    "lrs_attention_prefill_prepares": (c_int, [c_int]),
    "lrs_compute_units": (c_int, []),
    "lrs_gemm_lines_width": (c_int, [c_int, c_int, c_int]),
    "lrs_gemm_lines_splits": (c_int, [c_int, c_int, c_int]),
    "lrs_gemm_lines_split_pays": (c_int, [c_int, c_int, c_int]),
    "lrs_attention_prefill_group": (c_int, []),
    "lrs_attention_prefill_group_for": (c_int, [c_int, c_int]),
    "lrs_choose_tokens": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
    "lrs_choose_tokens_split": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "lrs_choose_tokens_static": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "lrs_choose_tokens_static_init": (c_int, []),
    "lrs_choose_tokens_static_max_parts": (c_int, []),
    "lrs_filter_logits": (c_int, [c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "lrs_round_rows": (c_int, [c_void_p, c_int, c_void_p, c_int64, c_void_p]),
    "lrs_norm_add": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_void_p, c_void_p]),
    "lrs_delta_state_rows": (c_int, [c_int]),
    "lrs_delta_rule": (c_int, [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                               c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p]),
    "lrs_moe_tile_rows": (c_int, [c_int, c_int]),
    "lrs_moe_max_tiles": (c_int, [c_int, c_int]),
    "lrs_moe_route": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p]),
    "lrs_moe_route_align": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int,
                                    c_int, c_int, c_int, c_float, c_void_p]),
    "lrs_moe_align": (c_int, [c_void_p, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p]),
    "lrs_moe_experts": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int,
                                c_int, c_int, c_void_p, c_float, c_float, c_void_p]),
    "lrs_layernorm": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_float, c_void_p]),
    "lrs_scale_add_layernorm": (c_int, [c_void_p, c_void_p, c_float, c_void_p, c_int, c_int, c_int, c_float, c_void_p, c_void_p]),
    "lrs_soft_cap": (c_int, [c_void_p, c_int64, c_float, c_void_p]),
    "lrs_latent_prep": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int, c_float, c_void_p, c_void_p,
                                c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p]),
    "lrs_latent_attention_groups_takes": (c_int, [c_int, c_int, c_int]),
    "lrs_latent_attention_groups": (c_int, [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                            c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int,
                                            c_void_p, c_void_p, c_void_p]),
    "lrs_head_gemm": (c_int, [c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "lrs_latent_attention": (c_int, [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                     c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p]),
    "lrs_moe_combine": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_float, c_void_p, c_int, c_float, c_void_p, c_void_p]),
}


def library():
    """Load (building first if needed) the kernel library; raises KernelError if impossible."""
    global _lib, _lib_path
    if _lib is None:
        try:
            path = _build.ensure_built()
            lib = ctypes.CDLL(str(path))
            _lib_path = str(path)
        except (_build.BuildError, OSError) as exc:
            raise KernelError(f"the HIP kernel library is not available: {exc}") from exc
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = restype, argtypes
        _lib = lib
        if torch.cuda.is_available():
            torch.cuda.init()
            _check(lib.lrs_gemm_prepare())   # device scratch is made now, never inside a step
            _check(lib.lrs_choose_tokens_static_init())
            _check(lib.lrs_library_gemm_prepare())
    return _lib


# ------------------------------------------------------------ launch plans
# Every kernel launch goes through _launch().  While a recording is open, the launch (entry point and
# arguments, without the stream) is also written down; the recording becomes a Plan, an array of 64-bit words
# that lrs_plan_run() walks in one call, making the same launches with the same arguments on the stream it
# is given.  A step whose shape has been seen before is then one call into the library instead of some
# hundreds of Python calls.  What is written down are addresses and sizes: a plan is good for as long as
# every buffer it names lives where it lived (the caller's business: see engine/step.py).
#
# PLAN_OPS fixes the number of each entry point inside a plan; csrc/plan_dispatch.inc, made from this list
# and _SIGNATURES by kernels/plan_codegen.py, is the other side (a test keeps the two in step).
PLAN_OPS = ("lrs_activation", "lrs_add_gathered", "lrs_add_into", "lrs_add_rmsnorm", "lrs_advance_decode", "lrs_advance_slots", "lrs_attention", "lrs_attention_decode",
            "lrs_attention_prefill", "lrs_axpby", "lrs_choose_tokens", "lrs_choose_tokens_split", "lrs_copy_to_pinned", "lrs_delta_rule", "lrs_delta_rule_channels", "lrs_embed", "lrs_fill_i32",
            "lrs_filter_logits", "lrs_gated_clamped", "lrs_gather_rows", "lrs_gemm", "lrs_gemm_lines_add_rmsnorm", "lrs_gemm_mid_add_norm_begin", "lrs_gemm_mid_qk_prep", "lrs_gemm_mid_scaled",
            "lrs_gemm_norm_chain", "lrs_head_gemm", "lrs_latent_attention", "lrs_latent_attention_groups", "lrs_latent_prep", "lrs_layernorm", "lrs_library_gemm", "lrs_moe_align", "lrs_moe_combine", "lrs_moe_experts", "lrs_moe_route", "lrs_moe_route_align", "lrs_norm_add",
            "lrs_qk_prep", "lrs_qkv_norm_prep", "lrs_rmsnorm", "lrs_rope_table", "lrs_rotate_unit_prep", "lrs_round_rows", "lrs_scale_add_layernorm", "lrs_scale_rows", "lrs_scale_values", "lrs_sigmoid_gate", "lrs_silu_mul", "lrs_soft_cap", "lrs_ssm")
_PLAN_INDEX = {name: index for index, name in enumerate(PLAN_OPS)}


class _Recording(threading.local):
    """The recording that is open on this thread, if any: launches made on another thread (a second runner, a
    sampler) are none of its business."""
    calls: list | None = None


_recording = _Recording()


class Plan:
    """A recorded sequence of launches, ready for plan_run()."""

    def __init__(self, calls: list):
        words: list[int] = []
        for name, args in calls:
            argtypes = _SIGNATURES[name][1][:-1]
            words.append(_PLAN_INDEX[name])
            for kind, value in zip(argtypes, args):
                if kind is c_float:
                    words.append(int.from_bytes(struct.pack("<f", value), "little"))
                elif value is None:
                    words.append(0)
                else:
                    words.append(int(value) & 0xFFFFFFFFFFFFFFFF)
        self.launches = len(calls)
        self.words = (ctypes.c_uint64 * max(len(words), 1))(*words)
        self.length = len(words)


def record_begin() -> None:
    """Start writing down the launches this thread makes (they still run as they are made)."""
    if _recording.calls is not None:
        raise KernelError("a recording of launches is already open")
    _recording.calls = []


def record_end() -> Plan:
    """Stop writing launches down; returns the plan of those made since record_begin()."""
    if _recording.calls is None:
        raise KernelError("no recording of launches is open")
    calls, _recording.calls = _recording.calls, None
    return Plan(calls)


def record_drop() -> None:
    """Stop writing launches down and forget them (after a failure)."""
    _recording.calls = None


def plan_run(plan: Plan) -> None:
    """Make the plan's launches, in order, on the current stream."""
    if plan.launches:
        _check(library().lrs_plan_run(plan.words, plan.length, plan.launches, _stream()))


def _launch(name: str, *args) -> None:
    code = getattr(_lib or library(), name)(*args)
    if code != 0:
        raise KernelError(library().lrs_last_error().decode())
    if _recording.calls is not None:
        if name not in _PLAN_INDEX:
            raise KernelError(f"{name} cannot be part of a recorded plan")
        _recording.calls.append((name, args[:-1]))


def loaded_library_path() -> str:
    library()
    return _lib_path


def _check(code: int) -> None:
    if code != 0:
        raise KernelError(library().lrs_last_error().decode())


# The handle of the current stream is asked for at every kernel launch; the raw query costs a
# fraction of a microsecond where torch.cuda.current_stream() builds an object in about nine.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"kernels take float32 or bfloat16, got {dtype}")


def _need(cond: bool, message: str) -> None:
    if not cond:
        raise KernelError(message)


def _dev(t: torch.Tensor, name: str, dtype=None) -> int:
    _need(isinstance(t, torch.Tensor) and t.is_cuda, f"{name} must be a device tensor")
    if dtype is not None:
        _need(t.dtype == dtype, f"{name} must be {dtype}, got {t.dtype}")
    return t.data_ptr()


def pinned_device_address(t: torch.Tensor) -> int:
    """The address under which kernels see the pinned host tensor `t`.  The owner of the tensor asks
    once and keeps the answer with the tensor (asking whether memory is pinned is slow)."""
    _need(not t.is_cuda and t.is_contiguous() and t.is_pinned(), "pinned_device_address needs a contiguous pinned host tensor")
    out = c_void_p()
    _check(library().lrs_host_device_pointer(t.data_ptr(), byref(out)))
    return out.value


def _rows(t: torch.Tensor, name: str) -> int:
    """Row stride of a 2-D tensor whose rows are contiguous."""
    _need(t.dim() == 2 and t.stride(1) == 1, f"{name} must be 2-D with contiguous rows, got shape {tuple(t.shape)} strides {t.stride()}")
    return t.stride(0)


def device_arch(device: int = 0) -> tuple[str, int]:
    buf = ctypes.create_string_buffer(256)
    cus = c_int(0)
    _check(library().lrs_device_arch(device, buf, 256, byref(cus)))
    return buf.value.decode(), cus.value


# ----------------------------------------------------------------- graphs
def graph_begin() -> None:
    _check(library().lrs_graph_begin(_stream()))


def graph_end() -> int:
    handle = c_void_p()
    _check(library().lrs_graph_end(_stream(), byref(handle)))
    return handle.value


def graph_launch(handle: int) -> None:
    _check(library().lrs_graph_launch(handle, _stream()))


def graph_destroy(handle: int) -> None:
    library().lrs_graph_destroy(handle)


def copy_h2d(dst: torch.Tensor, src: torch.Tensor, count: int) -> None:
    """Asynchronous copy of the first `count` elements of `src` into device `dst`.  `src` must be
    pinned host memory (the caller checks that once, when it allocates it: asking is slow)."""
    _need(src.device.type == "cpu" and src.is_contiguous() and dst.is_contiguous(), "copy_h2d needs a contiguous host source and a contiguous destination")
    _need(src.dtype == dst.dtype and 0 < count <= src.numel() and count <= dst.numel(), "copy_h2d: size or dtype mismatch")
    _launch("lrs_copy_h2d", _dev(dst, "dst"), src.data_ptr(), count * src.element_size(), _stream())


def copy_h2d_scatter(dst: torch.Tensor, src: torch.Tensor, count: int, tables: torch.Tensor, pairs_at: int, pairs: int) -> None:
    """copy_h2d() of the first `count` int32 elements (a multiple of 4) of pinned `src`, and in the same launch the `pairs`
    (offset, value) pairs that lie in `src` from element `pairs_at` (even) on written into `tables` (int32, on the
    device): tables.view(-1)[offset] = value.  The caller has checked the offsets."""
    _need(src.device.type == "cpu" and src.is_contiguous() and dst.is_contiguous() and src.dtype == dst.dtype == torch.int32,
          "copy_h2d_scatter needs contiguous int32 tensors, the source on the host")
    _need(0 <= count <= src.numel() and count <= dst.numel() and count % 4 == 0, "copy_h2d_scatter: the count must be a multiple of 4 inside both tensors (0: only the pairs)")
    _need(tables.dtype == torch.int32 and tables.is_contiguous() and pairs > 0 and pairs_at % 2 == 0 and pairs_at + 2 * pairs <= src.numel(),
          "copy_h2d_scatter: int32 tables and pairs inside the source, from an even element on")
    _launch("lrs_copy_h2d_scatter", _dev(dst, "dst"), src.data_ptr(), count * 4, _dev(tables, "tables"), pairs_at * 4, pairs, _stream())


def stream_read(src: torch.Tensor, sink: torch.Tensor, blocks: int) -> None:
    """Reads all of `src` once with `blocks` workgroups (a probe of the memory rate a kernel can reach)."""
    _need(src.is_contiguous() and sink.dtype == torch.int32 and sink.numel() >= blocks, "stream_read: contiguous source and an int32 sink of `blocks` elements")
    _launch("lrs_stream_read", _dev(src, "src"), src.numel() * src.element_size(), _dev(sink, "sink"), blocks, _stream())



def probe_lds(sink: torch.Tensor, blocks: int, iters: int, stride: int) -> None:
    """`blocks` workgroups read LDS `iters` x 8 times, 16 bytes a lane, rows `stride` bytes apart (microbench lds)."""
    _need(sink.dtype == torch.int32 and sink.numel() >= 256, "probe_lds: an int32 sink of 256 elements")
    _launch("lrs_probe_lds", _dev(sink, "sink"), blocks, iters, stride, _stream())


def probe_lines(data: torch.Tensor, sink: torch.Tensor, blocks: int, threads: int, bytes_each: int, pattern: int) -> None:
    """Measurement only: `blocks` workgroups stream `bytes_each` bytes each of `data` with 16-byte loads in the lane
    order `pattern` (0 fragment order, 1 whole lines, 2 a row to four neighbouring lanes)."""
    _need(sink.dtype == torch.int32 and sink.numel() >= 256, "probe_lines: an int32 sink of 256 elements")
    _need(data.is_contiguous(), "probe_lines: data must be contiguous")
    _launch("lrs_probe_lines", _dev(data, "data"), data.numel() * data.element_size(), _dev(sink, "sink"), blocks, threads, bytes_each, pattern, _stream())


def probe_mfma(sink: torch.Tensor, blocks: int, iters: int, valu: int, exps: bool) -> None:
    """`blocks` workgroups issue `iters` x 32 matrix instructions with `valu` multiply-adds after each (microbench mfma)."""
    _need(sink.dtype == torch.float32 and sink.numel() >= 256, "probe_mfma: a float32 sink of 256 elements")
    _launch("lrs_probe_mfma", _dev(sink, "sink"), blocks, iters, valu, int(bool(exps)), _stream())

def copy_to_pinned(dst: torch.Tensor, src: torch.Tensor, count: int) -> None:
    """The first `count` elements of device `src` into pinned host `dst`, by a kernel (the host reads
    them after synchronising the stream).  count * element size must be a multiple of 16."""
    _need(dst.device.type == "cpu" and dst.is_contiguous() and src.is_contiguous(), "copy_to_pinned needs a contiguous pinned host destination and a contiguous source")
    _need(src.dtype == dst.dtype and 0 < count <= src.numel() and count <= dst.numel(), "copy_to_pinned: size or dtype mismatch")
    _launch("lrs_copy_to_pinned", dst.data_ptr(), _dev(src, "src"), count * src.element_size(), _stream())


# ------------------------------------------------------------ elementwise
def embed(out: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, multiplier: float = 1.0) -> None:
    tokens, hidden = out.shape
    _need(out.is_contiguous() and table.is_contiguous() and table.dim() == 2 and table.shape[1] == hidden, "embed: out [T,H] and table [V,H] must agree")
    _need(ids.dtype == torch.int32 and ids.numel() >= tokens and ids.is_contiguous(), "embed: ids must be int32 [T]")
    _launch("lrs_embed", _dev(out, "out", torch.float32), _dev(table, "table"), dtype_code(table.dtype),
                               _dev(ids, "ids"), tokens, hidden, multiplier, _stream())


def rmsnorm(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float, rows: torch.Tensor | None = None) -> None:
    n_rows, hidden = out.shape
    _need(out.is_contiguous() and x.is_contiguous() and x.dim() == 2 and x.shape[1] == hidden, "rmsnorm: out and x must be contiguous [*, H]")
    _need(weight.is_contiguous() and weight.numel() == hidden, f"rmsnorm: weight must hold {hidden} values")
    if rows is None:
        _need(x.shape[0] >= n_rows, "rmsnorm: x has fewer rows than out")
    else:
        _need(rows.dtype == torch.int32 and rows.numel() >= n_rows and rows.is_contiguous(), "rmsnorm: rows must be int32")
    _launch("lrs_rmsnorm", _dev(out, "out"), dtype_code(out.dtype), _dev(x, "x", torch.float32), _dev(weight, "weight"),
                                 dtype_code(weight.dtype), None if rows is None else _dev(rows, "rows"), n_rows, hidden, eps, _stream())


def add_rmsnorm(out: torch.Tensor, x: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float) -> None:
    """x += y (float32 residual stream, bf16 addend), then out = RMSNorm(x) with `weight`, in one pass."""
    n_rows, hidden = x.shape
    _need(x.dtype == torch.float32 and x.is_contiguous() and y.dtype == torch.bfloat16 and y.is_contiguous() and y.shape == x.shape,
          "add_rmsnorm: x must be contiguous float32 [T, H] and y bf16 of the same shape")
    _need(out.is_contiguous() and out.shape == x.shape, "add_rmsnorm: out must be contiguous [T, H]")
    _need(weight.is_contiguous() and weight.numel() == hidden, f"add_rmsnorm: weight must hold {hidden} values")
    _launch("lrs_add_rmsnorm", _dev(out, "out"), dtype_code(out.dtype), _dev(x, "x"), _dev(y, "y"), _dev(weight, "weight"),
                                     dtype_code(weight.dtype), n_rows, hidden, eps, _stream())


def round_rows(out: torch.Tensor, x: torch.Tensor) -> None:
    """out = the float32 rows x in out's dtype (the residual stream as the activation a sublayer reads)."""
    _need(x.dtype == torch.float32 and x.is_contiguous() and out.is_contiguous() and out.shape == x.shape, "round_rows: out and x must be contiguous and of one shape")
    _launch("lrs_round_rows", _dev(out, "out"), dtype_code(out.dtype), _dev(x, "x"), x.numel(), _stream())


def _rounded(rounded: torch.Tensor | None, rows: int, hidden: int, who: str):
    if rounded is None:
        return None
    _need(rounded.dtype == torch.bfloat16 and rounded.is_contiguous() and rounded.shape == (rows, hidden), f"{who}: the rounded rows must be contiguous bfloat16 [T, H]")
    return _dev(rounded, "rounded")


def norm_add(residual: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float, rounded: torch.Tensor | None = None) -> None:
    """residual += weight * y * rsqrt(mean(y^2) + eps), row by row, in float32: the norm of a sublayer's output added to the
    stream.  rounded: bfloat16 [T, H] that receives the updated rows as well."""
    n_rows, hidden = y.shape
    _need(residual.dtype == torch.float32 and y.dtype == torch.float32 and residual.is_contiguous() and y.is_contiguous()
          and residual.shape[0] >= n_rows and residual.shape[1] == hidden, "norm_add: residual and y must be contiguous float32 [T, H]")
    _need(weight.is_contiguous() and weight.numel() == hidden, f"norm_add: weight must hold {hidden} values")
    _launch("lrs_norm_add", _dev(residual, "residual"), _dev(y, "y"), _dev(weight, "weight"), dtype_code(weight.dtype), n_rows, hidden, eps,
            _rounded(rounded, n_rows, hidden, "norm_add"), _stream())


def layernorm(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float, rows: torch.Tensor | None = None) -> None:
    """out = weight * (x - mean) / sqrt(variance + eps) per float32 row of x (of the rows listed in `rows` if given)."""
    n_rows, hidden = out.shape
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.shape[1] == hidden and x.is_contiguous() and out.is_contiguous(), "layernorm: x must be contiguous float32 [*, H] and out [rows, H]")
    _need(weight.is_contiguous() and weight.numel() == hidden, f"layernorm: weight must hold {hidden} values")
    if rows is None:
        _need(x.shape[0] >= n_rows, "layernorm: x has fewer rows than out")
    else:
        _need(rows.dtype == torch.int32 and rows.numel() >= n_rows and rows.is_contiguous(), "layernorm: rows must be int32")
    _launch("lrs_layernorm", _dev(out, "out"), dtype_code(out.dtype), _dev(x, "x"), _dev(weight, "weight"), dtype_code(weight.dtype),
            None if rows is None else _dev(rows, "rows"), n_rows, hidden, eps, _stream())


def scale_add_layernorm(residual: torch.Tensor, y: torch.Tensor, alpha: float, weight: torch.Tensor, eps: float,
                        rounded: torch.Tensor | None = None) -> None:
    """residual = layer norm (weight, eps) of alpha * residual + y, float32 rows in place; rounded: bfloat16 [T, H] that
    receives the new rows as well."""
    n_rows, hidden = residual.shape
    _need(residual.dtype == torch.float32 and y.dtype == torch.float32 and y.shape == residual.shape and residual.is_contiguous() and y.is_contiguous(),
          "scale_add_layernorm: residual and y must be contiguous float32 of one shape")
    _need(weight.is_contiguous() and weight.numel() == hidden, f"scale_add_layernorm: weight must hold {hidden} values")
    _launch("lrs_scale_add_layernorm", _dev(residual, "residual"), _dev(y, "y"), alpha, _dev(weight, "weight"), dtype_code(weight.dtype), n_rows,
            hidden, eps, _rounded(rounded, n_rows, hidden, "scale_add_layernorm"), _stream())


def soft_cap(x: torch.Tensor, cap: float) -> None:
    """x = cap * tanh(x / cap), in place on contiguous float32 values."""
    _need(x.dtype == torch.float32 and x.is_contiguous() and x.numel() > 0, "soft_cap: x must be contiguous float32")
    _launch("lrs_soft_cap", _dev(x, "x"), x.numel(), cap, _stream())


def rope_table(cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor, magnitude: float = 1.0) -> None:
    """cos, sin [T, half] = magnitude * cos / sin of (position * inv_freq), float32."""
    tokens, half = cos.shape
    _need(cos.is_contiguous() and sin.is_contiguous() and sin.shape == cos.shape, "rope_table: cos and sin must be contiguous [T, half]")
    _need(inv_freq.numel() == half and inv_freq.is_contiguous(), "rope_table: inv_freq must hold `half` values")
    _need(positions.dtype == torch.int32 and positions.numel() >= tokens and positions.is_contiguous(), "rope_table: positions must be int32 [T]")
    _launch("lrs_rope_table", _dev(cos, "cos", torch.float32), _dev(sin, "sin", torch.float32), _dev(positions, "positions"),
                                    _dev(inv_freq, "inv_freq", torch.float32), tokens, half, magnitude, _stream())


def qk_prep(qkv: torch.Tensor, nq: int, nkv: int, d: int, q_weight, k_weight, eps: float, cos, sin,
            k_pages, v_pages, slots, page_size: int, skip_q: bool = False) -> None:
    """Normalise and rotate the q and k heads of `qkv` [T, (nq+2*nkv)*d]; q in place, k and v into pages.
    skip_q: the q heads are left as they are (attention_prefill() with `prepare` takes them raw)."""
    tokens = qkv.shape[0]
    stride = _rows(qkv, "qkv")
    _need(qkv.shape[1] == (nq + 2 * nkv) * d, f"qk_prep: qkv width {qkv.shape[1]} is not (nq+2nkv)*d = {(nq + 2 * nkv) * d}")
    rot_half = 0
    if cos is not None:
        rot_half = cos.shape[1]
        _need(cos.shape[0] >= tokens and sin.shape == cos.shape and cos.is_contiguous() and sin.is_contiguous(), "qk_prep: rotary tables must be [T, half]")
        _need(cos.dtype == torch.float32 and sin.dtype == torch.float32, "qk_prep: rotary tables must be float32")
    w_dtype = qkv.dtype
    if q_weight is not None:
        _need(k_weight is not None and q_weight.numel() == d and k_weight.numel() == d and q_weight.dtype == k_weight.dtype, "qk_prep: q/k norm weights must both hold head_dim values")
        w_dtype = q_weight.dtype
    if nkv > 0:
        _need(k_pages.dim() == 4 and k_pages.shape[1:] == (nkv, page_size, d) and v_pages.shape == (k_pages.shape[0], nkv, d, page_size),
              f"qk_prep: key pages must be [pages, {nkv}, {page_size}, {d}] and value pages [pages, {nkv}, {d}, {page_size}]")
        _need(k_pages.is_contiguous() and v_pages.is_contiguous() and k_pages.dtype == qkv.dtype and v_pages.dtype == qkv.dtype, "qk_prep: pages must be contiguous and of the activation dtype")
        _need(slots.dtype == torch.int32 and slots.numel() >= tokens and slots.is_contiguous(), "qk_prep: slots must be int32 [T]")
    _launch("lrs_qk_prep", 
        _dev(qkv, "qkv"), dtype_code(qkv.dtype), tokens, stride, nq, nkv, d,
        None if q_weight is None else _dev(q_weight, "q_weight"), None if k_weight is None else _dev(k_weight, "k_weight"),
        dtype_code(w_dtype), eps, None if cos is None else cos.data_ptr(), None if sin is None else sin.data_ptr(), rot_half,
        None if nkv == 0 else _dev(k_pages, "k_pages"), None if nkv == 0 else _dev(v_pages, "v_pages"),
        None if nkv == 0 else _dev(slots, "slots"), page_size, int(bool(skip_q)), _stream())


@functools.lru_cache(maxsize=1)
def gemm_workspace_bytes() -> int:
    """Bytes of device memory a caller brings as `workspace` to the products that divide K between workgroups."""
    return int(library().lrs_gemm_workspace_bytes())


def _workspace(t: torch.Tensor | None, name: str) -> tuple:
    """(address, bytes) of a caller's workspace for the sums of K splits; (None, 0): the one the process keeps, which
    all callers that bring none share (their products must then stay on one stream)."""
    if t is None:
        return None, 0
    if isinstance(t, tuple):            # (address, bytes) that workspace_address() has checked before
        return t
    _need(t.is_cuda and t.is_contiguous() and t.numel() * t.element_size() >= gemm_workspace_bytes(),
          f"{name}: the workspace must be a contiguous device tensor of at least {gemm_workspace_bytes()} bytes")
    return t.data_ptr(), t.numel() * t.element_size()


def workspace_address(t: torch.Tensor) -> tuple:
    """(address, bytes) of a workspace tensor, checked once: callers that make many products a step pass this on as
    `workspace` instead of the tensor."""
    return _workspace(t, "workspace")


def gemm_mid_qk_prep_takes(dtype: torch.dtype, m: int, nq: int, nkv: int, d: int, k: int, rot_half: int,
                           choice: KernelChoice = DEFAULT_CHOICE) -> bool:
    """Whether gemm_mid_qk_prep() takes the shape: bf16, 17..128 rows, heads the vector form of qk_prep takes
    (head_dim 16, 32, 64, ... 1024, rotation over the whole head or none), cache written by this layer."""
    per_head = d // 16
    return (gemm_mid_takes(dtype, m, (nq + 2 * nkv) * d, k, MID_ROWS_PREFERRED, choice) and nkv > 0 and d % 16 == 0 and 0 < per_head <= 64
            and per_head & (per_head - 1) == 0 and rot_half in (0, d // 2))


def gemm_mid_qk_prep(qkv: torch.Tensor, a: torch.Tensor, w: torch.Tensor, sumsq: torch.Tensor | None, in_eps: float, nq: int, nkv: int,
                     d: int, q_weight, k_weight, eps: float, cos, sin, k_pages, v_pages, slots, page_size: int,
                     choice: KernelChoice = DEFAULT_CHOICE, workspace: torch.Tensor | None = None) -> None:
    """The q/k/v product of 17..128 bf16 rows (a @ w.T; with `sumsq` the input is a norm begun before it, as in
    gemm_mid_scaled) and qk_prep() of its result in two kernels: the one that prepares the heads adds up the sums of
    the product's K splits itself.  q goes into `qkv` [M, (nq+2*nkv)*d], k and v into the pages."""
    m, k = a.shape
    n = (nq + 2 * nkv) * d
    rot_half = 0 if cos is None else cos.shape[1]
    _need(a.dtype == torch.bfloat16 and gemm_mid_qk_prep_takes(w.dtype, m, nq, nkv, d, k, rot_half, choice), "gemm_mid_qk_prep: shape not taken (see gemm_mid_qk_prep_takes)")
    _need(w.shape == (n, k) and w.is_contiguous(), f"gemm_mid_qk_prep: weight must be contiguous [{n}, {k}]")
    _need(qkv.dtype == torch.bfloat16 and qkv.shape == (m, n), f"gemm_mid_qk_prep: qkv must be bf16 [{m}, {n}]")
    if sumsq is not None:
        _need(sumsq.dtype == torch.float32 and sumsq.dim() == 2 and sumsq.shape[1] == m and sumsq.is_contiguous() and in_eps > 0, f"gemm_mid_qk_prep: sumsq must be float32 [parts, {m}] and its eps positive")
    if cos is not None:
        _need(cos.shape[0] >= m and sin.shape == cos.shape and cos.is_contiguous() and sin.is_contiguous() and cos.dtype == torch.float32 and sin.dtype == torch.float32,
              "gemm_mid_qk_prep: rotary tables must be float32 [T, half]")
    w_dtype = torch.bfloat16
    if q_weight is not None:
        _need(k_weight is not None and q_weight.numel() == d and k_weight.numel() == d and q_weight.dtype == k_weight.dtype, "gemm_mid_qk_prep: q/k norm weights must both hold head_dim values")
        w_dtype = q_weight.dtype
    _need(k_pages.dim() == 4 and k_pages.shape[1:] == (nkv, page_size, d) and v_pages.shape == (k_pages.shape[0], nkv, d, page_size),
          f"gemm_mid_qk_prep: key pages must be [pages, {nkv}, {page_size}, {d}] and value pages [pages, {nkv}, {d}, {page_size}]")
    _need(k_pages.is_contiguous() and v_pages.is_contiguous() and k_pages.dtype == torch.bfloat16 and v_pages.dtype == torch.bfloat16, "gemm_mid_qk_prep: pages must be contiguous bf16")
    _need(slots.dtype == torch.int32 and slots.numel() >= m and slots.is_contiguous(), "gemm_mid_qk_prep: slots must be int32 [T]")
    _launch("lrs_gemm_mid_qk_prep", 
        _dev(qkv, "qkv"), _rows(qkv, "qkv"), _dev(a, "a"), _dev(w, "w"), m, k, _rows(a, "a"),
        None if sumsq is None else _dev(sumsq, "sumsq"), 0 if sumsq is None else sumsq.shape[0], in_eps if sumsq is not None else 0.0,
        nq, nkv, d, None if q_weight is None else _dev(q_weight, "q_weight"), None if k_weight is None else _dev(k_weight, "k_weight"),
        dtype_code(w_dtype), eps, None if cos is None else cos.data_ptr(), None if sin is None else sin.data_ptr(), rot_half,
        _dev(k_pages, "k_pages"), _dev(v_pages, "v_pages"), _dev(slots, "slots"), page_size, choice.word,
        *_workspace(workspace, "gemm_mid_qk_prep"), _stream())


def silu_mul(out: torch.Tensor, gate_up: torch.Tensor, interleaved: bool = False) -> None:
    """out = silu(gate) * up; gate_up holds [gate | up], or groups of 8 gate then 8 up columns if `interleaved`."""
    tokens, inter = out.shape
    _need(out.is_contiguous() and gate_up.is_contiguous() and gate_up.shape == (tokens, 2 * inter) and gate_up.dtype == out.dtype, "silu_mul: gate_up must be [T, 2I] and out [T, I], same dtype")
    _launch("lrs_silu_mul", _dev(out, "out"), _dev(gate_up, "gate_up"), dtype_code(out.dtype), tokens, inter, 1 if interleaved else 0, _stream())


def add_into(residual: torch.Tensor, y: torch.Tensor) -> None:
    """residual (float32) += y, same shape, both contiguous."""
    _need(residual.dtype == torch.float32 and residual.shape == y.shape and residual.is_contiguous() and y.is_contiguous(), "add_into: float32 residual and y of one contiguous shape needed")
    _launch("lrs_add_into", _dev(residual, "residual"), _dev(y, "y"), dtype_code(y.dtype), residual.numel(), _stream())


@functools.lru_cache(maxsize=4096)
def gemm_lines_width(m: int, n: int, k: int) -> int:
    """The tile width (256, 192 or 128 weight rows) the many-rows kernel with slices of whole lines would take
    for out [m, n] = x [m, k] w[n, k]^T, or 0 if that kernel does not take the product."""
    return int(library().lrs_gemm_lines_width(m, n, k))


@functools.lru_cache(maxsize=4096)
def gemm_lines_splits(m: int, n: int, k: int) -> int:
    """Into how many parts the many-rows kernel with slices of whole lines divides K for a product with too few
    tiles of 256 x 128 to go round the compute units (1: the tiles as they are), or 0 if it does not take the
    product that way."""
    return int(library().lrs_gemm_lines_splits(m, n, k))


@functools.lru_cache(maxsize=4096)
def gemm_split_pays(m: int, n: int, k: int) -> bool:
    """Whether a bfloat16 product of more than 128 rows is faster by this package's many-rows kernel with K divided
    between workgroups than by the vendor library (a rule from measurements, see `lrs_gemm_lines_split_pays`)."""
    return bool(library().lrs_gemm_lines_split_pays(m, n, k))


def few_rows_capacity() -> int:
    """Most rows the few-rows product kernel takes at all (callers use it up to KernelChoice.few_rows_max)."""
    return library().lrs_gemm_skinny_capacity()


def gemm_mid_shape(n: int, k: int, choice: KernelChoice = DEFAULT_CHOICE) -> tuple[int, int]:
    """(waves a workgroup, K splits) the kernel for 17..128 rows takes for a weight matrix [n, k]."""
    waves, splits = c_int(0), c_int(0)
    _check(library().lrs_gemm_mid_shape(n, k, choice.word, ctypes.addressof(waves), ctypes.addressof(splits)))
    return waves.value, splits.value


def gemm_mid_deal(m: int, n: int, k: int, choice: KernelChoice = DEFAULT_CHOICE) -> tuple[int, int, int, int]:
    """(waves a workgroup, K splits, workgroups along n, how many of them have 16 rows more than 16 * waves) for a
    product of m rows (17..128) with a weight matrix [n, k]."""
    waves, splits, groups, extras = c_int(0), c_int(0), c_int(0), c_int(0)
    _check(library().lrs_gemm_mid_deal(m, n, k, choice.word, ctypes.addressof(waves), ctypes.addressof(splits), ctypes.addressof(groups),
                                       ctypes.addressof(extras)))
    return waves.value, splits.value, groups.value, extras.value


# Rows up to which callers that may use the vendor library take this package's kernel for 17..128 rows instead.
# Measured on MI355X in whole decode steps (Qwen3-8B shape): 4-6 % faster than the library's products at
# batches of 24..64; at 128 rows a layer's four products take 141 us against 169 us (and a separate gated
# activation), only the LM head is slower (320 against 279 us).
MID_ROWS_PREFERRED = 128


def gemm_mid_takes(dtype: torch.dtype, m: int, n: int, k: int, most: int = 128, choice: KernelChoice = DEFAULT_CHOICE) -> bool:
    """Whether a product of m rows (at most `most`) can go to the kernel for 17..128 rows (weights streamed
    once, activations shared through LDS), which also writes the gated activation itself."""
    return dtype == torch.bfloat16 and 16 < m <= min(most, 128) and k % 256 == 0 and n % 16 == 0 and choice.mid


def norm_begin_parts(n: int) -> int:
    """Partial sums of squares per row that gemm_mid_add_norm_begin() leaves for a norm over n columns."""
    return library().lrs_norm_begin_parts(n)


def gemm_mid_add_norm_begin(residual: torch.Tensor, a: torch.Tensor, w: torch.Tensor, norm_weight: torch.Tensor,
                            next_x: torch.Tensor, next_sumsq: torch.Tensor, choice: KernelChoice = DEFAULT_CHOICE,
                            workspace: torch.Tensor | None = None) -> None:
    """residual (float32 [M, N]) += a @ w.T for 17..128 bf16 rows, and the first half of the RMSNorm that follows:
    next_x [M, N] = bf16(residual * norm_weight), next_sumsq [norm_begin_parts(N), M] = partial sums of residual^2.
    gemm_mid_scaled() (or scale_rows()) finishes the norm."""
    m, k = a.shape
    n = w.shape[0]
    _need(gemm_mid_takes(w.dtype, m, n, k, 128, choice) and a.dtype == torch.bfloat16, "gemm_mid_add_norm_begin: takes bf16 products of 17..128 rows, K % 256 == 0, N % 16 == 0")
    _need(w.dim() == 2 and w.is_contiguous() and w.shape[1] == k, f"gemm_mid_add_norm_begin: weight must be contiguous [N, {k}]")
    _need(residual.dtype == torch.float32 and residual.is_contiguous() and residual.shape == (m, n), f"gemm_mid_add_norm_begin: residual must be contiguous float32 [{m}, {n}]")
    _need(next_x.dtype == torch.bfloat16 and next_x.is_contiguous() and next_x.shape == (m, n), f"gemm_mid_add_norm_begin: next_x must be contiguous bf16 [{m}, {n}]")
    _need(next_sumsq.dtype == torch.float32 and next_sumsq.is_contiguous() and next_sumsq.shape == (norm_begin_parts(n), m),
          f"gemm_mid_add_norm_begin: next_sumsq must be contiguous float32 [{norm_begin_parts(n)}, {m}]")
    _need(norm_weight.is_contiguous() and norm_weight.numel() == n, f"gemm_mid_add_norm_begin: norm weight must hold {n} values")
    _launch("lrs_gemm_mid_add_norm_begin", _dev(residual, "residual"), _dev(a, "a"), _dev(w, "w"), _dev(norm_weight, "norm_weight"),
                                                 dtype_code(norm_weight.dtype), _dev(next_x, "next_x"), _dev(next_sumsq, "next_sumsq"),
                                                 m, n, k, _rows(a, "a"), choice.word, *_workspace(workspace, "gemm_mid_add_norm_begin"), _stream())


def gemm_mid_scaled(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, sumsq: torch.Tensor, eps: float, swiglu: bool = False,
                    choice: KernelChoice = DEFAULT_CHOICE, workspace: torch.Tensor | None = None) -> None:
    """out = (the RMSNorm that `a` and `sumsq` stand for) @ w.T for 17..128 rows: a = bf16(h * norm weight) [M, K],
    sumsq [parts, M] partial sums of h^2; row r of the product is multiplied by rsqrt(sum_p sumsq[p, r] / K + eps).
    swiglu as in gemm()."""
    m, k = a.shape
    n = w.shape[0]
    _need(gemm_mid_takes(w.dtype, m, n, k, 128, choice) and a.dtype == torch.bfloat16, "gemm_mid_scaled: takes bf16 products of 17..128 rows, K % 256 == 0, N % 16 == 0")
    _need(w.dim() == 2 and w.is_contiguous() and w.shape[1] == k, f"gemm_mid_scaled: weight must be contiguous [N, {k}]")
    _need(out.shape == (m, n // 2 if swiglu else n), f"gemm_mid_scaled: out must be [{m}, {n // 2 if swiglu else n}], got {tuple(out.shape)}")
    _need(out.dtype in (torch.bfloat16, torch.float32) and not (swiglu and out.dtype != torch.bfloat16), "gemm_mid_scaled: output must be bf16, or float32 without swiglu")
    _need(sumsq.dtype == torch.float32 and sumsq.dim() == 2 and sumsq.shape[1] == m and sumsq.is_contiguous() and eps > 0, f"gemm_mid_scaled: sumsq must be float32 [parts, {m}] and eps positive")
    mode = OUT_STORE if out.dtype == torch.bfloat16 else OUT_STORE_F32
    _launch("lrs_gemm_mid_scaled", _dev(out, "out"), mode, _dev(a, "a"), _dev(w, "w"), m, n, k, _rows(a, "a"), _rows(out, "out"),
                                         int(swiglu), _dev(sumsq, "sumsq"), sumsq.shape[0], eps, choice.word,
                                         *_workspace(workspace, "gemm_mid_scaled"), _stream())


def _int_vector(t: torch.Tensor, name: str, at_least: int) -> int:
    _need(t.dtype == torch.int32 and t.is_contiguous() and t.numel() >= at_least, f"{name} must be contiguous int32 with at least {at_least} elements")
    return _dev(t, name)


def advance_decode(token_ids: torch.Tensor, positions: torch.Tensor, token_request: torch.Tensor, seq_lens: torch.Tensor,
                   chosen: torch.Tensor, real_rows: torch.Tensor, draws: torch.Tensor | None = None) -> None:
    """A decode step's metadata moved on to the next step, on the device: the first real_rows[0] rows
    take the tokens in `chosen`, move one position on, lengthen their requests by one and (with
    `draws`, the counters of seeded sampling) count one more draw."""
    rows = token_ids.numel()
    _launch("lrs_advance_decode", _int_vector(token_ids, "token_ids", rows), _int_vector(positions, "positions", rows),
                                        _int_vector(token_request, "token_request", rows), _int_vector(seq_lens, "seq_lens", 1),
                                        _int_vector(chosen, "chosen", rows), None if draws is None else _int_vector(draws, "draws", rows),
                                        _int_vector(real_rows, "real_rows", 1), rows, _stream())


def advance_slots(slots: torch.Tensor, positions: torch.Tensor, token_request: torch.Tensor, block_table: torch.Tensor,
                  page_size: int, real_rows: torch.Tensor) -> None:
    """The cache slots of the (already advanced) positions of the first real_rows[0] rows, from the block table."""
    rows = slots.numel()
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.stride(1) == 1, "advance_slots: block_table must be int32 [R, blocks]")
    _launch("lrs_advance_slots", _int_vector(slots, "slots", rows), _int_vector(positions, "positions", rows),
                                       _int_vector(token_request, "token_request", rows), _dev(block_table, "block_table"),
                                       block_table.stride(0), page_size, _int_vector(real_rows, "real_rows", 1), rows, _stream())


def step_prepare_summary_size() -> int:
    return library().lrs_step_prepare_summary_size()


def step_prepare(meta, offsets, entries: int, packed, tokens_at: int, wants_at: int, pad_to: int, trash_slot: int, tables,
                 groups: int, max_blocks: int, page_size: int, query_group: int, summary) -> None:
    """Fill a step's metadata in the staging buffer `meta` (a numpy int32 view of pinned memory) on the host: see
    csrc/prepare.hip.  `packed` (numpy int32) holds, `entries` values each, the entries' state slots, context lengths,
    token counts and numbers of wanted places, then from `tokens_at` all tokens and from `wants_at` all wanted places;
    `offsets` (numpy int64) where each array lies in `meta`; `tables` a ctypes array of the host block tables' addresses;
    `summary` (numpy int32) takes T, R, logit rows, query groups, largest group, longest portion, longest context and
    the single rows at the step's head."""
    base = packed.ctypes.data
    code = library().lrs_step_prepare(meta.ctypes.data, offsets.ctypes.data, entries, base, base + 4 * entries, base + 8 * entries,
                                      base + 4 * tokens_at, base + 12 * entries, base + 4 * wants_at, pad_to, trash_slot, groups,
                                      ctypes.cast(tables, c_void_p), max_blocks, page_size, query_group, summary.ctypes.data)
    if code != 0:
        raise KernelError(library().lrs_last_error().decode())


def fill_i32(dst: torch.Tensor, value: int) -> None:
    _need(dst.dtype == torch.int32 and dst.is_contiguous(), "fill_i32: int32 contiguous tensor needed")
    _launch("lrs_fill_i32", _dev(dst, "dst"), value, dst.numel(), _stream())


def scatter_i32(dst: torch.Tensor, pairs: torch.Tensor, count: int, first: int = 0) -> None:
    """dst.view(-1)[offset_i] = value_i for the `count` (offset, value) pairs that lie in `pairs` (int32, on the device)
    from element `first` on.  The caller has checked that every offset lies inside dst."""
    _need(dst.dtype == torch.int32 and dst.is_contiguous() and pairs.dtype == torch.int32 and pairs.is_contiguous()
          and first >= 0 and first % 2 == 0 and 0 < 2 * count <= pairs.numel() - first,
          "scatter_i32: int32 contiguous tensors and 2 * count values in pairs from an even element on needed")
    _launch("lrs_scatter_i32", _dev(dst, "dst"), _dev(pairs, "pairs") + 4 * first, count, _stream())


def gather_rows(out: torch.Tensor, x: torch.Tensor, rows: torch.Tensor) -> None:
    n_rows, hidden = out.shape
    _need(out.is_contiguous() and x.is_contiguous() and x.shape[1] == hidden, "gather_rows: shapes disagree")
    _need(rows.dtype == torch.int32 and rows.numel() >= n_rows, "gather_rows: rows must be int32")
    _launch("lrs_gather_rows", _dev(out, "out", torch.float32), _dev(x, "x", torch.float32), _dev(rows, "rows"), n_rows, hidden, _stream())


# ------------------------------------------------------------------- gemm
def gemm_fuses_norm(dtype: torch.dtype, m: int, k: int, choice: KernelChoice = DEFAULT_CHOICE) -> bool:
    """Whether gemm() can take the float32 residual stream and normalise it on the way in."""
    return dtype == torch.bfloat16 and m <= choice.few_rows_max and k % 8 == 0


def gemm_norm_fusion_pays(n: int) -> bool:
    """Every workgroup of the fused kernel normalises the whole input again, so the fusion costs
    more than the norm kernel it saves once the weight matrix has many rows (measured on MI355X:
    even at 6144 rows it only breaks even)."""
    return n <= 4096


def gemm(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None = None, accumulate: bool = False,
         swiglu: bool = False, norm_weight: torch.Tensor | None = None, eps: float = 0.0, rows: torch.Tensor | None = None,
         count: int | None = None, choice: KernelChoice = DEFAULT_CHOICE, workspace: torch.Tensor | None = None) -> None:
    """out = a @ w.T (+ bias).  `accumulate` adds into a float32 `out` instead of storing.

    workspace: the caller's own device memory (gemm_workspace_bytes()) for the sums of K splits, which some shapes
    leave for a second kernel; without it the process-wide one is used, which is safe on one stream only.

    norm_weight: `a` is the float32 residual stream [*, K]; the product is taken of its RMSNorm
    (weight norm_weight, eps), of the `count` rows listed in `rows` if given, else of its first rows.
    swiglu: `w` holds gate and up rows interleaved in groups of 8; out [M, N/2] = silu(gate) * up.
    """
    n, k = w.shape
    lda, ldc = _rows(a, "a"), _rows(out, "out")
    _need(w.dim() == 2 and w.is_contiguous() and a.shape[1] == k, f"gemm: weight must be contiguous [N, {a.shape[1]}], got {tuple(w.shape)}")
    normed = norm_weight is not None
    if normed:
        m = count if rows is not None else out.shape[0]
        _need(a.dtype == torch.float32 and gemm_fuses_norm(w.dtype, m, k, choice), f"gemm: the fused norm input needs a float32 input, bf16 weights and at most {choice.few_rows_max} rows")
        _need(norm_weight.numel() == k and norm_weight.is_contiguous() and eps > 0, "gemm: norm weight must hold K values and eps be positive")
        if rows is None:
            _need(a.shape[0] >= m, "gemm: input has fewer rows than the output")
        else:
            _need(rows.dtype == torch.int32 and rows.numel() >= m and rows.is_contiguous(), "gemm: rows must be int32")
    else:
        m = a.shape[0]
        _need(rows is None, "gemm: a row gather needs the fused norm input")
        _need(a.dtype == w.dtype, f"gemm: a is {a.dtype} but w is {w.dtype}")
    _need(out.shape == (m, n // 2 if swiglu else n), f"gemm: out must be [{m}, {n // 2 if swiglu else n}], got {tuple(out.shape)}")
    if accumulate:
        _need(out.dtype == torch.float32, "gemm: accumulation needs a float32 output")
        mode = OUT_ADD_F32
    elif out.dtype == w.dtype:
        mode = OUT_STORE
    else:
        _need(out.dtype == torch.float32, "gemm: output must be of the weight dtype or float32")
        mode = OUT_STORE_F32
    if bias is not None:
        _need(bias.numel() == n and bias.dtype == w.dtype and bias.is_contiguous(), "gemm: bias must hold N values of the weight dtype")
    if swiglu:
        _need(w.dtype == torch.bfloat16 and n % 16 == 0 and k % 8 == 0 and bias is None and mode == OUT_STORE, "gemm: swiglu needs bf16, N % 16 == 0, K % 8 == 0, no bias, a stored output")
    _launch("lrs_gemm", _dev(out, "out"), mode, _dev(a, "a"), _dev(w, "w"), None if bias is None else _dev(bias, "bias"),
                              dtype_code(w.dtype), m, n, k, lda, ldc, None if rows is None else _dev(rows, "rows"),
                              None if not normed else _dev(norm_weight, "norm_weight"), dtype_code(norm_weight.dtype) if normed else 0,
                              eps, 1 if swiglu else 0, choice.word, *_workspace(workspace, "gemm"), _stream())


def gemm_lines_add_rmsnorm(residual: torch.Tensor, a: torch.Tensor, w: torch.Tensor, norm_weight: torch.Tensor, eps: float,
                           normed: torch.Tensor, workspace: torch.Tensor | None = None) -> None:
    """residual (float32 [M, N]) += a @ w.T for more than 128 bf16 rows of a shape that gemm_lines_splits() takes, and
    normed [M, N] = RMSNorm(residual) with `norm_weight` and `eps`: the product with its K divided between workgroups,
    and one kernel that adds up their sums, adds them to the residual stream and normalises the rows."""
    m, k = a.shape
    n = w.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.shape == (n, k) and w.is_contiguous() and m > 128
          and gemm_lines_splits(m, n, k) >= 1, "gemm_lines_add_rmsnorm: takes bf16 products of more than 128 rows that gemm_lines_splits() takes")
    _need(residual.dtype == torch.float32 and residual.is_contiguous() and residual.shape == (m, n), f"gemm_lines_add_rmsnorm: residual must be contiguous float32 [{m}, {n}]")
    _need(normed.is_contiguous() and normed.shape == (m, n), f"gemm_lines_add_rmsnorm: normed must be contiguous [{m}, {n}]")
    _need(norm_weight.is_contiguous() and norm_weight.numel() == n and eps > 0 and n % 4 == 0 and n <= 8192,
          f"gemm_lines_add_rmsnorm: the norm weight must hold {n} values, eps be positive and N a multiple of 4 up to 8192")
    _launch("lrs_gemm_lines_add_rmsnorm", _dev(residual, "residual"), _dev(a, "a"), _dev(w, "w"), m, n, k, _rows(a, "a"),
            _dev(norm_weight, "norm_weight"), dtype_code(norm_weight.dtype), eps, _dev(normed, "normed"), dtype_code(normed.dtype),
            *_workspace(workspace, "gemm_lines_add_rmsnorm"), _stream())


def library_gemm(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor) -> None:
    """out [M, N] = a [M, K] @ w[N, K].T by the vendor's matrix library (bfloat16 inputs, float32 sums; out bfloat16
    or float32): for products of more rows than this package's own kernels are made for."""
    m, k = a.shape
    n = w.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[1] == k and w.is_contiguous(),
          f"library_gemm: a and w must be bfloat16, w contiguous [N, {k}]")
    _need(out.shape == (m, n) and out.dtype in (torch.bfloat16, torch.float32), f"library_gemm: out must be bfloat16 or float32 [{m}, {n}]")
    _launch("lrs_library_gemm", _dev(out, "out"), 1 if out.dtype == torch.float32 else 0, _dev(a, "a"), _dev(w, "w"), m, n, k,
                                      _rows(a, "a"), _rows(out, "out"), _stream())


NORM_CHAIN_MAX_ROWS = 16


def gemm_chains_norm(dtype: torch.dtype, m: int, k: int, choice: KernelChoice = DEFAULT_CHOICE) -> bool:
    """Whether gemm_norm_chain() takes a product of m rows over k with weights of `dtype`."""
    return dtype == torch.bfloat16 and m <= min(NORM_CHAIN_MAX_ROWS, choice.few_rows_max) and k % 8 == 0


def norm_chain_parts(n: int) -> int:
    """Partial sums of squares per row that a product of n output columns leaves for the next norm."""
    return library().lrs_gemm_norm_chain_parts(n)


def gemm_norm_chain(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None = None,
                    accumulate: bool = False, swiglu: bool = False,
                    in_sumsq: torch.Tensor | None = None, in_eps: float = 0.0,
                    next_x: torch.Tensor | None = None, next_sumsq: torch.Tensor | None = None,
                    next_weight: torch.Tensor | None = None, choice: KernelChoice = DEFAULT_CHOICE) -> None:
    """out = a @ w.T (+ bias) for at most 16 bf16 rows, with an RMSNorm taken apart around it.

    in_sumsq [parts, M] float32: `a` holds bf16(h * norm weight); row r of the product is multiplied
    by rsqrt(sum_p in_sumsq[p, r] / K + in_eps), which completes the norm.
    next_x [M, N] bf16, next_sumsq [norm_chain_parts(N), M] float32, next_weight [N] (needs
    `accumulate`): besides adding into `out`, write bf16(out_new * next_weight) and the partial sums
    of out_new^2, the input of the next product called with in_sumsq."""
    n, k = w.shape
    m = a.shape[0]
    lda, ldc = _rows(a, "a"), _rows(out, "out")
    _need(w.dim() == 2 and w.is_contiguous() and a.shape[1] == k, f"gemm_norm_chain: weight must be contiguous [N, {a.shape[1]}], got {tuple(w.shape)}")
    _need(a.dtype == torch.bfloat16 and gemm_chains_norm(w.dtype, m, k, choice), "gemm_norm_chain: needs bf16 input and weights, at most 16 rows, K % 8 == 0")
    _need(out.shape == (m, n // 2 if swiglu else n), f"gemm_norm_chain: out must be [{m}, {n // 2 if swiglu else n}], got {tuple(out.shape)}")
    if accumulate:
        _need(out.dtype == torch.float32, "gemm_norm_chain: accumulation needs a float32 output")
        mode = OUT_ADD_F32
    elif out.dtype == w.dtype:
        mode = OUT_STORE
    else:
        _need(out.dtype == torch.float32, "gemm_norm_chain: output must be bf16 or float32")
        mode = OUT_STORE_F32
    if bias is not None:
        _need(bias.numel() == n and bias.dtype == w.dtype and bias.is_contiguous(), "gemm_norm_chain: bias must hold N values of the weight dtype")
    if swiglu:
        _need(n % 16 == 0 and bias is None and mode == OUT_STORE, "gemm_norm_chain: swiglu needs N % 16 == 0, no bias, a stored output")
    parts = 0
    if in_sumsq is not None:
        _need(in_sumsq.dtype == torch.float32 and in_sumsq.dim() == 2 and in_sumsq.shape[1] == m and in_sumsq.is_contiguous() and in_eps > 0,
              f"gemm_norm_chain: in_sumsq must be contiguous float32 [parts, {m}] and in_eps positive")
        parts = in_sumsq.shape[0]
    if next_x is not None:
        _need(accumulate and not swiglu, "gemm_norm_chain: only a product that adds into the residual stream can feed the next norm")
        _need(next_x.dtype == torch.bfloat16 and next_x.shape == (m, n) and next_x.is_contiguous(), f"gemm_norm_chain: next_x must be contiguous bf16 [{m}, {n}]")
        _need(next_sumsq is not None and next_sumsq.dtype == torch.float32 and next_sumsq.shape == (norm_chain_parts(n), m) and next_sumsq.is_contiguous(),
              f"gemm_norm_chain: next_sumsq must be contiguous float32 [{norm_chain_parts(n)}, {m}]")
        _need(next_weight is not None and next_weight.numel() == n and next_weight.is_contiguous(), "gemm_norm_chain: next_weight must hold N values")
    _launch("lrs_gemm_norm_chain", 
        _dev(out, "out"), mode, _dev(a, "a"), _dev(w, "w"), None if bias is None else _dev(bias, "bias"), m, n, k, lda, ldc,
        1 if swiglu else 0, None if in_sumsq is None else _dev(in_sumsq, "in_sumsq"), parts, in_eps,
        None if next_x is None else _dev(next_x, "next_x"), None if next_x is None else _dev(next_sumsq, "next_sumsq"),
        None if next_x is None else _dev(next_weight, "next_weight"), dtype_code(next_weight.dtype) if next_x is not None else 0,
        choice.word, _stream())


def scale_rows(out: torch.Tensor, x: torch.Tensor, sumsq: torch.Tensor, eps: float) -> None:
    """out[r] = x[r] * rsqrt(sum_p sumsq[p, r] / hidden + eps): completes a norm that gemm_norm_chain() began."""
    m, hidden = x.shape
    _need(x.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and out.shape == x.shape and x.is_contiguous() and out.is_contiguous(),
          "scale_rows: x and out must be contiguous bf16 of one shape")
    _need(sumsq.dtype == torch.float32 and sumsq.dim() == 2 and sumsq.shape[1] == m and sumsq.is_contiguous(), f"scale_rows: sumsq must be float32 [parts, {m}]")
    _launch("lrs_scale_rows", _dev(out, "out"), _dev(x, "x"), _dev(sumsq, "sumsq"), sumsq.shape[0], m, hidden, eps, _stream())


# -------------------------------------------------------------- attention
def _gates(gates: torch.Tensor | None, tokens: int, nq: int, dtype: torch.dtype, who: str) -> tuple:
    """(address, row stride) of a gate a head, [T, nq] in the activation dtype, rows of any stride; (None, 0): no gate."""
    if gates is None:
        return None, 0
    _need(gates.dim() == 2 and gates.shape == (tokens, nq) and gates.dtype == dtype and gates.stride(1) == 1, f"{who}: gates must be [{tokens}, {nq}] of the activation dtype")
    return _dev(gates, "gates"), gates.stride(0)


def _sinks(sinks: torch.Tensor | None, nq: int, who: str):
    if sinks is None:
        return None
    _need(sinks.dtype == torch.float32 and sinks.numel() == nq and sinks.is_contiguous(), f"{who}: sinks must be float32 [{nq}]")
    return _dev(sinks, "sinks")


def attention(out: torch.Tensor, q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
              token_request: torch.Tensor, positions: torch.Tensor, nq: int, scale: float, window: int = 0, keep_first: int = 0,
              sinks: torch.Tensor | None = None, softcap: float = 0.0, gates: torch.Tensor | None = None) -> None:
    """out [T, nq*dv]; q [T, >= nq*d] (leading nq*d columns of each row); key pages [P, nkv, page, d],
    value pages [P, nkv, dv, page].  window: a token at p sees keys above p - window; keep_first: and those below keep_first.
    sinks (float32 [nq]): the softmax's denominator of head h has one more term exp(sinks[h]), without key or value.
    softcap > 0: the scaled scores pass softcap * tanh(score / softcap) before the softmax.
    gates ([T, nq], rows of any stride): head h's output is multiplied by sigmoid(gates[t, h])."""
    tokens = out.shape[0]
    _need(k_pages.dim() == 4 and v_pages.dim() == 4 and k_pages.is_contiguous() and v_pages.is_contiguous(), "attention: pages must be contiguous")
    _, nkv, page_size, d = k_pages.shape
    dv = v_pages.shape[2]
    _need(v_pages.shape == (k_pages.shape[0], nkv, dv, page_size), "attention: key pages must be [P, nkv, page, d] and value pages [P, nkv, dv, page]")
    _need(out.shape[1] == nq * dv and q.shape[0] == tokens and q.shape[1] >= nq * d, "attention: q/out widths do not match nq*d and nq*dv")
    _need(q.dtype == k_pages.dtype == v_pages.dtype == out.dtype, "attention: q, pages and out must share a dtype")
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.stride(1) == 1, "attention: block_table must be int32 [R, blocks]")
    for name, t in (("token_request", token_request), ("positions", positions)):
        _need(t.dtype == torch.int32 and t.numel() >= tokens and t.is_contiguous(), f"attention: {name} must be int32 [T]")
    _launch("lrs_attention", 
        _dev(out, "out"), _rows(out, "out"), _dev(q, "q"), _rows(q, "q"), _dev(k_pages, "k_pages"), _dev(v_pages, "v_pages"),
        _dev(block_table, "block_table"), block_table.stride(0), _dev(token_request, "token_request"), _dev(positions, "positions"),
        dtype_code(q.dtype), tokens, nq, nkv, d, dv, page_size, scale, window, keep_first, _sinks(sinks, nq, "attention"), float(softcap),
        *_gates(gates, tokens, nq, q.dtype, "attention"), _stream())


def qkv_norm_prep(qkv: torch.Tensor, nq: int, nkv: int, d: int, dv: int, q_weight, k_weight, eps: float, cos, sin,
                  k_pages: torch.Tensor, v_pages: torch.Tensor, slots: torch.Tensor, page_size: int) -> None:
    """The rows of `qkv` [T, >= nq*d + nkv*d + nkv*dv] (q | k | v | whatever follows): q and k each divided by the root mean
    square of the whole part (all heads at once) and multiplied by a weight per column (float32 [nq*d], [nkv*d]; None: no
    norm), the first 2 * cos.shape[1] dims of every head rotated; q in place, k and v into the pages."""
    tokens = qkv.shape[0]
    stride = _rows(qkv, "qkv")
    _need(qkv.shape[1] >= (nq + nkv) * d + nkv * dv, "qkv_norm_prep: the rows hold fewer than q, k and v")
    rot_half = 0
    if cos is not None:
        rot_half = cos.shape[1]
        _need(cos.shape[0] >= tokens and sin.shape == cos.shape and cos.is_contiguous() and sin.is_contiguous()
              and cos.dtype == torch.float32 and sin.dtype == torch.float32, "qkv_norm_prep: rotary tables must be float32 [T, half]")
    if q_weight is not None:
        _need(k_weight is not None and q_weight.numel() == nq * d and k_weight.numel() == nkv * d and q_weight.dtype == k_weight.dtype == torch.float32
              and q_weight.is_contiguous() and k_weight.is_contiguous(), "qkv_norm_prep: norm weights must be float32 [nq*d] and [nkv*d]")
    _need(k_pages.dim() == 4 and k_pages.shape[1:] == (nkv, page_size, d) and v_pages.shape == (k_pages.shape[0], nkv, dv, page_size),
          f"qkv_norm_prep: key pages must be [pages, {nkv}, {page_size}, {d}] and value pages [pages, {nkv}, {dv}, {page_size}]")
    _need(k_pages.is_contiguous() and v_pages.is_contiguous() and k_pages.dtype == qkv.dtype and v_pages.dtype == qkv.dtype,
          "qkv_norm_prep: pages must be contiguous and of the activation dtype")
    _need(slots.dtype == torch.int32 and slots.numel() >= tokens and slots.is_contiguous(), "qkv_norm_prep: slots must be int32 [T]")
    _launch("lrs_qkv_norm_prep", _dev(qkv, "qkv"), dtype_code(qkv.dtype), tokens, stride, nq, nkv, d, dv,
            None if q_weight is None else _dev(q_weight, "q_weight"), None if k_weight is None else _dev(k_weight, "k_weight"), eps,
            None if cos is None else cos.data_ptr(), None if sin is None else sin.data_ptr(), rot_half, _dev(k_pages, "k_pages"),
            _dev(v_pages, "v_pages"), _dev(slots, "slots"), page_size, _stream())


def sigmoid_gate(out: torch.Tensor, gate: torch.Tensor) -> None:
    """out *= sigmoid(gate); out [T, C] and gate [T, C], or gate [T, C / group]: one value for every `group` neighbouring columns
    (a gate per head).  Rows may be strided (a gate that lies in a wider projection row)."""
    _need(out.dim() == 2 and gate.dim() == 2 and out.dtype == gate.dtype and gate.shape[0] == out.shape[0] and gate.shape[1] > 0
          and out.shape[1] % gate.shape[1] == 0, "sigmoid_gate: out [T, C] and gate [T, C / group] must be of one dtype")
    _launch("lrs_sigmoid_gate", _dev(out, "out"), _rows(out, "out"), _dev(gate, "gate"), _rows(gate, "gate"), dtype_code(out.dtype),
            out.shape[0], out.shape[1], out.shape[1] // gate.shape[1], _stream())


def rotate_unit_prep(qkv: torch.Tensor, nq: int, nkv: int, d: int, dv: int, eps: float, unit: bool, cos, sin, neighbours: bool,
                     k_pages: torch.Tensor, v_pages: torch.Tensor, slots: torch.Tensor, page_size: int, bias: torch.Tensor | None = None) -> None:
    """The rows of `qkv` [T, >= nq*d + nkv*d + nkv*dv] (q | k | v | whatever follows): the first 2 * cos.shape[1] dims of every q
    and k head rotated (pairs (j, j + half), or with `neighbours` (2j, 2j + 1)), then, with `unit`, every head divided by
    sqrt(mean of its squares + eps); q in place, k and v into the pages.  bias (float32, at least nq*d + nkv*d + nkv*dv values): added
    to q, k and v as they are read (the product that made the rows then left it out)."""
    tokens = qkv.shape[0]
    stride = _rows(qkv, "qkv")
    _need(qkv.shape[1] >= (nq + nkv) * d + nkv * dv, "rotate_unit_prep: the rows hold fewer than q, k and v")
    rot_half = 0
    if cos is not None:
        rot_half = cos.shape[1]
        _need(cos.shape[0] >= tokens and sin.shape == cos.shape and cos.is_contiguous() and sin.is_contiguous()
              and cos.dtype == torch.float32 and sin.dtype == torch.float32, "rotate_unit_prep: rotary tables must be float32 [T, half]")
    _need(k_pages.dim() == 4 and k_pages.shape[1:] == (nkv, page_size, d) and v_pages.shape == (k_pages.shape[0], nkv, dv, page_size),
          f"rotate_unit_prep: key pages must be [pages, {nkv}, {page_size}, {d}] and value pages [pages, {nkv}, {dv}, {page_size}]")
    _need(k_pages.is_contiguous() and v_pages.is_contiguous() and k_pages.dtype == qkv.dtype and v_pages.dtype == qkv.dtype,
          "rotate_unit_prep: pages must be contiguous and of the activation dtype")
    _need(slots.dtype == torch.int32 and slots.numel() >= tokens and slots.is_contiguous(), "rotate_unit_prep: slots must be int32 [T]")
    _need(bias is None or (bias.dtype == torch.float32 and bias.is_contiguous() and bias.numel() >= (nq + nkv) * d + nkv * dv),
          "rotate_unit_prep: the bias must be float32 and hold a value for every column of q, k and v")
    _launch("lrs_rotate_unit_prep", _dev(qkv, "qkv"), dtype_code(qkv.dtype), tokens, stride, nq, nkv, d, dv, float(eps), int(unit),
            None if cos is None else cos.data_ptr(), None if sin is None else sin.data_ptr(), rot_half, int(neighbours), _dev(k_pages, "k_pages"),
            _dev(v_pages, "v_pages"), _dev(slots, "slots"), page_size, None if bias is None else _dev(bias, "bias"), _stream())


def gated_clamped(out: torch.Tensor, gate_up: torch.Tensor, alpha: float, limit: float) -> None:
    """out [T, I] = g * sigmoid(alpha * g) * (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit), from gate_up [T, 2I]
    (gate columns, then up columns)."""
    tokens, inter = out.shape
    _need(gate_up.shape == (tokens, 2 * inter) and gate_up.dtype == out.dtype and gate_up.is_contiguous() and out.is_contiguous(),
          "gated_clamped: out must be [T, I] and gate_up [T, 2I], contiguous and of one dtype")
    _need(limit > 0, "gated_clamped: the limit must be positive")
    _launch("lrs_gated_clamped", _dev(out, "out"), _dev(gate_up, "gate_up"), dtype_code(out.dtype), tokens, inter, float(alpha), float(limit), _stream())


def add_gathered(out: torch.Tensor, table: torch.Tensor, ids: torch.Tensor) -> None:
    """out [T, C] float32 += table[ids[t]] (table [rows, C]; ids int32 [T] within the table)."""
    tokens, cols = out.shape
    _need(out.dtype == torch.float32 and out.is_contiguous() and table.dim() == 2 and table.shape[1] == cols and table.is_contiguous(),
          "add_gathered: out must be contiguous float32 [T, C] and table contiguous [rows, C]")
    _need(ids.dtype == torch.int32 and ids.numel() >= tokens and ids.is_contiguous(), "add_gathered: ids must be int32 [T]")
    _launch("lrs_add_gathered", _dev(out, "out"), _dev(table, "table"), dtype_code(table.dtype), _dev(ids, "ids"), tokens, cols, _stream())


def scale_values(x: torch.Tensor, factor: float) -> None:
    """x *= factor over contiguous float32 values."""
    _need(x.dtype == torch.float32 and x.is_contiguous() and x.numel() > 0, "scale_values: x must be contiguous float32")
    _launch("lrs_scale_values", _dev(x, "x"), x.numel(), float(factor), _stream())


def axpby(out: torch.Tensor, a: torch.Tensor, alpha: float, b: torch.Tensor, beta: float, norm_weight: torch.Tensor | None = None,
          eps: float = 0.0, normed: torch.Tensor | None = None) -> None:
    """out = alpha * a + beta * b over contiguous float32 [T, C] (out may be a or b).  norm_weight (float32 [C]): `normed`
    [T, C] also receives the RMS norm of the new rows times the weight."""
    for name, t in (("out", out), ("a", a), ("b", b)):
        _need(t.dtype == torch.float32 and t.is_contiguous() and t.shape == out.shape and t.dim() == 2, f"axpby: {name} must be contiguous float32 [T, C]")
    if norm_weight is not None:
        _need(norm_weight.dtype == torch.float32 and norm_weight.numel() == out.shape[1] and norm_weight.is_contiguous(), "axpby: the norm's weight must be float32 [C]")
        _need(normed is not None and normed.shape == out.shape and normed.is_contiguous(), "axpby: the normalised rows need a contiguous [T, C] buffer")
    _launch("lrs_axpby", _dev(out, "out"), _dev(a, "a"), alpha, _dev(b, "b"), beta, out.shape[0], out.shape[1],
            None if norm_weight is None else _dev(norm_weight, "norm_weight"), eps, None if norm_weight is None else _dev(normed, "normed"),
            0 if norm_weight is None else dtype_code(normed.dtype), _stream())


ACTIVATIONS = {"gelu": 0, "gelu_tanh": 1, "silu": 2, "relu": 3}


def activation(out: torch.Tensor, x: torch.Tensor, kind: str) -> None:
    """out = act(x) elementwise (out may be x): "gelu" (0.5 x (1 + erf(x / sqrt 2))), "gelu_tanh", "silu", "relu"."""
    _need(kind in ACTIVATIONS, f"activation: unknown kind {kind!r}; known: {', '.join(ACTIVATIONS)}")
    _need(out.shape == x.shape and out.dtype == x.dtype and out.is_contiguous() and x.is_contiguous() and x.numel() > 0,
          "activation: out and x must be contiguous, of one shape and dtype")
    _launch("lrs_activation", _dev(out, "out"), _dev(x, "x"), dtype_code(x.dtype), x.numel(), ACTIVATIONS[kind], _stream())


DECODE_HEAD_DIMS = (32, 64, 96, 128, 192)


def attention_decode_supported(dtype: torch.dtype, nq: int, nkv: int, d: int, page_size: int) -> bool:
    """Whether the matrix-core decode kernel takes this shape (else use attention())."""
    return dtype == torch.bfloat16 and d in DECODE_HEAD_DIMS and page_size % 16 == 0 and nq // nkv <= 16


@dataclass
class DecodePrepare:
    """What attention_decode() does to the raw q/k/v rows when it stands in for qk_prep(): per-head
    RMSNorm of q and k (weights None: none), rotation of the whole head by cos/sin [T, d/2] (None:
    none), and the write of the new key and value into the pages (kv_heads = the number of kv heads
    held in the rows; 0 for a layer that reads another layer's pages)."""
    q_weight: torch.Tensor | None
    k_weight: torch.Tensor | None
    eps: float
    cos: torch.Tensor | None
    sin: torch.Tensor | None
    kv_heads: int


def decode_prepare_supported(d: int, rotates: bool) -> bool:
    """Whether attention_decode() can do qk_prep()'s work for heads of d dims (it rotates pairs that
    lie 32-dim chunks apart: d a multiple of 64)."""
    return not rotates or d % 64 == 0


def attention_decode(out: torch.Tensor, q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                     token_request: torch.Tensor, positions: torch.Tensor, nq: int, scale: float, window: int = 0, splits: int = 1,
                     part_o: torch.Tensor | None = None, part_ml: torch.Tensor | None = None, max_context: int | None = None,
                     prepare: "DecodePrepare | None" = None, form: int = 0, keep_first: int = 0, sinks: torch.Tensor | None = None,
                     softcap: float = 0.0, gates: torch.Tensor | None = None) -> None:
    """attention() for a step with one query token per request, bfloat16 only; the keys of a token
    are divided between `splits` workgroups whose partial results meet in part_o / part_ml.
    keep_first (with a window and prepared heads): the first positions of a sequence stay visible behind the window; their
    share is one more partial result, so the buffers hold splits + 1 and are needed whatever `splits` is.

    prepare: `q` holds the raw rows of the q/k/v product and the kernel also does what qk_prep()
    does (see DecodePrepare); without it q, and the pages, must have been through qk_prep()."""
    tokens = out.shape[0]
    _need(k_pages.dim() == 4 and k_pages.is_contiguous() and v_pages.is_contiguous(), "attention_decode: pages must be contiguous")
    _, nkv, page_size, d = k_pages.shape
    _need(v_pages.shape == (k_pages.shape[0], nkv, d, page_size), "attention_decode: key pages must be [P, nkv, page, d] and value pages [P, nkv, d, page]")
    _need(attention_decode_supported(q.dtype, nq, nkv, d, page_size), f"attention_decode: unsupported shape nq={nq} nkv={nkv} d={d} page={page_size} {q.dtype}")
    _need(out.shape[1] == nq * d and q.shape[0] == tokens and q.shape[1] >= nq * d, "attention_decode: q/out widths do not match nq*d")
    _need(q.dtype == k_pages.dtype == v_pages.dtype == out.dtype, "attention_decode: q, pages and out must share a dtype")
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.stride(1) == 1, "attention_decode: block_table must be int32 [R, blocks]")
    for name, t in (("token_request", token_request), ("positions", positions)):
        _need(t.dtype == torch.int32 and t.numel() >= tokens and t.is_contiguous(), f"attention_decode: {name} must be int32 [T]")
    _need(keep_first >= 0 and (keep_first == 0 or (window > 0 and prepare is None)), "attention_decode: kept first positions need a window and prepared heads")
    slots = splits + (1 if keep_first else 0)
    if slots > 1:
        _need(part_o is not None and part_o.dtype == torch.float32 and part_o.is_contiguous() and part_o.numel() >= tokens * nq * slots * d, "attention_decode: part_o too small")
        _need(part_ml is not None and part_ml.dtype == torch.float32 and part_ml.is_contiguous() and part_ml.numel() >= tokens * nq * slots * 2, "attention_decode: part_ml too small")
    fused = [0, None, None, 0, 0.0, None, None, 0]
    if prepare is not None:
        _need(decode_prepare_supported(d, prepare.cos is not None), f"attention_decode: cannot rotate heads of {d} dims itself")
        _need((prepare.q_weight is None) == (prepare.k_weight is None), "attention_decode: q and k norm weights must come together")
        _need(prepare.kv_heads in (0, nkv) and q.shape[1] >= (nq + 2 * prepare.kv_heads) * d, "attention_decode: q rows must hold the q heads and kv_heads (0 or all) k and v heads")
        for name, w in (("q_weight", prepare.q_weight), ("k_weight", prepare.k_weight)):
            _need(w is None or (w.numel() == d and w.is_contiguous() and w.dtype == prepare.q_weight.dtype), f"attention_decode: {name} must hold head_dim values")
        for name, t in (("cos", prepare.cos), ("sin", prepare.sin)):
            _need((t is None) == (prepare.cos is None) and (t is None or (t.dtype == torch.float32 and t.shape == (tokens, d // 2) and t.is_contiguous())),
                  f"attention_decode: {name} must be float32 [{tokens}, {d // 2}]")
        normed = prepare.q_weight is not None
        _need(not normed or prepare.eps > 0, "attention_decode: eps must be positive")
        fused = [1, _dev(prepare.q_weight, "q_weight") if normed else None, _dev(prepare.k_weight, "k_weight") if normed else None,
                 dtype_code(prepare.q_weight.dtype) if normed else 0, prepare.eps,
                 None if prepare.cos is None else _dev(prepare.cos, "cos"), None if prepare.sin is None else _dev(prepare.sin, "sin"), prepare.kv_heads]
    _launch("lrs_attention_decode", 
        _dev(out, "out"), _rows(out, "out"), None if slots == 1 else _dev(part_o, "part_o"), None if slots == 1 else _dev(part_ml, "part_ml"),
        _dev(q, "q"), _rows(q, "q"), _dev(k_pages, "k_pages"), _dev(v_pages, "v_pages"), _dev(block_table, "block_table"), block_table.stride(0),
        _dev(token_request, "token_request"), _dev(positions, "positions"), tokens,
        block_table.shape[1] * page_size if max_context is None else max_context, nq, nkv, d, page_size, scale, window, keep_first, splits,
        form, *fused, _sinks(sinks, nq, "attention_decode"), float(softcap), *_gates(gates, tokens, nq, q.dtype, "attention_decode"), _stream())


def attention_prefill(out: torch.Tensor, q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                      token_request: torch.Tensor, positions: torch.Tensor, qblock_token0: torch.Tensor, qblock_count: torch.Tensor,
                      nq: int, scale: float, window: int = 0, max_count: int | None = None, max_context: int | None = None,
                      splits: int = 1, part_o: torch.Tensor | None = None, part_ml: torch.Tensor | None = None,
                      prepare: "DecodePrepare | None" = None, keep_first: int = 0, sinks: torch.Tensor | None = None,
                      softcap: float = 0.0, gates: torch.Tensor | None = None) -> None:
    """attention() on matrix cores for any bfloat16 step.  qblock_token0 / qblock_count list groups of at
    most attention_prefill_group() consecutive tokens of one request that together cover every token of
    the step once; `max_count` is the largest count among them (the group limit if not given) and
    `max_context` the longest context (position + 1) of any token (what the block table can hold if not given).
    splits > 1 divides every group's keys between that many workgroups (few queries over long contexts);
    their partial results meet in part_o [T, nq * splits * d] and part_ml [T, nq * splits * 2] float32.
    prepare (where attention_prefill_prepares(d)): `q` holds the raw q heads of the q/k/v product, and the kernel gives
    them their norm and rotation itself (q_weight, eps, cos, sin of DecodePrepare; kv_heads 0: the keys and values are in
    the pages already, from qk_prep(skip_q=True)).
    keep_first (with a window and prepared heads): the first positions of a sequence stay visible behind the window; their
    share is one more partial result, so the buffers hold splits + 1 and are needed whatever `splits` is."""
    tokens = out.shape[0]
    _need(k_pages.dim() == 4 and k_pages.is_contiguous() and v_pages.is_contiguous(), "attention_prefill: pages must be contiguous")
    _, nkv, page_size, d = k_pages.shape
    _need(v_pages.shape == (k_pages.shape[0], nkv, d, page_size), "attention_prefill: key pages must be [P, nkv, page, d] and value pages [P, nkv, d, page]")
    _need(attention_decode_supported(q.dtype, nq, nkv, d, page_size), f"attention_prefill: unsupported shape nq={nq} nkv={nkv} d={d} page={page_size} {q.dtype}")
    _need(out.shape[1] == nq * d and q.shape[0] == tokens and q.shape[1] >= nq * d, "attention_prefill: q/out widths do not match nq*d")
    _need(q.dtype == k_pages.dtype == v_pages.dtype == out.dtype, "attention_prefill: q, pages and out must share a dtype")
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.stride(1) == 1, "attention_prefill: block_table must be int32 [R, blocks]")
    for name, t in (("token_request", token_request), ("positions", positions)):
        _need(t.dtype == torch.int32 and t.numel() >= tokens and t.is_contiguous(), f"attention_prefill: {name} must be int32 [T]")
    n_blocks = qblock_token0.numel()
    _need(n_blocks > 0 and qblock_count.numel() == n_blocks and qblock_token0.dtype == qblock_count.dtype == torch.int32
          and qblock_token0.is_contiguous() and qblock_count.is_contiguous(), "attention_prefill: query blocks must be two int32 vectors of one length")
    _need(1 <= splits <= 64, f"attention_prefill: splits must be 1..64, got {splits}")
    _need(keep_first >= 0 and (keep_first == 0 or (window > 0 and prepare is None)), "attention_prefill: kept first positions need a window and prepared heads")
    slots = splits + (1 if keep_first else 0)
    if slots > 1:
        _need(part_o is not None and part_o.dtype == torch.float32 and part_o.is_contiguous() and part_o.numel() >= tokens * nq * slots * d, "attention_prefill: part_o too small")
        _need(part_ml is not None and part_ml.dtype == torch.float32 and part_ml.is_contiguous() and part_ml.numel() >= tokens * nq * slots * 2, "attention_prefill: part_ml too small")
    fused = [0, None, 0, 0.0, None, None]
    if prepare is not None:
        _need(attention_prefill_prepares(d), f"attention_prefill: heads of {d} dims must come prepared")
        _need(prepare.kv_heads == 0, "attention_prefill: prepares the queries only (kv_heads must be 0)")
        w = prepare.q_weight
        _need(w is None or (w.numel() == d and w.is_contiguous() and prepare.eps > 0), "attention_prefill: q_weight must hold head_dim values, eps be positive")
        for name, t in (("cos", prepare.cos), ("sin", prepare.sin)):
            _need((t is None) == (prepare.cos is None) and (t is None or (t.dtype == torch.float32 and t.dim() == 2 and t.shape[0] >= tokens
                                                                       and t.shape[1] == d // 2 and t.is_contiguous())),
                  f"attention_prefill: {name} must be float32 [{tokens}, {d // 2}]")
        fused = [1, None if w is None else _dev(w, "q_weight"), 0 if w is None else dtype_code(w.dtype), prepare.eps,
                 None if prepare.cos is None else _dev(prepare.cos, "cos"), None if prepare.sin is None else _dev(prepare.sin, "sin")]
    _launch("lrs_attention_prefill", 
        _dev(out, "out"), _rows(out, "out"), _dev(q, "q"), _rows(q, "q"), _dev(k_pages, "k_pages"), _dev(v_pages, "v_pages"),
        _dev(block_table, "block_table"), block_table.stride(0), _dev(token_request, "token_request"), _dev(positions, "positions"),
        _dev(qblock_token0, "qblock_token0"), _dev(qblock_count, "qblock_count"), n_blocks,
        attention_prefill_group() if max_count is None else max_count,
        block_table.shape[1] * page_size if max_context is None else max_context, nq, nkv, d, page_size, scale, window, keep_first,
        tokens, splits, None if slots == 1 else _dev(part_o, "part_o"), None if slots == 1 else _dev(part_ml, "part_ml"), *fused,
        _sinks(sinks, nq, "attention_prefill"), float(softcap), *_gates(gates, tokens, nq, q.dtype, "attention_prefill"), _stream())


def attention_prefill_prepares(d: int) -> bool:
    """Whether attention_prefill() can take raw q heads of d dims and prepare them itself."""
    return bool(library().lrs_attention_prefill_prepares(d))


def compute_units() -> int:
    """Compute units of the device (workgroups of one kernel that can start at the same time, per occupancy)."""
    return library().lrs_compute_units()


def attention_prefill_group(tokens: int | None = None, longest: int = 0) -> int:
    """Most tokens in one query group of attention_prefill(); with `tokens`, the group size that
    serves a step of that many tokens best (smaller groups fill the chip when there are few), given the
    longest context (position + 1) among them, if known (larger groups pay earlier behind a long context)."""
    if tokens is None:
        return library().lrs_attention_prefill_group()
    return library().lrs_attention_prefill_group_for(tokens, longest)


# --------------------------------------------------------------- sampling
_choose_scratch: dict = {}


def choose_tokens(out: torch.Tensor, logits: torch.Tensor, temperature=None, seeds=None, counters=None,
                  out_address: int | None = None, filtered: bool = False) -> None:
    """One token per row of logits into `out`, int32 [R] on the device; or, with `out_address` (from
    pinned_device_address(out)), into pinned host memory that the kernel writes directly and the
    host reads after synchronising the stream.  A row that holds a value that is not finite gets -1
    (the reference refuses such logits, mini_llm/sampling.py:104-113); `filtered`: filter_logits() has
    been over the rows, so those of positive temperature may hold -inf."""
    rows, vocab = logits.shape
    _need(out.dtype == torch.int32 and out.numel() >= rows and out.is_contiguous(), "choose_tokens: out must be int32 [R]")
    stride = _rows(logits, "logits")
    if out_address is None:
        out_pointer = _dev(out, "out")
    else:
        _need(not out.is_cuda, "choose_tokens: out_address goes with a pinned host tensor")
        out_pointer = out_address + out.storage_offset() * out.element_size()
    if temperature is not None:
        _need(temperature.dtype == torch.float32 and temperature.numel() >= rows, "choose_tokens: temperature must be float32 [R]")
        _need(seeds is not None and seeds.dtype == torch.int64 and seeds.numel() >= rows, "choose_tokens: seeds must be int64 [R]")
        _need(counters is not None and counters.dtype == torch.int32 and counters.numel() >= rows, "choose_tokens: counters must be int32 [R]")
    args = (None if temperature is None else _dev(temperature, "temperature"), None if temperature is None else _dev(seeds, "seeds"),
            None if temperature is None else _dev(counters, "counters"))
    if vocab >= 16384:   # large vocabulary: many workgroups per row, then one to pick among their results
        parts = -(-vocab // 4096)
        key = (logits.device, rows, parts)
        scratch = _choose_scratch.get(key)
        if scratch is None:
            scratch = _choose_scratch[key] = (torch.empty(rows * parts, dtype=torch.float32, device=logits.device),
                                              torch.empty(rows * parts, dtype=torch.int32, device=logits.device))
        _launch("lrs_choose_tokens_split", out_pointer, _dev(logits, "logits", torch.float32), stride, rows, vocab, *args,
                                                 _dev(scratch[0], "part_value"), _dev(scratch[1], "part_index"), parts, int(bool(filtered)), _stream())
        return
    _launch("lrs_choose_tokens", out_pointer, _dev(logits, "logits", torch.float32), stride, rows, vocab, *args, int(bool(filtered)), _stream())


def choose_tokens_static(out: torch.Tensor, logits: torch.Tensor, parts: int, temperature=None, seeds=None, counters=None,
                         filtered: bool = False) -> None:
    """choose_tokens() in its two-pass form (`parts` slices a row) for callers that must not allocate: the
    slices' results go to a fixed array inside the library (rows * parts at most
    lrs_choose_tokens_static_max_parts()), so nothing is allocated here or there.  Calls that overlap on
    one GPU share that array and race."""
    rows, vocab = logits.shape
    _need(out.dtype == torch.int32 and out.numel() >= rows and out.is_contiguous(), "choose_tokens_static: out must be int32 [R]")
    if temperature is not None:
        _need(temperature.dtype == torch.float32 and temperature.numel() >= rows, "choose_tokens_static: temperature must be float32 [R]")
        _need(seeds is not None and seeds.dtype == torch.int64 and seeds.numel() >= rows, "choose_tokens_static: seeds must be int64 [R]")
        _need(counters is not None and counters.dtype == torch.int32 and counters.numel() >= rows, "choose_tokens_static: counters must be int32 [R]")
    _launch("lrs_choose_tokens_static", 
        _dev(out, "out"), _dev(logits, "logits", torch.float32), _rows(logits, "logits"), rows, vocab,
        None if temperature is None else _dev(temperature, "temperature"), None if temperature is None else _dev(seeds, "seeds"),
        None if temperature is None else _dev(counters, "counters"), parts, int(bool(filtered)), _stream())


def filter_logits(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor | None, top_p: torch.Tensor | None) -> None:
    rows, vocab = logits.shape
    stride = _rows(logits, "logits")
    _need(temperature.dtype == torch.float32 and temperature.numel() >= rows, "filter_logits: temperature must be float32 [R]")
    if top_k is not None:
        _need(top_k.dtype == torch.int32 and top_k.numel() >= rows, "filter_logits: top_k must be int32 [R]")
    if top_p is not None:
        _need(top_p.dtype == torch.float32 and top_p.numel() >= rows, "filter_logits: top_p must be float32 [R]")
    _launch("lrs_filter_logits", _dev(logits, "logits", torch.float32), stride, rows, vocab, _dev(temperature, "temperature"),
                                       None if top_k is None else _dev(top_k, "top_k"), None if top_p is None else _dev(top_p, "top_p"), _stream())


# ------------------------------------------------------------------- gated delta rule
def delta_state_floats(heads: int, kv_heads: int, dim: int, vdim: int, taps: int) -> int:
    """Floats of one request's state row of a gated-delta-rule mixer: the matrix of every head in the order the scan
    holds it (dim padded to 16 lanes of 4, 8 or 16 rows), then the convolution's last taps - 1 inputs of every channel."""
    rows = library().lrs_delta_state_rows(dim)
    return heads * rows * 16 * vdim + (taps - 1) * (2 * kv_heads * dim + heads * vdim)


def delta_rule(out: torch.Tensor, proj: torch.Tensor, state: torch.Tensor, token_request: torch.Tensor, cu_seqlens: torch.Tensor,
               slot_ids: torch.Tensor, requests: int, conv_weight: torch.Tensor, kv_heads: int, heads: int, dim: int, vdim: int,
               a_log: torch.Tensor, dt_bias: torch.Tensor, norm_weight: torch.Tensor, eps: float, qkv: torch.Tensor, gates: torch.Tensor,
               raw: torch.Tensor) -> None:
    """One step of the gated delta rule for a ragged batch.  proj [T, >= C] holds each token's projections, columns
    q (kv_heads*dim) | k (kv_heads*dim) | v (heads*vdim) | output gate (heads*vdim) | step size (heads) | decay input
    (heads); state [slots, floats] float32 is read and written at the rows slot_ids names; out [T, heads*vdim]."""
    tokens = out.shape[0]
    channels = 2 * kv_heads * dim + heads * vdim
    taps = conv_weight.shape[1]
    _need(out.is_contiguous() and out.shape[1] == heads * vdim, "delta_rule: out must be contiguous [T, heads*vdim]")
    _need(proj.shape[0] >= tokens and proj.shape[1] >= channels + heads * vdim + 2 * heads, "delta_rule: proj holds too few columns")
    _need(state.dim() == 2 and state.dtype == torch.float32 and state.is_contiguous()
          and state.shape[1] >= delta_state_floats(heads, kv_heads, dim, vdim, taps), "delta_rule: state rows are too short")
    _need(conv_weight.shape == (channels, taps) and conv_weight.dtype == torch.float32 and conv_weight.is_contiguous(),
          f"delta_rule: the convolution's weights must be float32 [{channels}, taps]")
    for name, t, count in (("a_log", a_log, heads), ("dt_bias", dt_bias, heads), ("norm_weight", norm_weight, vdim)):
        _need(t.dtype == torch.float32 and t.numel() == count and t.is_contiguous(), f"delta_rule: {name} must hold {count} float32 values")
    for name, t, count in (("token_request", token_request, tokens), ("cu_seqlens", cu_seqlens, requests + 1), ("slot_ids", slot_ids, requests)):
        _need(t.dtype == torch.int32 and t.numel() >= count and t.is_contiguous(), f"delta_rule: {name} must be int32 [{count}]")
    _need(qkv.dtype == torch.float32 and qkv.is_contiguous() and qkv.numel() >= tokens * channels, "delta_rule: qkv scratch too small")
    _need(gates.dtype == torch.float32 and gates.is_contiguous() and gates.numel() >= tokens * 2 * heads, "delta_rule: gates scratch too small")
    _need(raw.dtype == torch.float32 and raw.is_contiguous() and raw.numel() >= tokens * heads * vdim, "delta_rule: read-out scratch too small")
    _launch("lrs_delta_rule", _dev(out, "out"), dtype_code(out.dtype), _dev(proj, "proj"), dtype_code(proj.dtype), _rows(proj, "proj"), tokens,
            requests, _dev(token_request, "token_request"), _dev(cu_seqlens, "cu_seqlens"), _dev(slot_ids, "slot_ids"), _dev(state, "state"),
            state.stride(0), _dev(conv_weight, "conv_weight"), taps, kv_heads, heads, dim, vdim, _dev(a_log, "a_log"), _dev(dt_bias, "dt_bias"),
            _dev(norm_weight, "norm_weight"), eps, _dev(qkv, "qkv"), _dev(gates, "gates"), _dev(raw, "raw"), _stream())


def delta_rule_channels(out: torch.Tensor, proj: torch.Tensor, state: torch.Tensor, token_request: torch.Tensor, cu_seqlens: torch.Tensor,
                        slot_ids: torch.Tensor, requests: int, conv_weight: torch.Tensor, kv_heads: int, heads: int, dim: int, vdim: int,
                        a_log: torch.Tensor, dt_bias: torch.Tensor, norm_weight: torch.Tensor, eps: float, qkv: torch.Tensor, gates: torch.Tensor,
                        raw: torch.Tensor, decay_up: torch.Tensor | None, decays: torch.Tensor, gate_up: torch.Tensor | None,
                        gate_in: torch.Tensor | None = None) -> None:
    """The gated delta rule with a decay per head and key channel and a sigmoid output gate, both from inputs of low rank.
    proj [T, >= C] columns: q (kv_heads*dim) | k (kv_heads*dim) | v (heads*vdim) | step size (heads) | decay input (rank_a) |
    gate input (rank_g); decay_up float32 [rank_a, heads*dim], dt_bias [heads*dim], gate_up float32 [rank_g, heads*vdim];
    decays [T, heads*dim] float32 scratch.  With decay_up and gate_up None the second matrices have been applied by the
    caller: `decays` holds the decays' inputs (before bias and softplus) and is turned into the decays in place, `gate_in`
    [T, heads*vdim] float32 holds the gate's.  Everything else as delta_rule()."""
    tokens = out.shape[0]
    channels = 2 * kv_heads * dim + heads * vdim
    taps = conv_weight.shape[1]
    given = decay_up is None
    _need(given == (gate_up is None) and given == (gate_in is not None), "delta_rule_channels: both second matrices, or both of their outputs")
    rank_a, rank_g = (-1, -1) if given else (decay_up.shape[0], gate_up.shape[0])
    _need(out.is_contiguous() and out.shape[1] == heads * vdim, "delta_rule_channels: out must be contiguous [T, heads*vdim]")
    _need(proj.shape[0] >= tokens and proj.shape[1] >= channels + heads + max(rank_a, 0) + max(rank_g, 0), "delta_rule_channels: proj holds too few columns")
    _need(state.dim() == 2 and state.dtype == torch.float32 and state.is_contiguous()
          and state.shape[1] >= delta_state_floats(heads, kv_heads, dim, vdim, taps), "delta_rule_channels: state rows are too short")
    _need(conv_weight.shape == (channels, taps) and conv_weight.dtype == torch.float32 and conv_weight.is_contiguous(),
          f"delta_rule_channels: the convolution's weights must be float32 [{channels}, taps]")
    vectors = [("a_log", a_log, (heads,)), ("dt_bias", dt_bias, (heads * dim,)), ("norm_weight", norm_weight, (vdim,))]
    if given:
        _need(gate_in.dtype == torch.float32 and gate_in.is_contiguous() and gate_in.dim() == 2 and gate_in.shape[0] >= tokens
              and gate_in.shape[1] == heads * vdim, f"delta_rule_channels: gate_in must be contiguous float32 [T, {heads * vdim}]")
        _need(decays.dim() == 2 and decays.shape[1] == heads * dim, f"delta_rule_channels: given decay inputs must be [T, {heads * dim}]")
    else:
        vectors += [("decay_up", decay_up, (rank_a, heads * dim)), ("gate_up", gate_up, (rank_g, heads * vdim))]
    for name, t, shape in vectors:
        _need(t.dtype == torch.float32 and tuple(t.shape) == shape and t.is_contiguous(), f"delta_rule_channels: {name} must be float32 {shape}")
    for name, t, count in (("token_request", token_request, tokens), ("cu_seqlens", cu_seqlens, requests + 1), ("slot_ids", slot_ids, requests)):
        _need(t.dtype == torch.int32 and t.numel() >= count and t.is_contiguous(), f"delta_rule_channels: {name} must be int32 [{count}]")
    for name, t, count in (("qkv", qkv, tokens * channels), ("gates", gates, tokens * 2 * heads), ("raw", raw, tokens * heads * vdim),
                           ("decays", decays, tokens * heads * dim)):
        _need(t.dtype == torch.float32 and t.is_contiguous() and t.numel() >= count, f"delta_rule_channels: {name} scratch too small")
    _launch("lrs_delta_rule_channels", _dev(out, "out"), dtype_code(out.dtype), _dev(proj, "proj"), dtype_code(proj.dtype), _rows(proj, "proj"), tokens,
            requests, _dev(token_request, "token_request"), _dev(cu_seqlens, "cu_seqlens"), _dev(slot_ids, "slot_ids"), _dev(state, "state"),
            state.stride(0), _dev(conv_weight, "conv_weight"), taps, kv_heads, heads, dim, vdim, _dev(a_log, "a_log"), _dev(dt_bias, "dt_bias"),
            _dev(norm_weight, "norm_weight"), eps, _dev(qkv, "qkv"), _dev(gates, "gates"), _dev(raw, "raw"), rank_a,
            None if given else _dev(decay_up, "decay_up"), _dev(decays, "decays"), rank_g, _dev(gate_in if given else gate_up, "gate_up"), _stream())


def state_space(out: torch.Tensor, proj: torch.Tensor, state: torch.Tensor, token_request: torch.Tensor, cu_seqlens: torch.Tensor,
                slot_ids: torch.Tensor, requests: int, conv_weight: torch.Tensor, conv_bias: torch.Tensor | None, groups: int, heads: int,
                state_size: int, vdim: int, a_log: torch.Tensor, dt_bias: torch.Tensor, skip: torch.Tensor, norm_weight: torch.Tensor,
                norm_parts: int, eps: float, qkv: torch.Tensor, gates: torch.Tensor, raw: torch.Tensor, skipped: torch.Tensor) -> None:
    """One step of the selective state space recurrence for a ragged batch: per head S <- exp(-exp(a_log) dt) S + dt B x^T,
    y = S^T C + skip x, then y * silu(z) normalised in `norm_parts` equal parts.  proj [T, >= C] columns: z (heads*vdim) |
    x (heads*vdim) | B (groups*state_size) | C (groups*state_size) | dt (heads); conv_weight float32 [heads*vdim + 2*groups*state_size,
    taps] over x | B | C; state [slots, floats] as the delta rule's with dim = state_size; out [T, heads*vdim]."""
    tokens = out.shape[0]
    inner = heads * vdim
    channels = inner + 2 * groups * state_size
    taps = conv_weight.shape[1]
    _need(out.is_contiguous() and out.shape[1] == inner, "state_space: out must be contiguous [T, heads*vdim]")
    _need(proj.shape[0] >= tokens and proj.shape[1] >= inner + channels + heads, "state_space: proj holds too few columns")
    _need(state.dim() == 2 and state.dtype == torch.float32 and state.is_contiguous()
          and state.shape[1] >= delta_state_floats(heads, groups, state_size, vdim, taps), "state_space: state rows are too short")
    _need(conv_weight.shape == (channels, taps) and conv_weight.dtype == torch.float32 and conv_weight.is_contiguous(),
          f"state_space: the convolution's weights must be float32 [{channels}, taps]")
    vectors = [("a_log", a_log, heads), ("dt_bias", dt_bias, heads), ("skip", skip, heads), ("norm_weight", norm_weight, inner)]
    if conv_bias is not None:
        vectors.append(("conv_bias", conv_bias, channels))
    for name, t, count in vectors:
        _need(t.dtype == torch.float32 and t.numel() == count and t.is_contiguous(), f"state_space: {name} must hold {count} float32 values")
    for name, t, count in (("token_request", token_request, tokens), ("cu_seqlens", cu_seqlens, requests + 1), ("slot_ids", slot_ids, requests)):
        _need(t.dtype == torch.int32 and t.numel() >= count and t.is_contiguous(), f"state_space: {name} must be int32 [{count}]")
    for name, t, count in (("qkv", qkv, tokens * channels), ("gates", gates, tokens * 2 * heads), ("raw", raw, tokens * inner), ("skipped", skipped, tokens * inner)):
        _need(t.dtype == torch.float32 and t.is_contiguous() and t.numel() >= count, f"state_space: {name} scratch too small")
    _need(norm_parts > 0 and inner % norm_parts == 0, f"state_space: {inner} values do not divide into {norm_parts} parts")
    _launch("lrs_ssm", _dev(out, "out"), dtype_code(out.dtype), _dev(proj, "proj"), dtype_code(proj.dtype), _rows(proj, "proj"), tokens,
            requests, _dev(token_request, "token_request"), _dev(cu_seqlens, "cu_seqlens"), _dev(slot_ids, "slot_ids"), _dev(state, "state"),
            state.stride(0), _dev(conv_weight, "conv_weight"), None if conv_bias is None else _dev(conv_bias, "conv_bias"), taps, groups, heads,
            state_size, vdim, _dev(a_log, "a_log"), _dev(dt_bias, "dt_bias"), _dev(skip, "skip"), _dev(norm_weight, "norm_weight"), norm_parts,
            eps, _dev(qkv, "qkv"), _dev(gates, "gates"), _dev(raw, "raw"), _dev(skipped, "skipped"), _stream())


# ------------------------------------------------------------------- routed experts
def moe_tile_rows(pairs: int, experts: int) -> int:
    """Rows of a tile of the grouped products for a step of `pairs` (token, choice) pairs: 32, or 128 once every expert
    gets 48 rows and more on average (see csrc/moe.hip)."""
    return 128 if pairs >= 48 * experts else 32


def moe_max_tiles(pairs: int, experts: int) -> int:
    """The most row tiles that `pairs` (token, choice) pairs of `experts` experts fill once sorted by expert."""
    return min(pairs, pairs // moe_tile_rows(pairs, experts) + experts)


@dataclass(frozen=True)
class RouteRule:
    """How routed experts are chosen and weighted.  kind "softmax_chosen": the largest (logit + bias), weighted by the
    softmax over the chosen (logit + bias) alone.  kind "sigmoid": scores s = sigmoid(logit); the largest (s + bias) are
    chosen (the bias takes part in the choice only), weighted by the chosen s over their sum (+ 1e-20), times `scale`; with
    `groups` the experts form that many equal groups of neighbours, a group scores the sum of its two largest (s + bias),
    and only experts of the `keep` best groups can be chosen."""
    kind: str = "softmax_chosen"
    groups: int = 0
    keep: int = 0
    scale: float = 1.0

    KINDS = ("softmax_chosen", "sigmoid", "sigmoid_scores")     # the last: chosen as under "sigmoid", weighted by the chosen s themselves (times scale)

    def words(self) -> tuple:
        _need(self.kind in self.KINDS, f"unknown routing rule {self.kind!r}; known: {', '.join(self.KINDS)}")
        return self.KINDS.index(self.kind), self.groups, self.keep, float(self.scale)


DEFAULT_RULE = RouteRule()


def moe_route(logits: torch.Tensor, bias: torch.Tensor | None, ids: torch.Tensor, weights: torch.Tensor, rule: RouteRule = DEFAULT_RULE) -> None:
    """ids, weights [T, top]: per token the `top` experts of logits [T, E] that `rule` chooses, and their weights."""
    tokens, top = ids.shape
    experts = logits.shape[1]
    _need(logits.dtype == torch.float32 and logits.shape[0] >= tokens and logits.stride(1) == 1, "moe_route: logits must be float32 [T, E]")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == experts and bias.is_contiguous()), "moe_route: bias must hold E float32 values")
    _need(ids.dtype == torch.int32 and ids.is_contiguous() and weights.dtype == torch.float32 and weights.is_contiguous()
          and weights.shape == ids.shape, "moe_route: ids must be int32 [T, top] and weights float32 [T, top]")
    _launch("lrs_moe_route", _dev(logits, "logits"), logits.stride(0), None if bias is None else _dev(bias, "bias"), _dev(ids, "ids"),
            _dev(weights, "weights"), tokens, experts, top, *rule.words(), _stream())


def moe_align(ids: torch.Tensor, experts: int, sorted_pairs: torch.Tensor, place: torch.Tensor, tile_expert: torch.Tensor) -> None:
    """Sorts the (token, choice) pairs of ids [T, top] by expert: sorted_pairs [tiles * tile rows] (pair index, -1 in the
    rows that pad an expert's run), place [T * top] (the row of each pair), tile_expert [tiles] (-1: tile not in use)."""
    pairs, tiles = ids.numel(), tile_expert.numel()
    tile = moe_tile_rows(pairs, experts)
    for name, t in (("ids", ids), ("sorted_pairs", sorted_pairs), ("place", place), ("tile_expert", tile_expert)):
        _need(t.dtype == torch.int32 and t.is_contiguous(), f"moe_align: {name} must be contiguous int32")
    _need(tiles >= moe_max_tiles(pairs, experts) and sorted_pairs.numel() >= tiles * tile and place.numel() >= pairs,
          "moe_align: the lists are too short for the step")
    _launch("lrs_moe_align", _dev(ids, "ids"), pairs, experts, _dev(sorted_pairs, "sorted_pairs"), sorted_pairs.numel(), _dev(place, "place"),
            _dev(tile_expert, "tile_expert"), tiles, _stream())


ROUTE_ALIGN_TOKENS = 32      # steps up to which one workgroup both chooses and sorts (its 16 waves take a token each, in turns)


def moe_route_align(logits: torch.Tensor, bias: torch.Tensor | None, ids: torch.Tensor, weights: torch.Tensor, sorted_pairs: torch.Tensor,
                    place: torch.Tensor, tile_expert: torch.Tensor, rule: RouteRule = DEFAULT_RULE) -> None:
    """moe_route() and moe_align() as one launch, for steps of at most ROUTE_ALIGN_TOKENS tokens."""
    tokens, top = ids.shape
    experts, pairs, tiles = logits.shape[1], ids.numel(), tile_expert.numel()
    _need(tokens <= ROUTE_ALIGN_TOKENS, f"moe_route_align: at most {ROUTE_ALIGN_TOKENS} tokens")
    _need(logits.dtype == torch.float32 and logits.shape[0] >= tokens and logits.stride(1) == 1, "moe_route_align: logits must be float32 [T, E]")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == experts and bias.is_contiguous()), "moe_route_align: bias must hold E float32 values")
    _need(ids.dtype == torch.int32 and ids.is_contiguous() and weights.dtype == torch.float32 and weights.is_contiguous()
          and weights.shape == ids.shape, "moe_route_align: ids must be int32 [T, top] and weights float32 [T, top]")
    for name, t in (("sorted_pairs", sorted_pairs), ("place", place), ("tile_expert", tile_expert)):
        _need(t.dtype == torch.int32 and t.is_contiguous(), f"moe_route_align: {name} must be contiguous int32")
    _need(tiles >= moe_max_tiles(pairs, experts) and sorted_pairs.numel() >= tiles * moe_tile_rows(pairs, experts) and place.numel() >= pairs,
          "moe_route_align: the lists are too short for the step")
    _launch("lrs_moe_route_align", _dev(logits, "logits"), logits.stride(0), None if bias is None else _dev(bias, "bias"), _dev(ids, "ids"),
            _dev(weights, "weights"), tokens, experts, top, _dev(sorted_pairs, "sorted_pairs"), sorted_pairs.numel(), _dev(place, "place"),
            _dev(tile_expert, "tile_expert"), tiles, *rule.words(), _stream())


def moe_experts(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, sorted_pairs: torch.Tensor, tile_expert: torch.Tensor, tile: int, top: int,
                gather: bool, relu_squared: bool, silu_pairs: bool = False, clamped_pairs: tuple | None = None,
                pair_weights: torch.Tensor | None = None) -> None:
    """out [tiles * tile rows, N] = rows of `a` times w[expert of the tile] [N, K], transposed, for every tile in use.
    tile: rows of a tile, as moe_tile_rows() gave them for the step that was sorted.
    gather: the row of a sorted pair is a[pair // top] (tokens); else `a` is in sorted order itself.
    silu_pairs: w holds a gate row 2j and an up row 2j + 1 for every feature j, and out [*, N / 2] = silu(gate) * up.
    clamped_pairs (alpha, limit): the same rows, out = g * sigmoid(alpha * g) * (u + 1) with g = min(p * gate, limit) and
    u = clamp(p * up, -limit, limit); p = pair_weights[pair] (float32 [T * top], the weight of the row's (token, choice) pair:
    the expert runs on p times its input) or 1."""
    experts, n, k = w.shape
    tiles = tile_expert.numel()
    _need(tile in (32, 128), "moe_experts: tiles have 32 or 128 rows")
    _need(w.is_contiguous() and a.dtype == w.dtype and a.shape[1] == k, "moe_experts: a [*, K] and w [E, N, K] must agree")
    pairs_act = silu_pairs or clamped_pairs is not None
    _need(relu_squared + silu_pairs + (clamped_pairs is not None) <= 1 and (not pairs_act or n % 4 == 0), "moe_experts: one activation, and pairs of rows four at a time")
    _need(pair_weights is None or (clamped_pairs is not None and pair_weights.dtype == torch.float32 and pair_weights.is_contiguous()),
          "moe_experts: weights on the inputs are float32 and come with the clamped activation")
    alpha, limit = clamped_pairs if clamped_pairs is not None else (0.0, 0.0)
    _need(out.shape == (tiles * tile, n // 2 if pairs_act else n) and out.dtype in (w.dtype, torch.float32), "moe_experts: out must be [tiles * tile rows, N] (N / 2 for pairs)")
    _need(gather or a.shape[0] >= tiles * tile, "moe_experts: sorted rows missing")
    _need(sorted_pairs.numel() >= tiles * tile, "moe_experts: sorted list too short")
    _launch("lrs_moe_experts", _dev(out, "out"), dtype_code(out.dtype), _rows(out, "out"), _dev(a, "a"), _dev(w, "w"), dtype_code(w.dtype),
            _rows(a, "a"), n, k, _dev(sorted_pairs, "sorted_pairs", torch.int32), _dev(tile_expert, "tile_expert", torch.int32), tiles, tile, top,
            int(gather), 3 if clamped_pairs is not None else 2 if silu_pairs else int(relu_squared),
            None if pair_weights is None else _dev(pair_weights, "pair_weights"), float(alpha), float(limit), _stream())


def moe_combine(residual: torch.Tensor, rows: torch.Tensor, place: torch.Tensor, weights: torch.Tensor | None, norm_weight: torch.Tensor | None,
                eps: float = 0.0, rounded: torch.Tensor | None = None, layer_norm_alpha: float | None = None, top: int | None = None,
                extra: torch.Tensor | None = None) -> None:
    """residual [T, H] += sum over a token's choices of weights[t, c] * rows[place[t, c]]; with norm_weight: the RMS
    norm (weight norm_weight, eps) of that sum instead of the sum itself; with layer_norm_alpha as well: residual becomes
    the layer norm (norm_weight, eps) of layer_norm_alpha * residual + sum.  rounded: bfloat16 [T, H] that receives the
    updated rows as well.  weights None (then `top` says how many choices a token has): every choice counts once.  extra
    (float32 [T, H]): rows added to a token's sum before any norm (what a part that runs for every token gave out)."""
    if weights is not None:
        tokens, top = weights.shape
    else:
        _need(top is not None and top > 0, "moe_combine: without weights the number of choices must be given")
        tokens = place.numel() // top if extra is None else extra.shape[0]
    hidden = rows.shape[1]
    _need(residual.dtype == torch.float32 and residual.is_contiguous() and residual.shape[0] >= tokens and residual.shape[1] == hidden
          and rows.dtype == torch.float32 and rows.is_contiguous(), "moe_combine: residual [T, H] and rows [*, H] must be contiguous float32")
    _need(place.dtype == torch.int32 and place.numel() >= tokens * top and place.is_contiguous() and (weights is None or (weights.dtype == torch.float32
          and weights.is_contiguous())), "moe_combine: place must be int32 [T * top] and weights float32 [T, top]")
    _need(extra is None or (extra.dtype == torch.float32 and extra.is_contiguous() and extra.shape[0] >= tokens and extra.shape[1] == hidden),
          "moe_combine: extra rows must be contiguous float32 [T, H]")
    _need(norm_weight is None or (norm_weight.numel() == hidden and norm_weight.is_contiguous()), "moe_combine: norm weight must hold H values")
    _need(layer_norm_alpha is None or norm_weight is not None, "moe_combine: a layer norm needs its weight")
    _launch("lrs_moe_combine", _dev(residual, "residual"), _dev(rows, "rows"), tokens, hidden, _dev(place, "place"), None if weights is None else _dev(weights, "weights"), top,
            None if norm_weight is None else _dev(norm_weight, "norm_weight"), 0 if norm_weight is None else dtype_code(norm_weight.dtype), eps,
            _rounded(rounded, tokens, hidden, "moe_combine"), int(layer_norm_alpha is not None), 0.0 if layer_norm_alpha is None else layer_norm_alpha,
            None if extra is None else _dev(extra, "extra"), _stream())


# ------------------------------------------------------------------- latent attention
def latent_prep(proj: torch.Tensor, q_col: int, kv_col: int, heads: int, dim: int, rot: int, rank: int, norm_weight: torch.Tensor, eps: float,
                cos: torch.Tensor | None, sin: torch.Tensor | None, pages: torch.Tensor, slots: torch.Tensor, queries: torch.Tensor,
                value_pages: torch.Tensor | None = None) -> None:
    """Per token of proj [T, columns]: the RMS norm (norm_weight, eps) of the `rank` latent values at column kv_col and the
    rotation (pairs 2i, 2i + 1; cos, sin [T, rot / 2], None: none) of the `rot` shared key values behind them, written into
    the token's row of pages [P, 1, page, rank + rot] (slots[t] < 0: not kept); and the rotation of the last `rot` of the
    dim + rot values of every head's query (from column q_col on) into queries [T, heads, rank + rot][..., rank:].
    value_pages [P, 1, rank, page]: receives the normed latent values as well, transposed inside a page."""
    tokens, width = proj.shape[0], rank + rot
    _need(proj.dim() == 2 and proj.stride(1) == 1 and proj.shape[1] >= max(q_col + heads * (dim + rot), kv_col + width), "latent_prep: proj rows are too short")
    _need(pages.dim() == 4 and pages.shape[1] == 1 and pages.shape[3] == width and pages.is_contiguous() and pages.dtype == proj.dtype,
          f"latent_prep: pages must be contiguous [P, 1, page, {width}] of the rows' dtype")
    _need(queries.shape == (tokens, heads, width) and queries.is_contiguous() and queries.dtype == proj.dtype, f"latent_prep: queries must be [{tokens}, {heads}, {width}]")
    _need(value_pages is None or (value_pages.shape == (pages.shape[0], 1, rank, pages.shape[2]) and value_pages.is_contiguous() and value_pages.dtype == pages.dtype),
          f"latent_prep: value pages must be contiguous [P, 1, {rank}, page] of the pages' dtype")
    _need(norm_weight.numel() == rank and norm_weight.is_contiguous(), f"latent_prep: the norm weight must hold {rank} values")
    _need(slots.dtype == torch.int32 and slots.numel() >= tokens and slots.is_contiguous(), "latent_prep: slots must be int32 [T]")
    for name, t in (("cos", cos), ("sin", sin)):
        _need((t is None) == (cos is None) and (t is None or (t.dtype == torch.float32 and t.shape == (tokens, rot // 2) and t.is_contiguous())),
              f"latent_prep: {name} must be float32 [{tokens}, {rot // 2}]")
    _launch("lrs_latent_prep", _dev(proj, "proj"), proj.stride(0), dtype_code(proj.dtype), tokens, q_col, kv_col, heads, dim, rot, rank,
            _dev(norm_weight, "norm_weight"), dtype_code(norm_weight.dtype), eps, None if cos is None else _dev(cos, "cos"),
            None if sin is None else _dev(sin, "sin"), _dev(pages, "pages"), None if value_pages is None else _dev(value_pages, "value_pages"), pages.shape[2],
            _dev(slots, "slots"), _dev(queries, "queries"), heads * width, _stream())


def head_gemm(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, transposed: bool) -> None:
    """out [T, heads, n] = per head h: w[h] a[t, h] with w [heads, n, k], or w[h]^T a[t, h] with w [heads, k, n] if `transposed`.
    out and a may be views with strides of their own between tokens and heads."""
    tokens, heads, n = out.shape
    k = a.shape[2]
    _need(a.shape[:2] == (tokens, heads) and a.stride(2) == 1 and out.stride(2) == 1 and a.dtype == out.dtype == w.dtype, "head_gemm: a [T, heads, k] and out [T, heads, n] of the weights' dtype")
    _need(w.is_contiguous() and w.shape == ((heads, k, n) if transposed else (heads, n, k)), f"head_gemm: w must be contiguous [{heads}, {k if transposed else n}, {n if transposed else k}]")
    _launch("lrs_head_gemm", _dev(out, "out"), out.stride(0), out.stride(1), _dev(a, "a"), a.stride(0), a.stride(1), _dev(w, "w"), n * k, int(transposed),
            dtype_code(w.dtype), tokens, heads, n, k, _stream())


def latent_attention(out: torch.Tensor, queries: torch.Tensor, pages: torch.Tensor, block_table: torch.Tensor, token_request: torch.Tensor,
                     positions: torch.Tensor, rank: int, scale: float, sink: torch.Tensor | None = None, gate: torch.Tensor | None = None,
                     window: int = 0) -> None:
    """out [T, heads * rank] = per (token, head): softmax over the request's kept rows j <= position (within `window` if
    given) of (queries[t, h] . row_j) * scale, with exp(sink[h]) as one more term of the denominator, times row_j[:rank],
    times sigmoid(gate[t, h]).  pages [P, 1, page, width]; gate: a [T, heads] view (contiguous along heads)."""
    tokens, heads, width = queries.shape
    _need(pages.dim() == 4 and pages.shape[1] == 1 and pages.shape[3] == width and pages.is_contiguous(), f"latent_attention: pages must be contiguous [P, 1, page, {width}]")
    _need(queries.is_contiguous() and out.shape == (tokens, heads * rank) and out.stride(1) == 1 and 0 < rank <= width, "latent_attention: queries [T, heads, width], out [T, heads * rank]")
    _need(queries.dtype == pages.dtype == out.dtype, "latent_attention: queries, pages and out must share a dtype")
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.stride(1) == 1, "latent_attention: block_table must be int32 [R, blocks]")
    for name, t in (("token_request", token_request), ("positions", positions)):
        _need(t.dtype == torch.int32 and t.numel() >= tokens and t.is_contiguous(), f"latent_attention: {name} must be int32 [T]")
    _need(sink is None or (sink.dtype == torch.float32 and sink.numel() == heads and sink.is_contiguous()), "latent_attention: sink must hold a float32 per head")
    _need(gate is None or (gate.shape == (tokens, heads) and gate.stride(1) == 1 and gate.dtype == out.dtype), "latent_attention: gate must be a [T, heads] view of the run's dtype")
    _launch("lrs_latent_attention", _dev(out, "out"), out.stride(0), _dev(queries, "queries"), heads * width, _dev(pages, "pages"),
            _dev(block_table, "block_table"), block_table.stride(0), _dev(token_request, "token_request"), _dev(positions, "positions"),
            None if sink is None else _dev(sink, "sink"), None if gate is None else _dev(gate, "gate"), 0 if gate is None else gate.stride(0),
            dtype_code(out.dtype), tokens, heads, rank, width, pages.shape[2], scale, window, _stream())


def latent_attention_groups_takes(dtype: torch.dtype, rank: int, width: int, page_size: int) -> bool:
    """Whether latent_attention_groups() takes the shape (else latent_attention())."""
    return dtype == torch.bfloat16 and bool(library().lrs_latent_attention_groups_takes(rank, width, page_size))


def latent_attention_groups(out: torch.Tensor, queries: torch.Tensor, pages: torch.Tensor, value_pages: torch.Tensor, block_table: torch.Tensor,
                            token_request: torch.Tensor, positions: torch.Tensor, group_token0: torch.Tensor | None, group_count: torch.Tensor | None,
                            max_count: int, rank: int, scale: float, sink: torch.Tensor | None = None, gate: torch.Tensor | None = None, window: int = 0,
                            splits: int = 1, part_o: torch.Tensor | None = None, part_ml: torch.Tensor | None = None) -> None:
    """latent_attention() on the matrix cores, bfloat16.  group_token0 / group_count list groups of at most max_count consecutive
    tokens of one request that together cover every token once (both None: every token alone); value_pages [P, 1, rank, page]
    holds the latent values once more, transposed inside a page.  splits > 1 divides every group's keys between that many
    workgroups; their results meet in part_o [T, heads * splits * rank] and part_ml [T, heads * splits * 2] float32."""
    tokens, heads, width = queries.shape
    page_size = pages.shape[2]
    _need(pages.dim() == 4 and pages.shape[1] == 1 and pages.shape[3] == width and pages.is_contiguous(), f"latent_attention_groups: pages must be contiguous [P, 1, page, {width}]")
    _need(value_pages.shape == (pages.shape[0], 1, rank, page_size) and value_pages.is_contiguous(), f"latent_attention_groups: value pages must be contiguous [P, 1, {rank}, page]")
    _need(latent_attention_groups_takes(queries.dtype, rank, width, page_size), f"latent_attention_groups: unsupported shape rank={rank} width={width} page={page_size} {queries.dtype}")
    _need(queries.is_contiguous() and out.shape == (tokens, heads * rank) and out.stride(1) == 1, "latent_attention_groups: queries [T, heads, width], out [T, heads * rank]")
    _need(queries.dtype == pages.dtype == value_pages.dtype == out.dtype, "latent_attention_groups: queries, pages and out must share a dtype")
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.stride(1) == 1, "latent_attention_groups: block_table must be int32 [R, blocks]")
    for name, t in (("token_request", token_request), ("positions", positions)):
        _need(t.dtype == torch.int32 and t.numel() >= tokens and t.is_contiguous(), f"latent_attention_groups: {name} must be int32 [T]")
    groups = tokens
    if group_token0 is not None or group_count is not None:
        groups = group_token0.numel()
        _need(groups > 0 and group_count.numel() == groups and group_token0.dtype == group_count.dtype == torch.int32 and group_token0.is_contiguous()
              and group_count.is_contiguous(), "latent_attention_groups: the groups must be two int32 vectors of one length")
    else:
        _need(max_count == 1, "latent_attention_groups: tokens without groups stand alone")
    _need(sink is None or (sink.dtype == torch.float32 and sink.numel() == heads and sink.is_contiguous()), "latent_attention_groups: sink must hold a float32 per head")
    _need(gate is None or (gate.shape == (tokens, heads) and gate.stride(1) == 1 and gate.dtype == out.dtype), "latent_attention_groups: gate must be a [T, heads] view of the run's dtype")
    _need(1 <= splits <= 64, f"latent_attention_groups: splits must be 1..64, got {splits}")
    if splits > 1:
        _need(part_o is not None and part_o.dtype == torch.float32 and part_o.is_contiguous() and part_o.numel() >= tokens * heads * splits * rank, "latent_attention_groups: part_o too small")
        _need(part_ml is not None and part_ml.dtype == torch.float32 and part_ml.is_contiguous() and part_ml.numel() >= tokens * heads * splits * 2, "latent_attention_groups: part_ml too small")
    _launch("lrs_latent_attention_groups", _dev(out, "out"), out.stride(0), _dev(queries, "queries"), heads * width, _dev(pages, "pages"),
            _dev(value_pages, "value_pages"), _dev(block_table, "block_table"), block_table.stride(0), _dev(token_request, "token_request"),
            _dev(positions, "positions"), None if group_token0 is None else _dev(group_token0, "group_token0"),
            None if group_count is None else _dev(group_count, "group_count"), groups, max_count, None if sink is None else _dev(sink, "sink"),
            None if gate is None else _dev(gate, "gate"), 0 if gate is None else gate.stride(0), tokens, heads, rank, width, page_size, scale, window,
            splits, None if splits == 1 else _dev(part_o, "part_o"), None if splits == 1 else _dev(part_ml, "part_ml"), _stream())
