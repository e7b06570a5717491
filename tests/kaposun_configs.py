"""Small Kaposun configurations of the tests' own, differing from each other in every size, constant, layer order and loop."""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


def dense(ff):
    return {"kind": "dense", "ff": ff}


def attention_sizes(heads, kv_heads, dim, vdim, scale, rot=None, mask=None):
    """rot: (base, dims) or (base, dims, factor); mask: (size,) or (size, keep_first)."""
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rot is not None:
        mixer["rot"] = {"base": rot[0], "dims": rot[1]}
        if len(rot) > 2:
            mixer["rot"]["scaling"] = {"factor": rot[2]}
    if mask is not None:
        mixer["mask"] = {"size": mask[0]}
        if len(mask) > 1:
            mixer["mask"]["keep_first"] = mask[1]
    return mixer


def attention(heads, kv_heads, dim, vdim, scale, rot=None, mask=None, mlp=None):
    return {"type": "attention", "mixer": attention_sizes(heads, kv_heads, dim, vdim, scale, rot, mask), "mlp": mlp}


def mamba(heads, groups, state, vdim, conv, norm_groups, mlp=None):
    return {"type": "mamba2", "mixer": {"heads": heads, "groups": groups, "state": state, "vdim": vdim, "conv": conv, "norm_groups": norm_groups},
            "mlp": mlp}


def parallel(left, right, left_scale, right_scale, mlp=None):
    """left: attention_sizes(...); right: (heads, kv_heads, dim, vdim, conv)."""
    return {"type": "parallel", "mixer": {"left": left, "right": dict(zip(("heads", "kv_heads", "dim", "vdim", "conv"), right)),
                                          "left_scale": left_scale, "right_scale": right_scale}, "mlp": mlp}


def model(vocab, width, eps, mult, layers, loop=None):
    raw = {"architecture": "Kaposun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult, "layers": layers}
    if loop is not None:
        raw["loop"] = dict(zip(("start", "stop", "times"), loop))
    return raw


# odd sizes throughout: values wider and narrower than keys, part of a head rotated with stretched positions, three heads to a key
# group, a window shorter than a page with kept positions, a looped stretch in the middle, a layer without feed-forward
ODD = model(173, 64, 1e-5, 0.7, [
    attention(6, 2, 16, 24, 0.3, rot=(500.0, 8, 4.0), mlp=dense(48)),
    mamba(3, 1, 20, 24, 3, 3, mlp=None),
    parallel(attention_sizes(2, 1, 32, 16, 0.2, mask=(9, 3)), (4, 2, 24, 8, 2), 0.8, 1.5, mlp=dense(40)),
    mamba(2, 2, 72, 40, 4, 1, mlp=dense(32)),
], loop=(1, 3, 2))
# sizes the matrix-core kernels take (heads of 64 and 128, values as wide as keys), kept positions that reach into a second
# page, a window of several pages, no loop at all, plain rotation of whole heads
CORES = model(300, 128, 2e-6, 0.35, [
    mamba(4, 4, 128, 64, 2, 4, mlp=dense(192)),
    attention(4, 2, 64, 64, 0.125, rot=(1e4, 64), mlp=dense(128)),
    parallel(attention_sizes(2, 1, 128, 128, 0.09, mask=(40, 17)), (2, 1, 128, 64, 4), 1.3, 0.4, mlp=dense(64)),
    attention(8, 2, 32, 32, 0.2, rot=(1e6, 16, 2.0), mlp=None),
])
# what a model may make equal or one: one head, one key group, a convolution of one tap, a window of one, nothing kept, scales
# and multiplier of one, a loop over the whole model and a layer that follows itself
ONES = model(90, 48, 3e-6, 1.0, [
    parallel(attention_sizes(1, 1, 16, 16, 0.25, mask=(1,)), (1, 1, 8, 8, 1), 1.0, 1.0, mlp=dense(24)),
    mamba(1, 1, 8, 16, 1, 1, mlp=None),
    attention(2, 2, 8, 8, 0.35, rot=(100.0, 8), mlp=dense(16)),
], loop=(0, 3, 2))
SELF_LOOP = model(120, 32, 1e-6, 0.5, [
    attention(2, 1, 16, 16, 0.25, rot=(1e4, 16, 8.0), mlp=dense(32)),
    parallel(attention_sizes(4, 4, 8, 12, 0.35, mask=(20, 2)), (2, 2, 16, 16, 3), 0.6, 0.9, mlp=None),
], loop=(1, 2, 3))
# sizes no kernel likes: a width, heads, states and a vocabulary that are multiples of neither 8 nor 16, five taps, 20 query heads
# on one key group, a rotated part of six dims, more kept positions than the window holds, a loop of one layer run once
AWKWARD = model(251, 100, 4e-6, 0.45, [
    mamba(5, 5, 12, 20, 5, 5, mlp=dense(90)),
    attention(20, 1, 20, 12, 0.22, rot=(3000.0, 6, 1.5), mlp=dense(44)),
    parallel(attention_sizes(3, 3, 40, 40, 0.16, mask=(6, 11)), (6, 3, 20, 12, 5), 0.9, 1.1, mlp=None),
    attention(2, 1, 36, 52, 0.17, mlp=dense(60)),
], loop=(2, 3, 1))
# wide enough that prompts go through the products for many rows (the vendor library's in bfloat16)
WIDE = model(1000, 512, 1e-6, 0.25, [
    mamba(8, 2, 64, 64, 4, 2, mlp=dense(512)),
    attention(8, 2, 64, 64, 0.125, rot=(1e5, 64, 2.0), mlp=dense(768)),
    parallel(attention_sizes(4, 2, 96, 96, 0.1, mask=(150, 5)), (4, 4, 64, 64, 4), 1.1, 0.7, mlp=dense(512)),
], loop=(0, 2, 2))


def write_folder(raw: dict, seed: int, folder, ranks=(5, 9), edit=None) -> Path:
    """A model folder with random weights for `raw`.  ranks: of the delta rule's decay and gate inputs (sizes that only the
    checkpoint's tensors give); edit(tensors) may change the tensors before they are written."""
    from safetensors.torch import load_file, save_file

    from llm_runtime_study_amd.config import config_from_dict
    from llm_runtime_study_amd.weights import write_model_dir

    folder = Path(folder)
    write_model_dir(config_from_dict(raw), seed=seed, model_dir=folder, init="scaled", free_size=ranks[0])
    assert json.loads((folder / "config.json").read_text()) == raw
    tensors = load_file(str(folder / "model.safetensors"))
    g = torch.Generator().manual_seed(seed + 1000)
    for name in list(tensors):
        if name.endswith(".g1"):      # the gate's rank differs from the decay's
            width = tensors[name].shape[1]
            outputs = tensors[name[:-1] + "2"].shape[0]
            tensors[name] = (torch.randn(ranks[1], width, generator=g) / math.sqrt(width)).to(torch.bfloat16)
            tensors[name[:-1] + "2"] = (torch.randn(outputs, ranks[1], generator=g) / math.sqrt(ranks[1])).to(torch.bfloat16)
    if edit is not None:
        edit(tensors)
    save_file({name: t.contiguous() for name, t in tensors.items()}, str(folder / "model.safetensors"))
    return folder
