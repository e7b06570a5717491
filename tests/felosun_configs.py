"""Small Felosun configurations of the tests' own, differing from each other in every size, constant and layer order."""

from __future__ import annotations

import json
from pathlib import Path


def experts(ff, limit, count, top, shared=None):
    """shared: (ff, limit) of the shared expert, or None."""
    out = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": count, "top": top}}
    if shared is not None:
        out["shared"] = {"ff": shared[0], "limit": shared[1]}
    return out


def windowed(heads, kv_heads, dim, vdim, scale, rot=None, mask=None, mlp=None, weights_of=None):
    """Layer of type "attention".  rot: (base, dims); mask: (size, keep_first)."""
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rot is not None:
        mixer["rot"] = {"base": rot[0], "dims": rot[1]}
    if mask is not None:
        mixer["mask"] = {"size": mask[0], "keep_first": mask[1]}
    out = {"type": "attention", "mixer": mixer, "mlp": mlp}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def capped(heads, kv_heads, dim, vdim, scale, rot=None, softcap=None, mlp=None, weights_of=None):
    """Layer of type "attention_2".  rot: (base, dims) or (base, dims, factor)."""
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rot is not None:
        mixer["rot"] = {"base": rot[0], "dims": rot[1]}
        if len(rot) > 2:
            mixer["rot"]["scaling"] = {"factor": rot[2]}
    if softcap is not None:
        mixer["softcap"] = softcap
    out = {"type": "attention_2", "mixer": mixer, "mlp": mlp}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def shares(layer, owner):
    """The entry of a layer that runs with layer `owner`'s weights: `layer`'s own entry once more, and whose weights."""
    return dict(json.loads(json.dumps(layer)), weights_of=owner)


def model(vocab, width, eps, positions, embedding_scale, logit_scale, layers):
    return {"architecture": "Felosun", "vocab": vocab, "width": width, "max_positions": positions, "norm": {"eps": eps},
            "embedding": {"scale": embedding_scale}, "logit_scale": logit_scale, "layers": layers}


# odd sizes throughout: values wider and narrower than keys, three heads to a key group, a rotated part of six dims that are
# stretched, a window shorter than a page with kept positions, an expert size that is odd, two of five experts, a layer
# without feed-forward, a layer that shares weights with one two places before it
_ODD_0 = capped(6, 2, 20, 12, 0.21, rot=(700.0, 6, 3.0), softcap=4.0, mlp=experts(22, 1.5, 5, 2, shared=(10, 0.7)))
_ODD_1 = windowed(3, 1, 24, 40, 0.3, rot=(3000.0, 24), mask=(9, 3), mlp=experts(15, 0.8, 7, 3, shared=(18, 2.0)))
ODD = model(211, 72, 1e-5, 160, 3.5, 0.6, [_ODD_0, _ODD_1, windowed(2, 2, 16, 16, 0.4, rot=(50.0, 4), mask=(13, 0)), shares(_ODD_0, 0), shares(_ODD_1, 1)])
# sizes the matrix-core kernels take (heads of 64, 128 and 32, values as wide as keys), kept positions that reach into a second
# page, a window of several pages, more experts than a wave has lanes, whole heads rotated
_CORES_1 = windowed(4, 2, 64, 64, 0.11, rot=(1e4, 64), mask=(40, 17), mlp=experts(64, 1.0, 70, 3, shared=(96, 1.2)))
CORES = model(300, 128, 2e-6, 256, 8.0, 0.3, [
    capped(2, 1, 128, 128, 0.08, rot=(1e5, 32, 2.0), softcap=20.0, mlp=experts(32, 3.0, 8, 1)),
    _CORES_1,
    capped(8, 2, 32, 32, 0.2, rot=(1e6, 16), softcap=6.0, mlp=experts(48, 0.9, 4, 4, shared=(16, 1.0))),
    shares(_CORES_1, 1),
])
# what a model may make equal or one: one head, one key group, one expert of which one is chosen, a window of one, nothing kept,
# a rotated part of one pair, no cap, no stretching, no shared expert, scales of one, every layer but the first sharing its weights
_ONES_0 = windowed(1, 1, 8, 8, 0.35, rot=(100.0, 2), mask=(1, 0), mlp=experts(12, 1.0, 1, 1))
ONES = model(90, 48, 3e-6, 128, 1.0, 1.0, [_ONES_0, shares(_ONES_0, 0), capped(1, 1, 16, 16, 0.25, mlp=experts(8, 0.5, 2, 1)), shares(_ONES_0, 0)])
# sizes no kernel likes: a width, heads and a vocabulary that are multiples of neither 8 nor 16, 20 query heads on one key group,
# more kept positions than the window holds, a layer that shares the weights of a later one
_AWKWARD_2 = capped(20, 1, 20, 12, 0.22, rot=(3000.0, 10, 1.5), softcap=50.0, mlp=experts(26, 1.1, 9, 2, shared=(7, 0.4)))
AWKWARD = model(251, 100, 4e-6, 200, 0.7, 2.5, [
    shares(_AWKWARD_2, 2),
    windowed(3, 3, 40, 40, 0.16, rot=(20.0, 40), mask=(6, 11), mlp=None),
    _AWKWARD_2,
    windowed(2, 1, 36, 52, 0.17, mask=(30, 2), mlp=experts(30, 2.0, 3, 3)),
])
# wide enough that prompts go through the products for many rows (the vendor library's in bfloat16) and the grouped products
# with large tiles
_WIDE_0 = capped(8, 2, 64, 64, 0.125, rot=(1e5, 64, 2.0), softcap=15.0, mlp=experts(256, 1.0, 4, 2, shared=(384, 1.0)))
WIDE = model(1000, 512, 1e-6, 512, 5.0, 0.5, [
    _WIDE_0,
    windowed(4, 2, 96, 96, 0.1, rot=(1e4, 48), mask=(150, 5), mlp=experts(128, 1.5, 6, 1, shared=(256, 1.0))),
    shares(_WIDE_0, 0),
])


def write_folder(raw: dict, seed: int, folder, edit=None) -> Path:
    """A model folder with random weights for `raw`; edit(tensors) may change the tensors before they are written.  The sinks
    are drawn wider than biases are, so that they carry weight in the softmax."""
    from safetensors.torch import load_file, save_file

    from llm_runtime_study_amd.config import config_from_dict
    from llm_runtime_study_amd.weights import write_model_dir

    folder = Path(folder)
    write_model_dir(config_from_dict(raw), seed=seed, model_dir=folder, init="scaled")
    assert json.loads((folder / "config.json").read_text()) == raw
    tensors = load_file(str(folder / "model.safetensors"))
    for name in list(tensors):
        if name.endswith(".sink"):
            tensors[name] = (tensors[name].float() * 20.0 + 1.0).to(tensors[name].dtype)
        if name == "pos":
            tensors[name] = (tensors[name].float() * 0.5).to(tensors[name].dtype)
    if edit is not None:
        edit(tensors)
    save_file({name: t.contiguous() for name, t in tensors.items()}, str(folder / "model.safetensors"))
    return folder
