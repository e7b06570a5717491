"""Typed Kaposun configuration read from the keys of its config.json.

A Kaposun model is a stack of layers listed in config.json, each with the kind of its mixer (`type`), the mixer's sizes and
constants (`mixer`) and its feed-forward (`mlp`: a dense one, or null for a layer without one).  A stretch of the layers may
run several times in a row with the same weights (`loop`).  Every size and constant is read from the file; what the file does
not say does not exist: attention without `rot` is not rotated, without `rot.scaling` it rotates plainly, without `mask` it
sees the whole context, a mask without `keep_first` keeps nothing behind its window.

    {"architecture": "Kaposun", "vocab": V, "width": W, "norm": {"eps": e}, "residual_mult": m,
     "loop": {"start": a, "stop": b, "times": n},
     "layers": [
        {"type": "mamba2", "mixer": {"heads", "groups", "state", "vdim", "conv", "norm_groups"}, "mlp": {"kind": "dense", "ff"} | null},
        {"type": "attention", "mixer": {"heads", "kv_heads", "dim", "vdim", "scale",
                                        "rot": {"base", "dims", "scaling": {"factor"}}, "mask": {"size", "keep_first"}}, "mlp": ...},
        {"type": "parallel", "mixer": {"left": {... as attention ...}, "right": {"heads", "kv_heads", "dim", "vdim", "conv"},
                                       "left_scale", "right_scale"}, "mlp": ...}, ...]}
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from ..errors import ConfigError
from .fields import required
from .napizen import _number
from .nobodra import MAX_POSITIONS, _positive, _section


@dataclass(frozen=True)
class KaposunStateSpace:
    heads: int
    groups: int
    state: int
    vdim: int
    conv: int
    norm_groups: int

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "KaposunStateSpace":
        made = cls(*(_positive(raw, name, where) for name in ("heads", "groups", "state", "vdim", "conv", "norm_groups")))
        if made.heads % made.groups:
            raise ConfigError(f"{where}: heads must be a multiple of groups, got {made.heads} and {made.groups}")
        if (made.heads * made.vdim) % made.norm_groups:
            raise ConfigError(f"{where}: the {made.heads * made.vdim} inner values do not divide into {made.norm_groups} norm groups")
        return made

    def to_json_dict(self) -> dict:
        return {"heads": self.heads, "groups": self.groups, "state": self.state, "vdim": self.vdim, "conv": self.conv,
                "norm_groups": self.norm_groups}


@dataclass(frozen=True)
class KaposunAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: float | None = None
    rot_dims: int | None = None
    rot_factor: float | None = None      # linear scaling: every frequency divided by it
    window: int | None = None
    keep_first: int = 0

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "KaposunAttention":
        heads, kv_heads = _positive(raw, "heads", where), _positive(raw, "kv_heads", where)
        dim, vdim = _positive(raw, "dim", where), _positive(raw, "vdim", where)
        if heads % kv_heads:
            raise ConfigError(f"{where}: heads must be a multiple of kv_heads, got {heads} and {kv_heads}")
        scale = _number(raw, "scale", where)
        if not scale > 0:
            raise ConfigError(f"{where}: scale must be positive, got {scale}")
        rot_base = rot_dims = rot_factor = window = None
        keep_first = 0
        if raw.get("rot") is not None:
            rot = _section(raw, "rot", where)
            rot_dims, rot_base = _positive(rot, "dims", where), _number(rot, "base", where)
            if rot_dims % 2 or rot_dims > dim or rot_base <= 0:
                raise ConfigError(f"{where}: rot.dims must be even and at most dim, rot.base positive, got {rot_dims} and {rot_base}")
            if rot.get("scaling") is not None:
                rot_factor = _number(_section(rot, "scaling", where), "factor", where)
                if not rot_factor > 0:
                    raise ConfigError(f"{where}: rot.scaling.factor must be positive, got {rot_factor}")
        if raw.get("mask") is not None:
            mask = _section(raw, "mask", where)
            window = _positive(mask, "size", where)
            if mask.get("keep_first") is not None:
                keep_first = required(mask, "keep_first", int)
                if keep_first < 0:
                    raise ConfigError(f"{where}: mask.keep_first must not be negative, got {keep_first}")
        return cls(heads, kv_heads, dim, vdim, scale, rot_base, rot_dims, rot_factor, window, keep_first)

    def to_json_dict(self) -> dict:
        out: dict = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.rot_dims is not None:
            out["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
            if self.rot_factor is not None:
                out["rot"]["scaling"] = {"factor": self.rot_factor}
        if self.window is not None:
            out["mask"] = {"size": self.window}
            if self.keep_first:
                out["mask"]["keep_first"] = self.keep_first
        return out


@dataclass(frozen=True)
class KaposunDelta:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "KaposunDelta":
        made = cls(*(_positive(raw, name, where) for name in ("heads", "kv_heads", "dim", "vdim", "conv")))
        if made.heads % made.kv_heads:
            raise ConfigError(f"{where}: heads must be a multiple of kv_heads, got {made.heads} and {made.kv_heads}")
        return made

    def to_json_dict(self) -> dict:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}


@dataclass(frozen=True)
class KaposunSideBySide:
    left: KaposunAttention
    right: KaposunDelta
    left_scale: float
    right_scale: float

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "KaposunSideBySide":
        return cls(KaposunAttention.from_dict(_section(raw, "left", where), f"{where} (left)"),
                   KaposunDelta.from_dict(_section(raw, "right", where), f"{where} (right)"),
                   _number(raw, "left_scale", where), _number(raw, "right_scale", where))

    def to_json_dict(self) -> dict:
        return {"left": self.left.to_json_dict(), "right": self.right.to_json_dict(), "left_scale": self.left_scale,
                "right_scale": self.right_scale}


MIXERS = {"mamba2": KaposunStateSpace, "attention": KaposunAttention, "parallel": KaposunSideBySide}


@dataclass(frozen=True)
class KaposunLayer:
    type: str                       # "mamba2" | "attention" | "parallel"
    mixer: Any                      # the dataclass MIXERS names for the type
    ff: int | None                  # the dense feed-forward's inner size; None: the layer has none

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], index: int) -> "KaposunLayer":
        where = f"layer {index}"
        if not isinstance(raw, dict):
            raise ConfigError(f"{where} must be an object")
        kind = raw.get("type")
        if kind not in MIXERS:
            raise ConfigError(f"{where}: unknown type {kind!r}; expected one of: {', '.join(MIXERS)}")
        mlp = raw.get("mlp")
        ff = None
        if mlp is not None:
            if not isinstance(mlp, dict):
                raise ConfigError(f"{where}: `mlp` must be an object or null")
            if mlp.get("kind") != "dense":
                raise ConfigError(f"{where}: unknown feed-forward kind {mlp.get('kind')!r}; expected 'dense'")
            ff = _positive(mlp, "ff", where)
        return cls(kind, MIXERS[kind].from_dict(_section(raw, "mixer", where), where), ff)

    def to_json_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_json_dict(), "mlp": None if self.ff is None else {"kind": "dense", "ff": self.ff}}


@dataclass(frozen=True)
class KaposunConfig:
    vocab_size: int
    width: int
    norm_eps: float
    residual_mult: float             # the factor of a layer's output in x <- x + m * (mixer(h) + feed_forward(h))
    layers: tuple
    loop: tuple | None = None        # (start, stop, times): layers start .. stop-1 run `times` times in a row
    eos_token_ids: tuple = ()        # the design names no end-of-sequence token: generation runs to its length limit
    model_type: str = "kaposun"

    ARCHITECTURE = "Kaposun"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "KaposunConfig":
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("layers must be a non-empty list")
        eps = _number(_section(raw, "norm", "config.json"), "eps", "config.json")
        if eps <= 0:
            raise ConfigError(f"norm.eps must be positive, got {eps}")
        loop = None
        if raw.get("loop") is not None:
            section = _section(raw, "loop", "config.json")
            start, stop, times = required(section, "start", int), required(section, "stop", int), _positive(section, "times", "loop")
            if not 0 <= start <= stop <= len(layers):
                raise ConfigError(f"loop: start and stop must lie within the {len(layers)} layers, got {start} and {stop}")
            loop = (start, stop, times)
        return cls(vocab_size=_positive(raw, "vocab", "config.json"), width=_positive(raw, "width", "config.json"), norm_eps=eps,
                   residual_mult=_number(raw, "residual_mult", "config.json", 1.0),
                   layers=tuple(KaposunLayer.from_dict(layer, index) for index, layer in enumerate(layers)), loop=loop)

    def layer_order(self) -> tuple:
        """The layers in the order they run: the looped stretch as many times as the loop says."""
        count = len(self.layers)
        if self.loop is None:
            return tuple(range(count))
        start, stop, times = self.loop
        return tuple(range(start)) + tuple(range(start, stop)) * times + tuple(range(stop, count))

    @property
    def random_rank(self) -> int:
        """The rank of the delta rule's low-rank inputs (decay, output gate) when weights are drawn at random: a checkpoint's
        tensors give it otherwise, config.json does not."""
        return max(4, self.width // 32)

    def validate_context_length(self, max_seq_len: int) -> None:
        if not 0 < max_seq_len <= MAX_POSITIONS:
            raise ConfigError(f"max_seq_len must be within 1..{MAX_POSITIONS}, got {max_seq_len}")

    def to_json_dict(self) -> dict:
        out = {"architecture": self.ARCHITECTURE, "vocab": self.vocab_size, "width": self.width, "norm": {"eps": self.norm_eps},
               "residual_mult": self.residual_mult, "layers": [layer.to_json_dict() for layer in self.layers]}
        if self.loop is not None:
            out["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        return out
