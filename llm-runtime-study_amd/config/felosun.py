"""Typed Felosun configuration read from the keys of its config.json.

A Felosun model is a stack of layers listed in config.json, each with the kind of its attention mixer (`type`:
"attention" or "attention_2"), the mixer's sizes and constants (`mixer`) and its feed-forward (`mlp`, or null for a layer
without one).  A layer with `weights_of: j` owns no tensors: it runs with layer j's (mixer, feed-forward and norms) and a cache
of its own; the rest of its entry must equal layer j's.  A learned vector per position is added to the scaled embedding, and the
logits are multiplied by a constant.  Nothing is assumed that the file does not say: a mixer without `mask` sees the whole
context, one without `rot` is not rotated, `rot.scaling` absent means plain frequencies, `softcap` absent no cap on the
scores, `shared` absent no shared expert; `embedding.scale` and `logit_scale` default to 1.

    {"architecture": "Felosun", "vocab": V, "width": W, "max_positions": P, "norm": {"eps": e}, "embedding": {"scale": s},
     "logit_scale": c, "layers": [
        {"type": "attention", "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "mask": {"size", "keep_first"},
                                        "rot": {"base", "dims"}}, "mlp": {...} | null},
        {"type": "attention_2", "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "softcap",
                                          "rot": {"base", "dims", "scaling": {"factor"}}}, "mlp": {...} | null},
        {"type": ..., "mixer": ..., "mlp": ..., "weights_of": j}, ...]}
    mlp: {"kind": "moe", "expert": {"ff", "limit"}, "router": {"experts", "top"}, "shared": {"ff", "limit"}}
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from ..errors import ConfigError
from .fields import optional, required
from .nobodra import _positive, _section


def _positive_number(raw: Mapping[str, Any], name: str, where: str) -> float:
    try:
        value = float(required(raw, name, (int, float)))
    except ConfigError as exc:
        raise ConfigError(f"{where}: {exc}") from None
    if not value > 0 or value != value or value == float("inf"):
        raise ConfigError(f"{where}: {name} must be positive and finite, got {value}")
    return value


@dataclass(frozen=True)
class FelosunExperts:
    ff: int
    limit: float
    experts: int
    top: int
    shared_ff: int | None = None
    shared_limit: float | None = None

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "FelosunExperts":
        if raw.get("kind") != "moe":
            raise ConfigError(f"{where}: unknown feed-forward kind {raw.get('kind')!r}; expected 'moe'")
        router, expert = _section(raw, "router", where), _section(raw, "expert", where)
        shared_ff = shared_limit = None
        if raw.get("shared") is not None:
            shared = _section(raw, "shared", where)
            shared_ff, shared_limit = _positive(shared, "ff", f"{where} shared"), _positive_number(shared, "limit", f"{where} shared")
        made = cls(_positive(expert, "ff", where), _positive_number(expert, "limit", where), _positive(router, "experts", where),
                   _positive(router, "top", where), shared_ff, shared_limit)
        if made.top > made.experts:
            raise ConfigError(f"{where}: top {made.top} exceeds the {made.experts} experts")
        return made

    def to_json_dict(self) -> dict:
        out = {"kind": "moe", "expert": {"ff": self.ff, "limit": self.limit}, "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff, "limit": self.shared_limit}
        return out


@dataclass(frozen=True)
class FelosunLayer:
    type: str                       # "attention" | "attention_2"
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    mlp: FelosunExperts | None
    rot_base: float | None = None
    rot_dims: int | None = None
    rot_factor: float | None = None     # every frequency divided by it
    window: int | None = None
    keep_first: int = 0
    softcap: float | None = None
    weights_of: int | None = None

    TYPES = ("attention", "attention_2")

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], index: int) -> "FelosunLayer":
        where = f"layer {index}"
        if not isinstance(raw, dict):
            raise ConfigError(f"{where} must be an object")
        kind = raw.get("type")
        if kind not in cls.TYPES:
            raise ConfigError(f"{where}: unknown type {kind!r}; expected one of: {', '.join(cls.TYPES)}")
        mixer = _section(raw, "mixer", where)
        mlp = raw.get("mlp")
        if mlp is not None and not isinstance(mlp, dict):
            raise ConfigError(f"{where}: `mlp` must be an object or null")
        made: dict = dict(type=kind, heads=_positive(mixer, "heads", where), kv_heads=_positive(mixer, "kv_heads", where),
                          dim=_positive(mixer, "dim", where), vdim=_positive(mixer, "vdim", where), scale=_positive_number(mixer, "scale", where),
                          mlp=None if mlp is None else FelosunExperts.from_dict(mlp, where))
        if made["heads"] % made["kv_heads"]:
            raise ConfigError(f"{where}: heads must be a multiple of kv_heads, got {made['heads']} and {made['kv_heads']}")
        if mixer.get("rot") is not None:
            rot = _section(mixer, "rot", where)
            made["rot_dims"], made["rot_base"] = _positive(rot, "dims", where), _positive_number(rot, "base", where)
            if made["rot_dims"] % 2 or made["rot_dims"] > made["dim"]:
                raise ConfigError(f"{where}: rot.dims must be even and at most dim, got {made['rot_dims']}")
            if rot.get("scaling") is not None:
                made["rot_factor"] = _positive_number(_section(rot, "scaling", where), "factor", where)
        # The constants below are written for one type each in the design (the window for "attention", the cap and the stretched
        # positions for "attention_2"); every mechanism is a parameter of the same mixer, so a file that gives one to the other
        # type is served as it says.
        if mixer.get("mask") is not None:
            mask = _section(mixer, "mask", where)
            made["window"] = _positive(mask, "size", where)
            kept = optional(mask, "keep_first", int, 0)
            if kept < 0:
                raise ConfigError(f"{where}: mask.keep_first must not be negative, got {kept}")
            made["keep_first"] = kept
        if mixer.get("softcap") is not None:
            made["softcap"] = _positive_number(mixer, "softcap", where)
        shared = raw.get("weights_of")
        if shared is not None and (not isinstance(shared, int) or isinstance(shared, bool)):
            raise ConfigError(f"{where}: weights_of must be a layer's number")
        return cls(weights_of=shared, **made)

    def same_shape_as(self, other: "FelosunLayer") -> bool:
        """Whether the two entries agree in everything but whose weights they run with."""
        mine, theirs = self.to_json_dict(), other.to_json_dict()
        mine.pop("weights_of", None), theirs.pop("weights_of", None)
        return mine == theirs

    def to_json_dict(self) -> dict:
        mixer: dict = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.rot_dims is not None:
            mixer["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
            if self.rot_factor is not None:
                mixer["rot"]["scaling"] = {"factor": self.rot_factor}
        if self.window is not None:
            mixer["mask"] = {"size": self.window, "keep_first": self.keep_first}
        if self.softcap is not None:
            mixer["softcap"] = self.softcap
        out = {"type": self.type, "mixer": mixer, "mlp": None if self.mlp is None else self.mlp.to_json_dict()}
        if self.weights_of is not None:
            out["weights_of"] = self.weights_of
        return out


@dataclass(frozen=True)
class FelosunConfig:
    vocab_size: int
    width: int
    norm_eps: float
    max_positions: int
    embedding_scale: float
    logit_scale: float
    layers: tuple
    eos_token_ids: tuple = ()        # the design names no end-of-sequence token: generation runs to its length limit
    model_type: str = "felosun"

    ARCHITECTURE = "Felosun"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "FelosunConfig":
        entries = raw.get("layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("layers must be a non-empty list")
        eps = _positive_number(_section(raw, "norm", "config.json"), "eps", "config.json norm")
        # what the entry of a layer that runs with another's weights leaves out (its feed-forward, say) is the owner's
        entries = [dict(entries[layer["weights_of"]], **layer) if isinstance(layer, dict) and isinstance(layer.get("weights_of"), int)
                   and not isinstance(layer.get("weights_of"), bool) and 0 <= layer["weights_of"] < len(entries)
                   and isinstance(entries[layer["weights_of"]], dict) else layer for layer in entries]
        layers = tuple(FelosunLayer.from_dict(layer, index) for index, layer in enumerate(entries))
        for index, layer in enumerate(layers):
            if layer.weights_of is None:
                continue
            if not 0 <= layer.weights_of < len(layers) or layer.weights_of == index:
                raise ConfigError(f"layer {index}: weights_of must name another layer, got {layer.weights_of}")
            owner = layers[layer.weights_of]
            if owner.weights_of is not None:
                raise ConfigError(f"layer {index}: weights_of names layer {layer.weights_of}, which has no tensors of its own")
            if not layer.same_shape_as(owner):
                raise ConfigError(f"layer {index}: a layer that runs with layer {layer.weights_of}'s weights must equal it in type, mixer and mlp")
        embedding = raw.get("embedding")
        scale = 1.0 if embedding is None else float(optional(_section(raw, "embedding", "config.json"), "scale", (int, float), 1.0))
        return cls(vocab_size=_positive(raw, "vocab", "config.json"), width=_positive(raw, "width", "config.json"), norm_eps=eps,
                   max_positions=_positive(raw, "max_positions", "config.json"), embedding_scale=scale,
                   logit_scale=float(optional(raw, "logit_scale", (int, float), 1.0)), layers=layers)

    def owners(self) -> tuple:
        """The numbers of the layers that have tensors of their own, in order."""
        return tuple(index for index, layer in enumerate(self.layers) if layer.weights_of is None)

    def validate_context_length(self, max_seq_len: int) -> None:
        if not 0 < max_seq_len <= self.max_positions:
            raise ConfigError(f"max_seq_len must be within 1..{self.max_positions} (the positions that have a learned vector), got {max_seq_len}")

    def to_json_dict(self) -> dict:
        return {"architecture": self.ARCHITECTURE, "vocab": self.vocab_size, "width": self.width, "max_positions": self.max_positions,
                "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale}, "logit_scale": self.logit_scale,
                "layers": [layer.to_json_dict() for layer in self.layers]}
