"""Kaposun: configuration -> ModelSpec.

Every layer has one RMS norm whose output both sublayers read, and adds their sum, times a constant m of the model, to the
stream: with x = norm1(h), h <- h + m * (mixer(x) + feed_forward(x)).  The mixer is one of
  a selective state space recurrence (a matrix per head written by outer products, a gated norm in parts at its output),
  grouped-query attention whose q and k are normalised over the whole projection, rotated in halves with every frequency
    divided by a constant, seeing the whole context,
  two mixers side by side, their outputs added with a weight each: attention of that kind without rotation, behind a sliding
    window that keeps a sequence's first positions visible, with a sigmoid gate on the heads' outputs; and the gated delta rule
    with a decay per head and key channel.
The feed-forward is two matrices with the exact gelu between them.  A stretch of the layers may run several times in a row
with the same weights, each run with a cache or state of its own.  The model's norm follows the last layer; the head is the
embedding table.

Checkpoint tensors are named without a `.weight` ending: `embed`, `final.norm`, `l<i>.norm1`, `l<i>.mix.in`, `l<i>.mix.conv.b`,
`l<i>.mix.q.norm`, `l<i>.mix.left.g`, `l<i>.mix.right.q.conv`, `l<i>.mix.right.a1`, `l<i>.mlp.up`.
"""

from __future__ import annotations

from ..config.kaposun import KaposunAttention, KaposunConfig, KaposunDelta, KaposunStateSpace
from ..config.nobodra import MAX_POSITIONS
from ..parts import PartSpec
from .nobodra import checkpoint_name as _short_name
from .spec import ModelSpec, ScheduleEntry

LAYER_NAMES = {"mixer": "mix", "feed_forward": "mlp", "norm": "norm1"}


def checkpoint_name(name: str) -> str:
    """The checkpoint's name of the tensor that the parts call `name`."""
    return _short_name(name).replace("conv.bias", "conv.b")


def _attention(config: KaposunConfig, sizes: KaposunAttention, gated: bool) -> PartSpec:
    position = PartSpec("none")
    if sizes.rot_dims is not None:
        position = PartSpec("rope_half", {"rotary_dim": sizes.rot_dims, "theta": sizes.rot_base, "factor": sizes.rot_factor or 1.0})
    return PartSpec("gqa_attention", {
        "hidden_size": config.width, "num_heads": sizes.heads, "num_kv_heads": sizes.kv_heads, "head_dim": sizes.dim, "value_dim": sizes.vdim,
        "position": position, "qk_norm": True, "qk_norm_eps": config.norm_eps, "norm_over": "projection", "scale": sizes.scale,
        "window": sizes.window, "keep_first": sizes.keep_first if sizes.window is not None else 0, "output_gate": gated})


def _delta(config: KaposunConfig, sizes: KaposunDelta) -> PartSpec:
    # the ranks of the decay's and the gate's inputs are what the checkpoint's tensors hold
    return PartSpec("gated_delta_rule", {
        "hidden_size": config.width, "num_heads": sizes.heads, "num_kv_heads": sizes.kv_heads, "head_dim": sizes.dim, "value_dim": sizes.vdim,
        "conv_taps": sizes.conv, "norm_eps": config.norm_eps, "channel_decay": True})


def _state_space(config: KaposunConfig, sizes: KaposunStateSpace) -> PartSpec:
    return PartSpec("state_space", {
        "hidden_size": config.width, "num_heads": sizes.heads, "num_groups": sizes.groups, "state_size": sizes.state, "value_dim": sizes.vdim,
        "conv_taps": sizes.conv, "norm_parts": sizes.norm_groups, "norm_eps": config.norm_eps})


def _mixer(config: KaposunConfig, layer) -> PartSpec:
    if layer.type == "mamba2":
        return _state_space(config, layer.mixer)
    if layer.type == "attention":
        return _attention(config, layer.mixer, gated=False)
    pair = layer.mixer
    return PartSpec("side_by_side", {"left": _attention(config, pair.left, gated=True), "right": _delta(config, pair.right),
                                     "left_scale": pair.left_scale, "right_scale": pair.right_scale})


def build_spec(config: KaposunConfig) -> ModelSpec:
    norm = PartSpec("rmsnorm", {"size": config.width, "eps": config.norm_eps})
    layers = []
    for layer in config.layers:
        params = {"mixer": _mixer(config, layer), "norm": norm, "multiplier": config.residual_mult, "names": LAYER_NAMES}
        if layer.ff is not None:
            params["feed_forward"] = PartSpec("dense_mlp", {"hidden_size": config.width, "intermediate_size": layer.ff, "activation": "gelu"})
        layers.append(PartSpec("parallel", params))
    return ModelSpec(
        architecture=KaposunConfig.ARCHITECTURE, vocab_size=config.vocab_size, hidden_size=config.width, layers=tuple(layers),
        schedule=tuple(ScheduleEntry(i) for i in config.layer_order()), final_norm=norm, max_positions=MAX_POSITIONS,
        eos_token_ids=(), tie_head=True, embedding_name="embed", head_name="head", final_norm_prefix="final.norm", layer_prefix="l{index}",
        checkpoint_dtype="bfloat16", checkpoint_name=checkpoint_name)
