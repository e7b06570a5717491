"""Felosun: configuration -> ModelSpec.

The embedding is scaled and a learned vector per position added.  Every layer normalises what its sublayers give out
(h += norm1(mixer(h)), h += norm2(feed_forward(h)), the sublayers reading h itself), with plain RMS norms.  A layer's mixer
is grouped-query attention whose q and k heads are rotated first and then divided by their own root mean square, of two kinds:
  "attention"    biases on q, k and v; neighbouring dims (2i, 2i + 1) rotated; a sliding window that keeps a sequence's first
                 positions visible; a learned sink per head in the softmax's denominator;
  "attention_2"  no biases; dims (i, i + rot/2) rotated with every frequency divided by a constant; the scaled scores capped
                 by cap * tanh(score / cap); the whole context; one sigmoid gate per head on the heads' outputs.
(The window, the cap and the stretched positions are constants of a layer's entry: a layer of either kind has what its entry gives.)
The feed-forward is a set of routed experts chosen by their largest sigmoid scores, each run on its score times the
token (not weighted afterwards, not renormalised), with a clamped gated activation, and a shared expert beside them.  A layer
may run with another layer's weights and a cache of its own: such a layer is a second schedule entry of the layer it names.
The model's norm, the head and a constant factor on the logits follow the last layer.

Checkpoint tensors are named without a `.weight` ending: `embed`, `pos`, `head`, `final.norm`, `l<i>.norm1`, `l<i>.mix.q`,
`l<i>.mix.q.b`, `l<i>.mix.sink`, `l<i>.mix.g`, `l<i>.mlp.router`, `l<i>.mlp.e<j>.gate`, `l<i>.mlp.shared.up`, i being the
layer's number in config.json.
"""

from __future__ import annotations

from ..config.felosun import FelosunConfig, FelosunLayer
from ..parts import PartSpec
from .nobodra import checkpoint_name as _short_name
from .spec import ModelSpec, ScheduleEntry

LAYER_NAMES = {"mixer": "mix", "feed_forward": "mlp", "mixer_norm": "norm1", "ff_norm": "norm2"}
SWISH_ALPHA = 1.702      # the design's constant in g * sigmoid(alpha * g)


def checkpoint_name(name: str) -> str:
    """The checkpoint's name of the tensor that the parts call `name`."""
    name = _short_name(name)
    return name[:-len(".bias")] + ".b" if name.endswith(".bias") else name


def _mixer(config: FelosunConfig, layer: FelosunLayer) -> PartSpec:
    first = layer.type == "attention"
    position = PartSpec("none")
    if layer.rot_dims is not None and first:
        position = PartSpec("rope_interleaved", {"rotary_dim": layer.rot_dims, "theta": layer.rot_base, "factor": layer.rot_factor or 1.0})
    elif layer.rot_dims is not None:
        position = PartSpec("rope_half", {"rotary_dim": layer.rot_dims, "theta": layer.rot_base, "factor": layer.rot_factor or 1.0})
    return PartSpec("gqa_attention", {
        "hidden_size": config.width, "num_heads": layer.heads, "num_kv_heads": layer.kv_heads, "head_dim": layer.dim, "value_dim": layer.vdim,
        "position": position, "unit_norm_after_rotation": True, "qk_norm_eps": config.norm_eps, "scale": layer.scale,
        "bias": first, "window": layer.window, "keep_first": layer.keep_first if layer.window is not None else 0, "sink": first,
        "score_cap": layer.softcap, "output_gate": False if first else "head"})


def _feed_forward(config: FelosunConfig, layer: FelosunLayer) -> PartSpec:
    mlp = layer.mlp
    shared = None
    if mlp.shared_ff is not None:
        shared = PartSpec("swiglu", {"hidden_size": config.width, "intermediate_size": mlp.shared_ff, "activation": "clamped",
                                     "alpha": SWISH_ALPHA, "limit": mlp.shared_limit})
    return PartSpec("routed_experts", {
        "hidden_size": config.width, "intermediate_size": mlp.ff, "num_experts": mlp.experts, "top": mlp.top, "rule": "sigmoid_scores",
        "activation": "clamped_gated", "activation_alpha": SWISH_ALPHA, "activation_limit": mlp.limit, "weight_on": "input", "shared": shared})


def build_spec(config: FelosunConfig) -> ModelSpec:
    norm = PartSpec("rmsnorm", {"size": config.width, "eps": config.norm_eps})
    owners = config.owners()
    place = {number: index for index, number in enumerate(owners)}
    layers = []
    for number in owners:
        layer = config.layers[number]
        params = {"mixer": _mixer(config, layer), "mixer_norm": norm, "names": LAYER_NAMES}
        if layer.mlp is not None:
            params["feed_forward"] = _feed_forward(config, layer)
            params["ff_norm"] = norm
        layers.append(PartSpec("outnorm", params))
    # a layer that runs with another's weights is one more run of that layer, with a cache of its own
    schedule = tuple(ScheduleEntry(place[number if layer.weights_of is None else layer.weights_of]) for number, layer in enumerate(config.layers))
    return ModelSpec(
        architecture=FelosunConfig.ARCHITECTURE, vocab_size=config.vocab_size, hidden_size=config.width, layers=tuple(layers),
        schedule=schedule, final_norm=norm, max_positions=config.max_positions, eos_token_ids=(),
        embedding_multiplier=config.embedding_scale, embedding_name="embed", head_name="head", final_norm_prefix="final.norm",
        layer_prefix="l{index}", layer_numbers=owners, checkpoint_dtype="bfloat16", checkpoint_name=checkpoint_name,
        after_embedding=PartSpec("learned_positions", {"rows": config.max_positions, "size": config.width}), after_embedding_prefix="pos",
        after_head=None if config.logit_scale == 1.0 else PartSpec("scale", {"factor": config.logit_scale}))
