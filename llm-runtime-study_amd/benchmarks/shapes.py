"""Layer sizes of the Qwen3 dense models the benchmarks run with random weights (config.json keys)."""

QWEN3_8B = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "vocab_size": 151936, "hidden_size": 4096,
    "intermediate_size": 12288, "num_hidden_layers": 36, "num_attention_heads": 32, "num_key_value_heads": 8,
    "head_dim": 128, "max_position_embeddings": 40960, "rms_norm_eps": 1e-6, "rope_theta": 1000000.0,
    "hidden_act": "silu", "attention_bias": False, "attention_dropout": 0.0, "tie_word_embeddings": False,
    "torch_dtype": "bfloat16", "bos_token_id": 151643, "eos_token_id": 151645,
}
# the other dense models of the family (the reference's own published figures are for the smallest)
SHAPES = {
    "0.6b": dict(QWEN3_8B, hidden_size=1024, intermediate_size=3072, num_hidden_layers=28, num_attention_heads=16, tie_word_embeddings=True),
    "1.7b": dict(QWEN3_8B, hidden_size=2048, intermediate_size=6144, num_hidden_layers=28, num_attention_heads=16, tie_word_embeddings=True),
    "4b": dict(QWEN3_8B, hidden_size=2560, intermediate_size=9728, num_hidden_layers=36, num_attention_heads=32, tie_word_embeddings=True),
    "8b": QWEN3_8B,
    "14b": dict(QWEN3_8B, hidden_size=5120, intermediate_size=17408, num_hidden_layers=40, num_attention_heads=40),
    "32b": dict(QWEN3_8B, hidden_size=5120, intermediate_size=25600, num_hidden_layers=64, num_attention_heads=64),
}


def nobodra_like(shape: dict, layers: int, experts: int = 32, top: int = 8, window: int = 4096, attention_only: bool = False) -> dict:
    """A Nobodra configuration with the layer sizes of a dense shape above, for measurements beside it: the same width,
    vocabulary and heads; three gated-delta-rule layers to every sliding-window attention layer (with `attention_only` every
    layer is a sliding-window attention layer); the dense feed-forward's
    three matrices of `intermediate_size` as `top` of `experts` experts of two matrices each with as many weights in use
    per token (to a multiple of 128); half of every attention head rotated."""
    width, heads, kv_heads, dim = shape["hidden_size"], shape["num_attention_heads"], shape["num_key_value_heads"], shape["head_dim"]
    ff = max(128, round(3 * shape["intermediate_size"] / (2 * top) / 128) * 128)
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    attention = {"type": "attention", "mlp": mlp, "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5,
                                                            "mask": {"size": window}, "rot": {"base": 1000000.0, "dims": dim // 2}}}
    delta = {"type": "delta", "mlp": mlp, "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "conv": 4}}
    return {"architecture": "Nobodra", "vocab": shape["vocab_size"], "width": width, "norm": {"eps": 1e-6},
            "layers": [attention if index % 4 == 3 or attention_only else delta for index in range(layers)]}


def felosun_like(shape: dict, layers: int, experts: int = 32, top: int = 8, window: int = 4096, keep_first: int = 8, positions: int = 40960) -> dict:
    """A Felosun configuration with the layer sizes of a dense shape above, for measurements beside a model of equal sizes: the
    same width, vocabulary and heads; in turn a layer of capped attention over the whole context (half of every head rotated,
    stretched positions, a gate a head) and a layer of windowed attention with kept first positions and sinks (half of every head
    rotated in neighbouring pairs); `top` of `experts` clamped gated experts and a shared expert of the same size, together as
    many weights in use per token as the dense feed-forward (to a multiple of 128)."""
    width, heads, kv_heads, dim = shape["hidden_size"], shape["num_attention_heads"], shape["num_key_value_heads"], shape["head_dim"]
    ff = max(128, round(shape["intermediate_size"] / (top + 1) / 128) * 128)
    mlp = {"kind": "moe", "expert": {"ff": ff, "limit": 7.0}, "router": {"experts": experts, "top": top}, "shared": {"ff": ff, "limit": 7.0}}
    sizes = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5}
    capped = {"type": "attention_2", "mlp": mlp, "mixer": dict(sizes, rot={"base": 1000000.0, "dims": dim // 2, "scaling": {"factor": 4.0}}, softcap=50.0)}
    windowed = {"type": "attention", "mlp": mlp, "mixer": dict(sizes, rot={"base": 10000.0, "dims": dim // 2}, mask={"size": window, "keep_first": keep_first})}
    return {"architecture": "Felosun", "vocab": shape["vocab_size"], "width": width, "max_positions": positions, "norm": {"eps": 1e-6},
            "embedding": {"scale": 1.0}, "logit_scale": 0.5, "layers": [(capped, windowed)[index % 2] for index in range(layers)]}


def napizen_like(shape: dict, layers: int, experts: int = 32, top: int = 8, rank: int = 512, rot: int = 64) -> dict:
    """A Napizen configuration with the layer sizes of a dense shape above, for measurements beside it: the same width,
    vocabulary and number of heads; heads of the shape's size plain and `rot` rotated dims, values of the shape's head size,
    `rank` latent values a position; layers with the dense feed-forward of the shape's `intermediate_size` in turn with layers
    of `top` of `experts` gated experts with as many weights in use per token (to a multiple of 128), chosen among half of
    eight groups."""
    width, heads, dim = shape["hidden_size"], shape["num_attention_heads"], shape["head_dim"]
    ff = max(128, round(shape["intermediate_size"] / top / 128) * 128)
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": dim, "kv_rank": rank, "scale": (dim + rot) ** -0.5,
             "rot": {"base": 500000.0, "dims": rot, "scaling": {"factor": 8.0, "original": 8192, "fast": 24.0, "slow": 2.0}}}
    dense = {"kind": "dense", "ff": shape["intermediate_size"]}
    routed = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": 2.5, "groups": {"count": 8, "keep": 4}}}
    return {"architecture": "Napizen", "vocab": shape["vocab_size"], "width": width, "norm": {"eps": 1e-6}, "postln_alpha": 2.0,
            "embedding": {"scale": 1.0}, "logit_softcap": 50.0,
            "layers": [{"type": "latent_attention", "mixer": mixer, "mlp": routed if index % 2 else dense} for index in range(layers)]}


def kaposun_like(shape: dict, layers: int, window: int = 4096, keep_first: int = 8, state: int = 128) -> dict:
    """A Kaposun configuration with the layer sizes of a dense shape above, for measurements beside it: the same width,
    vocabulary, heads and dense feed-forward size (two matrices where the shape has three); in turn a state space layer
    (inner size twice the width in heads of 64 values, `state` numbers a value, 8 groups), an attention layer over the whole
    context with stretched rotation, a layer of windowed attention with kept first positions and an output gate beside the
    gated delta rule with channel decays, and another attention layer; no stretch of layers runs twice."""
    width, heads, kv_heads, dim = shape["hidden_size"], shape["num_attention_heads"], shape["num_key_value_heads"], shape["head_dim"]
    mlp = {"kind": "dense", "ff": shape["intermediate_size"]}
    sizes = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5}
    attention = {"type": "attention", "mlp": mlp, "mixer": dict(sizes, rot={"base": 500000.0, "dims": dim, "scaling": {"factor": 4.0}})}
    state_space = {"type": "mamba2", "mlp": mlp, "mixer": {"heads": 2 * width // 64, "groups": 8, "state": state, "vdim": 64, "conv": 4, "norm_groups": 8}}
    pair = {"type": "parallel", "mlp": mlp, "mixer": {"left": dict(sizes, mask={"size": window, "keep_first": keep_first}),
                                                      "right": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "conv": 4},
                                                      "left_scale": 1.0, "right_scale": 1.0}}
    return {"architecture": "Kaposun", "vocab": shape["vocab_size"], "width": width, "norm": {"eps": 1e-6}, "residual_mult": 0.5,
            "layers": [(state_space, attention, pair, attention)[index % 4] for index in range(layers)]}
