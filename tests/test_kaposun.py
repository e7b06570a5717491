"""Kaposun without a GPU: its configuration, the tensors it asks a checkpoint for, what its layers keep between steps, the
order in which a looped stretch runs, and the plain implementation's mechanisms against properties that follow from their
definitions."""

import json
import math

import pytest
import torch

from tests import kaposun_configs as configs
from tests.plain import kaposun as plain

F64 = torch.float64


def test_configuration_reads_back_and_names_its_tensors(tmp_path):
    from llm_runtime_study_amd.config import config_from_dict, load_config, spec_for
    from llm_runtime_study_amd.config.kaposun import KaposunConfig
    from llm_runtime_study_amd.models import DecoderModel
    from llm_runtime_study_amd.parts import BothNeeds, PagedKVNeed, StateNeed

    for raw in (configs.ODD, configs.CORES, configs.ONES, configs.SELF_LOOP, configs.WIDE, configs.AWKWARD):
        config = config_from_dict(raw)
        assert isinstance(config, KaposunConfig) and config.to_json_dict() == raw
        model = DecoderModel(spec_for(config))
        names = model.tensors()
        assert {"embed", "final.norm", "l0.norm1"} <= set(names) and not any(name.endswith(".weight") for name in names)
        assert not any(".norm2" in name for name in names)          # one norm a layer
        width = raw["width"]
        for index, layer in enumerate(raw["layers"]):
            m, p = layer["mixer"], f"l{index}.mix."
            if layer["type"] == "mamba2":
                inner, bc = m["heads"] * m["vdim"], m["groups"] * m["state"]
                assert names[p + "in"].shape == (2 * inner + 2 * bc + m["heads"], width)
                assert names[p + "conv"].shape == (inner + 2 * bc, m["conv"]) and names[p + "conv.b"].shape == (inner + 2 * bc,)
                assert names[p + "norm"].shape == (inner,) and names[p + "D"].shape == (m["heads"],) and names[p + "o"].shape == (width, inner)
            elif layer["type"] == "attention":
                assert names[p + "q.norm"].shape == (m["heads"] * m["dim"],) and names[p + "k.norm"].shape == (m["kv_heads"] * m["dim"],)
                assert names[p + "v"].shape == (m["kv_heads"] * m["vdim"], width) and names[p + "o"].shape == (width, m["heads"] * m["vdim"])
                assert p + "g" not in names
            else:
                left, right = m["left"], m["right"]
                assert names[p + "left.g"].shape == (left["heads"] * left["vdim"], width)
                assert names[p + "left.q.norm"].shape == (left["heads"] * left["dim"],)
                assert names[p + "right.q.conv"].shape == (right["kv_heads"] * right["dim"], right["conv"])
                assert names[p + "right.v.conv"].shape == (right["heads"] * right["vdim"], right["conv"])
                assert names[p + "right.dt_bias"].shape == (right["heads"] * right["dim"],) and names[p + "right.b"].shape == (right["heads"], width)
                assert names[p + "right.a2"].shape[0] == right["heads"] * right["dim"] and names[p + "right.g2"].shape[0] == right["heads"] * right["vdim"]
                assert names[p + "right.norm"].shape == (right["vdim"],)
            if layer["mlp"] is None:
                assert not any(name.startswith(f"l{index}.mlp.") for name in names)
            else:
                assert names[f"l{index}.mlp.up"].shape == (layer["mlp"]["ff"], width) and names[f"l{index}.mlp.down"].shape == (width, layer["mlp"]["ff"])
        order = plain.layer_order(raw)
        assert [entry.layer for entry in model.spec.schedule] == order
        needs = model.cache_needs()
        assert len(needs) == len(order)              # every run of a looped layer keeps a cache or state of its own
        for index, need in zip(order, needs):
            layer = raw["layers"][index]
            if layer["type"] == "mamba2":
                assert isinstance(need, StateNeed) and need.dtype == torch.float32
            elif layer["type"] == "attention":
                m = layer["mixer"]
                assert isinstance(need, PagedKVNeed) and (need.num_kv_heads, need.head_dim, need.window) == (m["kv_heads"], m["dim"], None)
                assert (need.value_dim or need.head_dim) == m["vdim"]
            else:
                left = layer["mixer"]["left"]
                assert isinstance(need, BothNeeds) and need.state.dtype == torch.float32
                assert (need.paged.window, need.paged.keep_first) == (left["mask"]["size"], left["mask"].get("keep_first", 0))
        assert model.graph_safe() and model.plan_safe()
    folder = configs.write_folder(configs.ODD, 3, tmp_path / "m", ranks=(3, 7))
    assert load_config(folder).to_json_dict() == configs.ODD
    _, tensors = plain.load_folder(folder)
    assert tensors["l2.mix.right.a1"].shape[0] == 3 and tensors["l2.mix.right.g2"].shape[1] == 7


def test_a_looped_stretch_runs_in_a_row():
    from llm_runtime_study_amd.config import config_from_dict

    assert config_from_dict(configs.ODD).layer_order() == (0, 1, 2, 1, 2, 3)
    assert config_from_dict(configs.ONES).layer_order() == (0, 1, 2, 0, 1, 2)
    assert config_from_dict(configs.SELF_LOOP).layer_order() == (0, 1, 1, 1)
    assert config_from_dict(configs.CORES).layer_order() == (0, 1, 2, 3)
    once = json.loads(json.dumps(configs.ODD))
    once["loop"] = {"start": 2, "stop": 2, "times": 5}          # an empty stretch: nothing runs twice
    assert config_from_dict(once).layer_order() == (0, 1, 2, 3)


@pytest.mark.parametrize("broken,message", [
    (lambda raw: raw["layers"][0].update(type="conv"), "unknown type"),
    (lambda raw: raw["layers"][0]["mixer"].update(kv_heads=4), "multiple of kv_heads"),
    (lambda raw: raw["layers"][0]["mixer"]["rot"].update(dims=18), "rot.dims"),
    (lambda raw: raw["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda raw: raw["layers"][1]["mixer"].update(groups=2), "multiple of groups"),
    (lambda raw: raw["layers"][1]["mixer"].update(norm_groups=5), "norm groups"),
    (lambda raw: raw["layers"][2]["mixer"].pop("right"), "right"),
    (lambda raw: raw["layers"][2]["mixer"]["left"]["mask"].update(keep_first=-1), "keep_first"),
    (lambda raw: raw["layers"][3].update(mlp={"kind": "moe", "ff": 8}), "feed-forward kind"),
    (lambda raw: raw["loop"].update(stop=9), "loop"),
    (lambda raw: raw.pop("norm"), "norm"),
    (lambda raw: raw.update(layers=[]), "non-empty"),
])
def test_configuration_refuses(broken, message):
    from llm_runtime_study_amd.config import config_from_dict
    from llm_runtime_study_amd.errors import ConfigError

    raw = json.loads(json.dumps(configs.ODD))
    broken(raw)
    with pytest.raises(ConfigError, match=message):
        config_from_dict(raw)


def test_checkpoint_names():
    from llm_runtime_study_amd.models.kaposun import checkpoint_name

    assert [checkpoint_name(name) for name in ("l3.mix.in_proj.weight", "l3.mix.conv.weight", "l3.mix.conv.bias", "l0.mix.left.q_norm.weight",
                                                "l0.mix.left.g_proj.weight", "l0.mix.right.k_conv.weight", "l0.mix.right.a2_proj.weight", "l0.mix.right.dt_bias",
                                                "l1.mlp.up_proj.weight", "l1.norm1.weight", "final.norm.weight", "embed")] == \
        ["l3.mix.in", "l3.mix.conv", "l3.mix.conv.b", "l0.mix.left.q.norm", "l0.mix.left.g", "l0.mix.right.k.conv", "l0.mix.right.a2", "l0.mix.right.dt_bias",
         "l1.mlp.up", "l1.norm1", "final.norm", "embed"]


def test_parts_refuse_what_their_kernels_do_not_take():
    from llm_runtime_study_amd.parts import PartSpec, create

    base = {"hidden_size": 8, "num_heads": 2, "num_kv_heads": 1, "head_dim": 8, "qk_norm": True, "norm_over": "projection"}
    with pytest.raises(ValueError, match="needs a window"):
        create("mixer", PartSpec("gqa_attention", dict(base, keep_first=2)))
    with pytest.raises(ValueError, match="norm_over"):
        create("mixer", PartSpec("gqa_attention", dict(base, norm_over="token")))
    with pytest.raises(ValueError, match="per-head norms"):
        create("mixer", PartSpec("gqa_attention", dict(base, norm_over="head", keep_first=2, window=4)))
    assert "k_proj.bias" in create("mixer", PartSpec("gqa_attention", dict(base, bias=True))).tensors()      # biases are added in the projection
    ssm = {"hidden_size": 8, "num_heads": 4, "num_groups": 2, "state_size": 8, "value_dim": 6, "conv_taps": 2, "norm_parts": 3, "norm_eps": 1e-6}
    create("mixer", PartSpec("state_space", ssm))
    with pytest.raises(ValueError, match="parts"):
        create("mixer", PartSpec("state_space", dict(ssm, norm_parts=5)))
    with pytest.raises(ValueError, match="num_groups"):
        create("mixer", PartSpec("state_space", dict(ssm, num_groups=3)))
    attention = PartSpec("gqa_attention", dict(base, window=4))
    with pytest.raises(ValueError, match="one set of pages"):
        create("mixer", PartSpec("side_by_side", {"left": attention, "right": attention}))
    with pytest.raises(ValueError, match="unknown activation"):
        create("feed_forward", PartSpec("dense_mlp", {"hidden_size": 8, "intermediate_size": 8, "activation": "tanh"}))


# ------------------------------------------------------------- the plain mechanisms against their definitions
def test_plain_norms_and_activations():
    torch.manual_seed(0)
    x = torch.randn(4, 12, dtype=F64)
    torch.testing.assert_close(plain.unit_rms(x, 0.0).pow(2).mean(-1), torch.ones(4, dtype=F64))
    tiny = 1e-4 * x
    assert (plain.unit_rms(tiny, 1e-2).pow(2).mean(-1) < 1e-4).all()             # eps under the root tames tiny rows
    torch.testing.assert_close(plain.gelu_exact(x), torch.nn.functional.gelu(x))
    assert (plain.gelu_exact(x) - torch.nn.functional.gelu(x, approximate="tanh")).abs().max() > 1e-5
    torch.testing.assert_close(plain.soft_plus(torch.tensor([-50.0, 0.0, 50.0], dtype=F64)), torch.tensor([math.exp(-50.0), math.log(2.0), 50.0], dtype=F64))
    torch.testing.assert_close(plain.swish(x), torch.nn.functional.silu(x))


def test_plain_taps_and_turns():
    x = torch.arange(12, dtype=F64).view(6, 2)
    taps = torch.tensor([[0.0, 0.0, 1.0], [1.0, 0.0, 0.0]], dtype=F64)
    y = plain.causal_taps(x, taps, torch.tensor([0.0, 5.0], dtype=F64))
    torch.testing.assert_close(y[:, 0], x[:, 0])                                                     # the last tap is the current token's
    torch.testing.assert_close(y[:, 1], 5.0 + torch.cat((torch.zeros(2, dtype=F64), x[:4, 1])))      # the first looks two back, zeros before the start
    q = torch.randn(5, 2, 8, dtype=F64)
    r = plain.turn_front(q, 100.0, 4, 1.0)
    torch.testing.assert_close(r[0], q[0])                                                           # position 0 is not turned
    torch.testing.assert_close(r[..., 4:], q[..., 4:])
    torch.testing.assert_close(r[..., :4].norm(dim=-1), q[..., :4].norm(dim=-1))
    angle = 3 * 100.0 ** (-2.0 / 4)
    torch.testing.assert_close(r[3, 1, 1], q[3, 1, 1] * math.cos(angle) - q[3, 1, 3] * math.sin(angle))
    torch.testing.assert_close(r[3, 1, 3], q[3, 1, 3] * math.cos(angle) + q[3, 1, 1] * math.sin(angle))
    # stretched positions: dividing every frequency by 4 turns position 4 as plain rotation turns position 1
    torch.testing.assert_close(plain.turn_front(q, 100.0, 4, 4.0)[4], plain.turn_front(q[[4, 4]], 100.0, 4, 1.0)[1])


def test_plain_window_keeps_the_first_positions():
    seen = [[j for j in range(12) if plain.sees(i, j, 3, 2)] for i in range(12)]
    assert seen[0] == [0] and seen[2] == [0, 1, 2] and seen[4] == [0, 1, 2, 3, 4] and seen[5] == [0, 1, 3, 4, 5] and seen[11] == [0, 1, 9, 10, 11]
    assert [j for j in range(12) if plain.sees(11, j, 3, 0)] == [9, 10, 11] and [j for j in range(5) if plain.sees(4, j, None, 0)] == list(range(5))
    torch.manual_seed(1)
    n, width, heads, groups, d, e = 9, 12, 4, 2, 6, 5
    x = torch.randn(n, width, dtype=F64)
    w = {"q": torch.randn(heads * d, width, dtype=F64), "k": torch.randn(groups * d, width, dtype=F64), "v": torch.randn(groups * e, width, dtype=F64),
         "o": torch.randn(width, heads * e, dtype=F64), "q.norm": torch.ones(heads * d, dtype=F64), "k.norm": torch.ones(groups * d, dtype=F64),
         "g": torch.zeros(heads * e, width, dtype=F64)}
    sizes = dict(heads=heads, groups=groups, d=d, e=e, eps=1e-6, scale=0.3)
    full = plain.softmax_attention(x, w, **sizes)
    torch.testing.assert_close(plain.softmax_attention(x, w, **sizes, window=n), full)
    torch.testing.assert_close(plain.softmax_attention(x, w, **sizes, window=2, kept=n), full)           # everything kept: the window hides nothing
    torch.testing.assert_close(plain.softmax_attention(x, w, **sizes, gated=True), 0.5 * full)           # a gate of sigmoid(0)
    one = plain.softmax_attention(x, w, **sizes, window=1)                                               # a window of one: the token's own value
    alone = (x @ w["v"].T).view(n, groups, e).repeat_interleave(heads // groups, 1).reshape(n, heads * e) @ w["o"].T
    torch.testing.assert_close(one, alone)
    # the norm is over the whole projection: scaling one head's rows of W_q changes the other heads' queries too
    scaled = dict(w, q=torch.cat((5.0 * w["q"][:d], w["q"][d:])))
    q_rows = plain.unit_rms(x @ scaled["q"].T, 1e-6)
    assert (q_rows[:, d:] - plain.unit_rms(x @ w["q"].T, 1e-6)[:, d:]).abs().max() > 0.1


def test_plain_state_space_against_its_closed_form():
    """With B, C, dt and the decay made constant (zero projections, convolution of bias alone), the state is a geometric
    sum: y_t = (sum_{s<=t} a^(t-s) dt (B.C) u_s) + D u_t."""
    torch.manual_seed(2)
    heads, groups, state, e, taps, width, n = 2, 1, 3, 4, 2, 6, 7
    inner, bc = heads * e, groups * state
    w_in = torch.zeros(2 * inner + 2 * bc + heads, width, dtype=F64)
    w_in[inner:2 * inner] = torch.randn(inner, width, dtype=F64)                   # only u depends on the input
    conv = torch.zeros(inner + 2 * bc, taps, dtype=F64)
    conv[:inner, -1] = 1.0
    bias = torch.cat((torch.zeros(inner, dtype=F64), torch.full((2 * bc,), 0.7, dtype=F64)))
    w = {"in": w_in, "conv": conv, "conv.b": bias, "dt_bias": torch.tensor([0.3, -0.2], dtype=F64), "A_log": torch.tensor([-0.5, 0.4], dtype=F64),
         "D": torch.tensor([1.5, -0.5], dtype=F64), "norm": torch.ones(inner, dtype=F64), "o": torch.eye(inner, dtype=F64)}
    x = torch.randn(n, width, dtype=F64)
    got = plain.state_space(x, w, heads=heads, groups=groups, state=state, e=e, taps=taps, parts=1, eps=1e-9)
    u = plain.swish(x @ w_in[inner:2 * inner].T).view(n, heads, e)
    b_dot_c = state * plain.swish(torch.tensor(0.7, dtype=F64)) ** 2
    dt = plain.soft_plus(w["dt_bias"])
    a = torch.exp(-torch.exp(w["A_log"]) * dt)
    y = torch.zeros(n, heads, e, dtype=F64)
    for t in range(n):
        for s in range(t + 1):
            y[t] += (a ** (t - s) * dt * b_dot_c)[:, None] * u[s]
        y[t] += w["D"][:, None] * u[t]
    gated = y.reshape(n, inner) * plain.swish(torch.zeros((), dtype=F64))       # z is zero: the gate is silu(0) = 0 ...
    assert gated.abs().max() == 0 and got.abs().max() < 1e-6                  # ... and so is the output: the gate comes before the norm
    w_in[:inner] = torch.randn(inner, width, dtype=F64)
    got = plain.state_space(x, w, heads=heads, groups=groups, state=state, e=e, taps=taps, parts=2, eps=1e-9)
    gated = (y.reshape(n, inner) * plain.swish(x @ w_in[:inner].T)).view(n, 2, inner // 2)
    torch.testing.assert_close(got, plain.unit_rms(gated, 1e-9).reshape(n, inner))


def test_plain_delta_rule_with_channel_decay():
    """A decay per key channel: what was written under channel 0 fades, what was written under channel 3 stays; reading
    right after a full-step write gives the value back."""
    d, e = 6, 5
    k1, k2 = torch.zeros(d, dtype=F64), torch.zeros(d, dtype=F64)
    k1[0], k2[3] = 1.0, 1.0
    torch.manual_seed(3)
    v1, v2 = torch.randn(e, dtype=F64), torch.randn(e, dtype=F64)
    g = torch.ones(d, dtype=F64)
    g[0] = 0.5
    memory = torch.zeros(d, e, dtype=F64)
    for k, v in ((k1, v1), (k2, v2)):
        memory = g[:, None] * memory
        memory = memory + torch.outer(k, 1.0 * (v - memory.T @ k))
    torch.testing.assert_close(memory.T @ k2, v2)              # the read-out sees the current token's write
    torch.testing.assert_close(memory.T @ k1, 0.5 * v1)        # one step of channel 0's decay
    memory = g[:, None] * memory
    torch.testing.assert_close(memory.T @ k2, v2)
    torch.testing.assert_close(memory.T @ k1, 0.25 * v1)


def test_plain_model_is_causal_and_its_loop_reuses_weights(tmp_path):
    folder = configs.write_folder(configs.SELF_LOOP, 9, tmp_path / "m")
    raw, tensors = plain.load_folder(folder)
    tokens = torch.randint(0, raw["vocab"], (30,)).tolist()
    streams = []
    logits = plain.forward(raw, tensors, tokens, streams)
    assert logits.shape == (30, raw["vocab"]) and len(streams) == 4
    shorter = plain.forward(raw, tensors, tokens[:17])
    torch.testing.assert_close(logits[:17], shorter)
    unrolled = json.loads(json.dumps(raw))
    unrolled["layers"] = [raw["layers"][0]] + [raw["layers"][1]] * 3
    unrolled.pop("loop")
    copies = dict(tensors)
    for name, t in tensors.items():
        if name.startswith("l1."):
            copies["l2." + name[3:]] = copies["l3." + name[3:]] = t
    torch.testing.assert_close(plain.forward(unrolled, copies, tokens), logits)
