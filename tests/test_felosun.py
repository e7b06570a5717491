"""Felosun without a GPU: its configuration, the tensors it asks a checkpoint for, what its layers keep between steps, layers
that share weights, and the plain implementation's mechanisms against properties that follow from their definitions."""

import copy
import math

import pytest
import torch

from tests import felosun_configs as configs
from tests.plain import felosun as plain

F64 = torch.float64
ALL = {"odd": configs.ODD, "cores": configs.CORES, "ones": configs.ONES, "awkward": configs.AWKWARD, "wide": configs.WIDE}


def test_configuration_reads_back_and_names_its_tensors():
    from llm_runtime_study_amd.config import config_from_dict, spec_for
    from llm_runtime_study_amd.config.felosun import FelosunConfig
    from llm_runtime_study_amd.models import DecoderModel
    from llm_runtime_study_amd.parts import PagedKVNeed

    for raw in ALL.values():
        config = config_from_dict(raw)
        assert isinstance(config, FelosunConfig) and config.to_json_dict() == raw
        model = DecoderModel(spec_for(config))
        names = model.tensors()
        width = raw["width"]
        assert {"embed", "pos", "head", "final.norm"} <= set(names) and not any(name.endswith(".weight") for name in names)
        assert names["pos"].shape == (raw["max_positions"], width)
        owners = [index for index, layer in enumerate(raw["layers"]) if "weights_of" not in layer]
        for index, layer in enumerate(raw["layers"]):
            m, p = layer["mixer"], f"l{index}.mix."
            if "weights_of" in layer:
                assert not any(name.startswith(f"l{index}.") for name in names)       # no tensors of its own
                continue
            assert names[p + "q"].shape == (m["heads"] * m["dim"], width) and names[p + "k"].shape == (m["kv_heads"] * m["dim"], width)
            assert names[p + "v"].shape == (m["kv_heads"] * m["vdim"], width) and names[p + "o"].shape == (width, m["heads"] * m["vdim"])
            if layer["type"] == "attention":
                assert names[p + "q.b"].shape == (m["heads"] * m["dim"],) and names[p + "v.b"].shape == (m["kv_heads"] * m["vdim"],)
                assert names[p + "sink"].shape == (m["heads"],) and p + "g" not in names
            else:
                assert names[p + "g"].shape == (m["heads"], width) and p + "sink" not in names and p + "q.b" not in names
            mlp = layer["mlp"]
            if mlp is None:
                assert not any(name.startswith(f"l{index}.mlp.") or name == f"l{index}.norm2" for name in names)
                continue
            assert names[f"l{index}.norm2"].shape == (width,)
            assert names[f"l{index}.mlp.router"].shape == (mlp["router"]["experts"], width)
            last = mlp["router"]["experts"] - 1
            assert names[f"l{index}.mlp.e{last}.gate"].shape == (mlp["expert"]["ff"], width)
            assert names[f"l{index}.mlp.e0.down"].shape == (width, mlp["expert"]["ff"])
            assert (f"l{index}.mlp.shared.up" in names) == ("shared" in mlp)
            if "shared" in mlp:
                assert names[f"l{index}.mlp.shared.down"].shape == (width, mlp["shared"]["ff"])
        # every run has a cache of its own, and a layer that shares weights is one more run of the layer it names
        assert [owners[entry.layer] for entry in model.spec.schedule] == [layer.get("weights_of", index) for index, layer in enumerate(raw["layers"])]
        needs = model.cache_needs()
        assert len(needs) == len(raw["layers"])
        for layer, need in zip(raw["layers"], needs):
            m = layer["mixer"]
            assert isinstance(need, PagedKVNeed) and need.num_kv_heads == m["kv_heads"] and need.head_dim == m["dim"]
            assert need.window == m.get("mask", {}).get("size") and need.keep_first == m.get("mask", {}).get("keep_first", 0)


def test_what_the_file_leaves_out_does_not_exist():
    from llm_runtime_study_amd.config import config_from_dict

    raw = copy.deepcopy(configs.ODD)
    del raw["embedding"], raw["logit_scale"]
    del raw["layers"][0]["mixer"]["softcap"], raw["layers"][0]["mixer"]["rot"]["scaling"], raw["layers"][0]["mlp"]["shared"]
    del raw["layers"][1]["mixer"]["mask"], raw["layers"][2]["mixer"]["rot"]
    raw["layers"][3], raw["layers"][4] = configs.shares(raw["layers"][0], 0), configs.shares(raw["layers"][1], 1)
    config = config_from_dict(raw)
    assert config.embedding_scale == 1.0 and config.logit_scale == 1.0
    first, second, third = config.layers[:3]
    assert first.softcap is None and first.rot_factor is None and first.mlp.shared_ff is None
    assert second.window is None and second.keep_first == 0 and third.rot_dims is None
    # the entry of a layer that runs with another's weights may leave out what equals the owner's
    del raw["layers"][4]["mlp"]
    assert config_from_dict(raw).layers[4].mlp == config.layers[1].mlp


def refused(change):
    from llm_runtime_study_amd.config import config_from_dict
    from llm_runtime_study_amd.errors import ConfigError

    raw = copy.deepcopy(configs.ODD)
    change(raw)
    with pytest.raises(ConfigError) as caught:
        config_from_dict(raw)
    return str(caught.value)


def test_refusals_name_the_layer():
    assert "layer 2" in refused(lambda raw: raw["layers"][2].update(type="mamba"))
    assert "heads" in refused(lambda raw: raw["layers"][0]["mixer"].update(heads=5))
    assert "rot.dims" in refused(lambda raw: raw["layers"][0]["mixer"]["rot"].update(dims=7))
    assert "rot.dims" in refused(lambda raw: raw["layers"][0]["mixer"]["rot"].update(dims=22))
    assert "factor" in refused(lambda raw: raw["layers"][0]["mixer"]["rot"].update(scaling={"factor": 0.0}))
    assert "softcap" in refused(lambda raw: raw["layers"][0]["mixer"].update(softcap=-5.0))
    assert "size" in refused(lambda raw: raw["layers"][1]["mixer"]["mask"].pop("size"))
    assert "top" in refused(lambda raw: raw["layers"][0]["mlp"]["router"].update(top=6))
    assert "limit" in refused(lambda raw: raw["layers"][0]["mlp"]["expert"].pop("limit"))
    assert "kind" in refused(lambda raw: raw["layers"][0]["mlp"].update(kind="dense"))
    assert "keep_first" in refused(lambda raw: raw["layers"][1]["mixer"]["mask"].update(keep_first=-1))
    assert "weights_of" in refused(lambda raw: raw["layers"][3].update(weights_of=3))
    assert "weights_of" in refused(lambda raw: raw["layers"][3].update(weights_of=9))
    assert "no tensors of its own" in refused(lambda raw: raw["layers"][4].update(weights_of=3))
    assert "must equal" in refused(lambda raw: raw["layers"][3]["mixer"].update(scale=0.5))
    assert "max_positions" in refused(lambda raw: raw.pop("max_positions"))
    assert "eps" in refused(lambda raw: raw["norm"].update(eps=0.0))


def test_a_constant_given_to_the_other_type_is_served():
    """The window is written for one type of layer, the cap and the stretched positions for the other; each is a parameter of
    the same mixer, so a file that gives one to the other type gets it."""
    from llm_runtime_study_amd.config import config_from_dict, spec_for

    raw = copy.deepcopy(configs.ODD)
    raw["layers"][1]["mixer"]["rot"]["scaling"] = {"factor": 2.0}
    raw["layers"][1]["mixer"]["softcap"] = 5.0
    raw["layers"][0]["mixer"]["mask"] = {"size": 4, "keep_first": 1}
    raw["layers"][3], raw["layers"][4] = configs.shares(raw["layers"][0], 0), configs.shares(raw["layers"][1], 1)
    config = config_from_dict(raw)
    assert config.to_json_dict() == raw
    spec = spec_for(config)
    first, second = spec.layers[0].params["mixer"].params, spec.layers[1].params["mixer"].params
    assert first["window"] == 4 and first["keep_first"] == 1 and first["score_cap"] == 4.0 and first["output_gate"] == "head"
    assert second["score_cap"] == 5.0 and second["position"].params["factor"] == 2.0 and second["sink"] is True


def test_context_length_is_bounded_by_the_learned_positions():
    from llm_runtime_study_amd.config import config_from_dict
    from llm_runtime_study_amd.errors import ConfigError

    config = config_from_dict(configs.ODD)
    config.validate_context_length(configs.ODD["max_positions"])
    with pytest.raises(ConfigError):
        config.validate_context_length(configs.ODD["max_positions"] + 1)


def test_parts_refuse_what_they_cannot_run():
    from llm_runtime_study_amd.parts import PartSpec, create

    sizes = {"hidden_size": 32, "num_heads": 2, "num_kv_heads": 1, "head_dim": 16}
    with pytest.raises(ValueError):
        create("mixer", PartSpec("gqa_attention", dict(sizes, qk_norm=True, unit_norm_after_rotation=True)))
    with pytest.raises(ValueError):
        create("mixer", PartSpec("gqa_attention", dict(sizes, score_cap=0.0)))
    with pytest.raises(ValueError):
        create("mixer", PartSpec("gqa_attention", dict(sizes, output_gate="token")))
    with pytest.raises(ValueError):
        create("mixer", PartSpec("gqa_attention", dict(sizes, sink=True, kv_shared=True)))
    experts = {"hidden_size": 32, "intermediate_size": 8, "num_experts": 4, "top": 2}
    with pytest.raises(ValueError):
        create("feed_forward", PartSpec("routed_experts", dict(experts, activation="clamped_gated")))              # no limit
    with pytest.raises(ValueError):
        create("feed_forward", PartSpec("routed_experts", dict(experts, activation="silu_gated", weight_on="input")))
    with pytest.raises(ValueError):
        create("feed_forward", PartSpec("swiglu", {"hidden_size": 32, "intermediate_size": 8, "activation": "clamped"}))
    gate = create("mixer", PartSpec("gqa_attention", dict(sizes, output_gate="head", value_dim=24)))
    assert gate.tensors()["g_proj.weight"].shape == (2, 32) and gate.tensors()["o_proj.weight"].shape == (32, 48)


# ------------------------------------------------------------------------------------- the plain mechanisms
def values(*shape, seed=0, scale=1.0):
    return scale * torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F64)


def attention_weights(kind, m, seed=1, width=24):
    w = {"q": values(m["heads"] * m["dim"], width, seed=seed), "k": values(m["kv_heads"] * m["dim"], width, seed=seed + 1),
         "v": values(m["kv_heads"] * m["vdim"], width, seed=seed + 2), "o": values(width, m["heads"] * m["vdim"], seed=seed + 3)}
    if kind == "attention":
        w.update({"q.b": values(m["heads"] * m["dim"], seed=seed + 4), "k.b": values(m["kv_heads"] * m["dim"], seed=seed + 5),
                  "v.b": values(m["kv_heads"] * m["vdim"], seed=seed + 6), "sink": values(m["heads"], seed=seed + 7)})
    else:
        w["g"] = values(m["heads"], width, seed=seed + 8)
    return w


def test_which_keys_a_window_with_kept_positions_shows():
    mask = {"size": 4, "keep_first": 2}
    assert [j for j in range(12) if plain.visible(9, j, mask)] == [0, 1, 6, 7, 8, 9]
    assert [j for j in range(12) if plain.visible(3, j, mask)] == [0, 1, 2, 3]
    assert [j for j in range(12) if plain.visible(9, j, {"size": 1})] == [9]
    assert [j for j in range(5) if plain.visible(3, j, None)] == [0, 1, 2, 3]


def test_rotation_layouts_and_stretching():
    x = values(5, 2, 8, seed=3)
    rot = {"base": 100.0, "dims": 4}
    near, halves = plain.turn(x, rot, "neighbours"), plain.turn(x, rot, "halves")
    assert torch.equal(near[..., 4:], x[..., 4:]) and torch.equal(halves[..., 4:], x[..., 4:])        # the rest of a head passes
    assert torch.equal(near[0], x[0])                                                                # position 0 turns nothing
    p, rate = 3, 100.0 ** (-2.0 / 4)
    u, v = x[p, 1, 2], x[p, 1, 3]                                                                    # neighbours: pair 1 is dims (2, 3)
    assert torch.allclose(near[p, 1, 2], u * math.cos(p * rate) - v * math.sin(p * rate))
    assert torch.allclose(near[p, 1, 3], v * math.cos(p * rate) + u * math.sin(p * rate))
    u, v = x[p, 1, 1], x[p, 1, 3]                                                                    # halves: pair 1 is dims (1, 3)
    assert torch.allclose(halves[p, 1, 1], u * math.cos(p * rate) - v * math.sin(p * rate))
    stretched = plain.turn(x, dict(rot, scaling={"factor": 3.0}), "halves")
    assert torch.allclose(stretched[3], plain.turn(x[3:4], rot, "halves", first_position=1)[0])      # position 3 at a third of the pace
    assert torch.allclose(near.pow(2).sum(-1), x.pow(2).sum(-1))                                     # a rotation keeps lengths


def test_a_sink_takes_weight_and_gives_nothing():
    m = {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 6, "scale": 0.3, "mask": {"size": 5, "keep_first": 1}, "rot": {"base": 50.0, "dims": 8}}
    w = attention_weights("attention", m)
    x = values(11, 24, seed=9)
    seen = []
    plain.attention(x, w, m, 1e-5, "attention", weights_out=seen)
    for h, i, keys, weights in seen:
        assert keys == [j for j in range(i + 1) if plain.visible(i, j, m["mask"])]
        assert 0 < float(weights.sum()) < 1                                      # the rest is the sink's share
    far_below, far_above = dict(w, sink=torch.full((2,), -80.0, dtype=F64)), dict(w, sink=torch.full((2,), 80.0, dtype=F64))
    seen = []
    plain.attention(x, far_below, m, 1e-5, "attention", weights_out=seen)
    assert all(abs(float(weights.sum()) - 1) < 1e-12 for _, _, _, weights in seen)
    assert plain.attention(x, far_above, m, 1e-5, "attention").abs().max() < 1e-20
    only_first = dict(w, sink=torch.tensor([80.0, -80.0], dtype=F64))              # a sink per head: the second head is untouched
    o = dict(w, o=torch.eye(12, dtype=F64))
    both = plain.attention(x, dict(o, sink=far_below["sink"]), m, 1e-5, "attention")
    one = plain.attention(x, dict(o, sink=only_first["sink"]), m, 1e-5, "attention")
    assert one[:, :6].abs().max() < 1e-20 and torch.allclose(one[:, 6:], both[:, 6:])


def test_heads_are_unit_after_the_rotation_so_their_length_does_not_matter():
    m = {"heads": 2, "kv_heads": 2, "dim": 8, "vdim": 8, "scale": 0.4, "softcap": 3.0, "rot": {"base": 30.0, "dims": 4, "scaling": {"factor": 2.0}}}
    w = attention_weights("attention_2", m)
    x = values(9, 24, seed=4)
    base = plain.attention(x, w, m, 1e-9, "attention_2")
    assert torch.allclose(plain.attention(x, dict(w, q=7.0 * w["q"], k=0.2 * w["k"]), m, 1e-9, "attention_2"), base, atol=1e-6)
    # the cap bounds what a score can say: with a tiny cap every visible key weighs the same, and the output is the running mean
    flat = plain.attention(x, dict(w, o=torch.eye(16, dtype=F64), g=torch.zeros(2, 24, dtype=F64)), dict(m, softcap=1e-9), 1e-9, "attention_2")
    v = (x @ w["v"].T)
    mean = torch.cumsum(v, 0) / torch.arange(1, 10, dtype=F64)[:, None]
    assert torch.allclose(flat, 0.5 * mean, atol=1e-6)                             # sigmoid(0) = 1/2: the gate of a head, one number


def test_the_gate_is_one_number_a_head():
    m = {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 4, "scale": 0.4}
    w = attention_weights("attention_2", m)
    w["o"] = torch.eye(8, dtype=F64)
    x = values(6, 24, seed=5)
    open_gate = plain.attention(x, dict(w, g=torch.zeros(2, 24, dtype=F64)), m, 1e-6, "attention_2") * 2.0
    gated = plain.attention(x, w, m, 1e-6, "attention_2")
    factor = plain.logistic(x @ w["g"].T)
    assert torch.allclose(gated[:, :4], open_gate[:, :4] * factor[:, :1]) and torch.allclose(gated[:, 4:], open_gate[:, 4:] * factor[:, 1:])


def test_experts_run_on_their_score_times_the_token():
    mlp = configs.experts(6, 0.9, 4, 2, shared=(4, 0.5))
    w = {"router": values(4, 10, seed=1)}
    for e in range(4):
        w.update({f"e{e}.gate": values(6, 10, seed=10 + e), f"e{e}.up": values(6, 10, seed=20 + e), f"e{e}.down": values(10, 6, seed=30 + e)})
    w.update({"shared.gate": values(4, 10, seed=40), "shared.up": values(4, 10, seed=41), "shared.down": values(10, 4, seed=42)})
    x = values(7, 10, seed=2)
    out = plain.routed_ff(x, w, mlp)
    indices, scores = plain.choose(x @ w["router"].T, 2)
    assert (scores > 0).all() and (scores < 1).all() and float(scores.sum(-1).max()) != 1.0          # sigmoid scores, not renormalised
    by_hand = torch.zeros_like(x)
    weighted_after = torch.zeros_like(x)
    for i in range(7):
        for e, s in zip(indices[i].tolist(), scores[i]):
            by_hand[i] += plain.expert(s * x[i], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], 0.9)
            weighted_after[i] += s * plain.expert(x[i], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], 0.9)
    shared = plain.expert(x, w["shared.gate"], w["shared.up"], w["shared.down"], 0.5)
    assert torch.allclose(out, by_hand + shared)
    assert not torch.allclose(out, weighted_after + shared, atol=1e-3)                               # the place of the weight matters
    # the clamps: beyond the limit the gate stops growing and the up value is held on both sides
    one = {"gate": torch.ones(1, 1, dtype=F64), "up": torch.ones(1, 1, dtype=F64), "down": torch.ones(1, 1, dtype=F64)}
    big, small = torch.tensor([[50.0]], dtype=F64), torch.tensor([[-50.0]], dtype=F64)
    assert torch.allclose(plain.expert(big, one["gate"], one["up"], one["down"], 2.0), torch.tensor([[2.0 * float(plain.logistic(torch.tensor(3.404))) * 3.0]], dtype=F64))
    assert torch.allclose(plain.expert(small, one["gate"], one["up"], one["down"], 2.0),
                          torch.tensor([[-50.0 * float(plain.logistic(torch.tensor(-50.0 * 1.702))) * (-2.0 + 1.0)]], dtype=F64))


def test_layers_that_share_weights_against_the_same_layers_written_out(tmp_path):
    raw = configs.ONES
    g = torch.Generator().manual_seed(5)
    from llm_runtime_study_amd.config import config_from_dict, spec_for
    from llm_runtime_study_amd.models import DecoderModel

    names = DecoderModel(spec_for(config_from_dict(raw))).tensors()
    weights = {name: torch.randn(spec.shape, generator=g, dtype=F64) / math.sqrt(spec.shape[-1]) for name, spec in names.items()}
    written = copy.deepcopy(raw)
    for index, layer in enumerate(written["layers"]):
        owner = layer.pop("weights_of", None)
        if owner is not None:
            weights.update({f"l{index}." + name[len(f"l{owner}."):]: t for name, t in list(weights.items()) if name.startswith(f"l{owner}.")})
    ids = [3, 80, 11, 11, 42, 7, 0, 65]
    streams = []
    assert torch.allclose(plain.forward(weights, raw, ids, streams), plain.forward(weights, written, ids))
    assert len(streams) == len(raw["layers"])


def test_first_tokens_and_embedding():
    raw = configs.ODD
    from llm_runtime_study_amd.config import config_from_dict, spec_for
    from llm_runtime_study_amd.models import DecoderModel

    g = torch.Generator().manual_seed(6)
    names = DecoderModel(spec_for(config_from_dict(raw))).tensors()
    weights = {name: torch.randn(spec.shape, generator=g, dtype=F64) / math.sqrt(spec.shape[-1]) for name, spec in names.items()}
    one = plain.forward(weights, raw, [17])
    two = plain.forward(weights, raw, [17, 17])
    assert torch.allclose(one[0], two[0])                                # causal: the first row does not see the second token
    assert not torch.allclose(two[0], two[1], atol=1e-3)                 # the same token at another position: the learned vector, the rotation
    moved = dict(weights, pos=torch.zeros_like(weights["pos"]))
    assert not torch.allclose(plain.forward(moved, raw, [17])[0], one[0], atol=1e-3)
