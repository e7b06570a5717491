"""Felosun on the GPU against the plain implementation (tests/plain/felosun.py): each mechanism alone (requests of unequal
length stepped side by side, pages given back and used again), then whole models of the tests' own sizes under every way of
cutting their requests into steps, keys planted on either side of a window's edge and of the kept first positions, a key far
back among hundreds, sinks that outweigh every key, long decoding, and greedy generation through Engine and scheduler."""

import math

import numpy as np
import pytest
import torch

from tests import felosun_configs as configs
from tests import traces
from tests.plain import felosun as plain
from tests.test_parts_gpu import PartHarness, close
from tests.test_replay_gpu import round64, run_replay

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
F64 = torch.float64


def bf16_values(*shape, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(*shape, generator=g)).to(torch.bfloat16).double()


def short(name: str) -> str:
    """A part's name of a tensor as the plain functions (and a checkpoint) spell it."""
    name = name.removesuffix(".weight").replace("_proj", "")
    name = name.replace("experts.", "e")
    return name[:-len(".bias")] + ".b" if name.endswith(".bias") else name


def part_weights(part, seed):
    out = {}
    for number, (name, spec) in enumerate(part.tensors().items()):
        if spec.role == "bias":
            out[name] = bf16_values(*spec.shape, scale=0.5, seed=seed + number)
        else:
            out[name] = bf16_values(*spec.shape, scale=1.0 / math.sqrt(spec.shape[-1]), seed=seed + number)
    return out


def bound(part, w, dtype):
    part.bind({name: t.to(torch.bfloat16).cuda() for name, t in w.items()}, dtype)
    return {short(name): t for name, t in w.items()}


SCHEDULE = [[("a", 15), ("b", 1)], [("a", 1), ("b", 17)], [("b", 16), ("a", 2)], [("a", 33)], [("a", 1), ("b", 1)], [("b", 5), ("a", 18)],
            [("c", 3)], [("c", 16)], [("c", 1), ("a", 1)], [("a", 1), ("c", 2)]]
LENGTHS = {"a": 72, "b": 40, "c": 22}


def step_through(part, dtype, inputs, width, schedule=SCHEDULE, release_before=(6, "b"), page_size=16):
    """The rows a mixer gives for `inputs` {key: [n, width]} when their tokens arrive as `schedule` says: portions beside
    single tokens, portions that end inside, at and just past pages; before step `release_before[0]` the request
    release_before[1] ends and the next admitted takes its slot and pages."""
    harness = PartHarness([part.cache_need()], dtype, page_size=page_size)
    live, at, got = {}, {key: 0 for key in inputs}, {key: [] for key in inputs}
    for number, step in enumerate(schedule):
        if release_before is not None and number == release_before[0]:
            harness.cache.release(live.pop(release_before[1]))
        entries = []
        for key, n in step:
            if key not in live:
                live[key] = harness.cache.admit(key)
            entries.append((live[key], [0] * n))
        ctx = harness.context(entries)
        x = torch.cat([inputs[key][at[key]:at[key] + n] for key, n in step]).to(dtype).cuda()
        out = torch.full((x.shape[0], width), 0.5, dtype=torch.float32, device="cuda")
        part.forward(ctx, x, out, ctx.layer_cache(0), accumulate=number % 2 == 0)
        torch.cuda.synchronize()
        row = 0
        for key, n in step:
            got[key].append(out[row:row + n].cpu().double() - (0.5 if number % 2 == 0 else 0.0))
            row, at[key] = row + n, at[key] + n
            harness.cache.trim(live[key])
    return {key: torch.cat(rows) for key, rows in got.items()}, live


# ------------------------------------------------------------------------------------- mechanisms alone
WINDOWED_SHAPES = [
    # heads, kv, d, e, scale, rot (base, dims), window, kept
    (4, 2, 16, 24, 0.3, (500.0, 8), None, 0),        # values wider than keys, half a head rotated, the whole context
    (6, 2, 32, 16, 0.2, None, 9, 3),                 # a window shorter than a page, three kept, no rotation
    (2, 1, 64, 64, 0.125, (1e4, 64), None, 0),       # the matrix cores' shape, whole heads rotated
    (4, 4, 64, 64, 0.125, (30.0, 16), 20, 0),        # ... behind a window that keeps nothing
    (2, 2, 128, 128, 0.09, (1e5, 32), 21, 18),       # kept positions that reach into the second page
    (1, 1, 8, 8, 0.35, (100.0, 2), 1, 0),            # a window of one, one pair rotated
    (3, 1, 48, 40, 0.15, (1e6, 48), 30, 30),         # as many kept as the window holds
    (16, 1, 32, 32, 0.2, (77.0, 32), 24, 5),         # sixteen heads on one key group
    (3, 3, 20, 20, 0.25, (9.0, 6), 40, 1),           # a head size that is no multiple of eight
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,groups,d,e,scale,rot,window,kept", WINDOWED_SHAPES)
def test_windowed_attention_with_sink_part(dtype, heads, groups, d, e, scale, rot, window, kept):
    from llm_runtime_study_amd.parts import PartSpec, create

    width = 56
    position = PartSpec("none") if rot is None else PartSpec("rope_interleaved", {"rotary_dim": rot[1], "theta": rot[0]})
    part = create("mixer", PartSpec("gqa_attention", {"hidden_size": width, "num_heads": heads, "num_kv_heads": groups, "head_dim": d, "value_dim": e,
                                                     "position": position, "unit_norm_after_rotation": True, "qk_norm_eps": 1e-3, "scale": scale,
                                                     "bias": True, "window": window, "keep_first": kept, "sink": True}))
    w = part_weights(part, 50)
    w["sink"] = (w["sink"] * 3.0 + 1.0).to(torch.bfloat16).double()          # sinks that weigh as much as a handful of keys
    named = bound(part, w, dtype)
    assert named["sink"].shape == (heads,) and named["q.b"].shape == (heads * d,) and "g" not in named
    m = {"heads": heads, "kv_heads": groups, "dim": d, "vdim": e, "scale": scale}
    if rot is not None:
        m["rot"] = {"base": rot[0], "dims": rot[1]}
    if window is not None:
        m["mask"] = {"size": window, "keep_first": kept}
    inputs = {key: bf16_values(n, width, seed=300 + i) for i, (key, n) in enumerate(LENGTHS.items())}
    want = {key: plain.attention(x, named, m, 1e-3, "attention") for key, x in inputs.items()}
    for page_size in (16, 4):
        got, live = step_through(part, dtype, inputs, width, page_size=page_size)
        for key in inputs:
            close(got[key], want[key][:got[key].shape[0]], dtype, f32=5e-5, bf16=2e-2)
    if window is not None and window < 40:
        first_kept_pages = -(-kept // 4)
        assert live["a"].first_live[0] > first_kept_pages         # pages between the kept positions and the window went back
        assert all(page >= 0 for page in live["a"].tables[0][:first_kept_pages])


CAPPED_SHAPES = [
    # heads, kv, d, e, scale, rot (base, dims, factor), cap
    (4, 2, 16, 24, 0.3, (500.0, 8, 4.0), 2.0),        # values wider than keys, half a head rotated and stretched, a cap that bites
    (6, 2, 32, 32, 0.2, None, 30.0),                  # no rotation, a cap far above the scores
    (2, 1, 64, 64, 0.125, (1e4, 64, 1.0), 4.0),       # the matrix cores' shape
    (4, 4, 96, 96, 0.1, (2e4, 24, 4.0), 5.0),         # heads of 96, a quarter rotated (a rotated half that is no multiple of eight)
    (2, 2, 128, 128, 0.09, (1e5, 64, 2.0), 3.0),      # heads of 128: capped scores go through the kernel for any head size
    (1, 1, 8, 8, 0.35, (100.0, 2, 8.0), None),        # one head, one pair, no cap at all
    (5, 1, 24, 12, 0.25, (9.0, 24, 1.5), 1.0),        # five heads on one key group, values narrower than keys
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,groups,d,e,scale,rot,cap", CAPPED_SHAPES)
def test_capped_attention_with_head_gates_part(dtype, heads, groups, d, e, scale, rot, cap):
    from llm_runtime_study_amd.parts import PartSpec, create

    width = 56
    position = PartSpec("none") if rot is None else PartSpec("rope_half", {"rotary_dim": rot[1], "theta": rot[0], "factor": rot[2]})
    part = create("mixer", PartSpec("gqa_attention", {"hidden_size": width, "num_heads": heads, "num_kv_heads": groups, "head_dim": d, "value_dim": e,
                                                     "position": position, "unit_norm_after_rotation": True, "qk_norm_eps": 1e-3, "scale": scale,
                                                     "score_cap": cap, "output_gate": "head"}))
    w = part_weights(part, 80)
    w["g_proj.weight"] = (w["g_proj.weight"] * 4.0).to(torch.bfloat16).double()      # gates well away from one half
    named = bound(part, w, dtype)
    assert named["g"].shape == (heads, width) and "sink" not in named and "q.b" not in named
    m = {"heads": heads, "kv_heads": groups, "dim": d, "vdim": e, "scale": scale}
    if rot is not None:
        m["rot"] = {"base": rot[0], "dims": rot[1], "scaling": {"factor": rot[2]}}
    if cap is not None:
        m["softcap"] = cap
    inputs = {key: bf16_values(n, width, seed=400 + i) for i, (key, n) in enumerate(LENGTHS.items())}
    want = {key: plain.attention(x, named, m, 1e-3, "attention_2") for key, x in inputs.items()}
    for page_size in (16, 4):
        got, _ = step_through(part, dtype, inputs, width, page_size=page_size)
        for key in inputs:
            close(got[key], want[key][:got[key].shape[0]], dtype, f32=5e-5, bf16=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,groups,d,e", [(4, 2, 64, 64), (2, 1, 128, 128), (3, 1, 24, 40)])
def test_every_constant_on_either_kind_part(dtype, heads, groups, d, e):
    """A window with kept positions, a cap and stretched positions are parameters of one mixer: the kind with sinks and biases
    under a cap and stretched positions, the kind with head gates behind a window with kept positions (the gate then meets the
    kept positions' share in the merge of partial results)."""
    from llm_runtime_study_amd.parts import PartSpec, create

    width = 56
    sizes = {"hidden_size": width, "num_heads": heads, "num_kv_heads": groups, "head_dim": d, "value_dim": e, "unit_norm_after_rotation": True,
             "qk_norm_eps": 1e-4, "scale": 0.15, "window": 19, "keep_first": 4, "score_cap": 1.5}
    m = {"heads": heads, "kv_heads": groups, "dim": d, "vdim": e, "scale": 0.15, "mask": {"size": 19, "keep_first": 4}, "softcap": 1.5,
         "rot": {"base": 300.0, "dims": 8, "scaling": {"factor": 3.0}}}
    inputs = {key: bf16_values(n, width, seed=500 + i) for i, (key, n) in enumerate(LENGTHS.items())}
    for kind in ("attention", "attention_2"):
        first = kind == "attention"
        position = PartSpec("rope_interleaved" if first else "rope_half", {"rotary_dim": 8, "theta": 300.0, "factor": 3.0})
        part = create("mixer", PartSpec("gqa_attention", dict(sizes, position=position, bias=first, sink=first, output_gate=False if first else "head")))
        w = part_weights(part, 90)
        if not first:
            w["g_proj.weight"] = (w["g_proj.weight"] * 4.0).to(torch.bfloat16).double()
        named = bound(part, w, dtype)
        want = {key: plain.attention(x, named, m, 1e-4, kind) for key, x in inputs.items()}
        for page_size in (16, 4):
            got, _ = step_through(part, dtype, inputs, width, page_size=page_size)
            for key in inputs:
                close(got[key], want[key][:got[key].shape[0]], dtype, f32=5e-5, bf16=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("splits", ["few keys", "many keys"])
def test_a_sink_that_outweighs_every_key_and_one_that_weighs_nothing(dtype, splits):
    """Heads of the matrix cores' shape: the first head's sink towers over every score (its output is nothing), the second's
    lies far below them (its output is the plain softmax), in a prompt's portion, in single tokens, with the keys whole and
    divided between workgroups."""
    from llm_runtime_study_amd.parts import PartSpec, create

    width, heads, d = 128, 2, 64
    length = 40 if splits == "few keys" else 700
    part = create("mixer", PartSpec("gqa_attention", {"hidden_size": width, "num_heads": heads, "num_kv_heads": 1, "head_dim": d,
                                                     "unit_norm_after_rotation": True, "qk_norm_eps": 1e-5, "scale": 0.05, "bias": True, "sink": True}))
    w = part_weights(part, 7)
    w["sink"] = torch.tensor([60.0, -60.0], dtype=F64)
    w["o_proj.weight"] = torch.eye(width, heads * d, dtype=F64)
    named = bound(part, w, dtype)
    m = {"heads": heads, "kv_heads": 1, "dim": d, "vdim": d, "scale": 0.05}
    x = bf16_values(length, width, seed=11)
    want = plain.attention(x, named, m, 1e-5, "attention")
    assert want[:, :d].abs().max() < 1e-12 and want[:, d:].abs().mean() > 1e-2
    schedule = [[("a", length - 3)], [("a", 1)], [("a", 2)]]
    got, _ = step_through(part, dtype, {"a": x}, width, schedule=schedule, release_before=None) if length <= 256 else (None, None)
    if got is None:
        harness = PartHarness([part.cache_need()], dtype, max_step_tokens=1024)
        request = harness.cache.admit("a")
        rows, at = [], 0
        for n in (length - 3, 1, 2):
            ctx = harness.context([(request, [0] * n)])
            out = torch.zeros(n, width, dtype=torch.float32, device="cuda")
            part.forward(ctx, x[at:at + n].to(dtype).cuda(), out, ctx.layer_cache(0), accumulate=False)
            rows.append(out.cpu().double())
            at += n
        got = {"a": torch.cat(rows)}
    assert got["a"][:, :d].abs().max() < 1e-6
    close(got["a"][:, d:], want[:, d:], dtype, f32=5e-5, bf16=2e-2)


ROUTED_SHAPES = [
    # width, ff, experts, top, limit, shared (ff, limit), tokens
    (64, 32, 8, 2, 1.0, (48, 1.0), 19),
    (64, 32, 8, 2, 1.0, None, 1),                   # a single token
    (72, 15, 7, 3, 0.8, (18, 2.0), 37),             # an odd expert size, a width that is no multiple of 64
    (128, 64, 70, 3, 1.5, (96, 0.6), 50),           # more experts than a wave has lanes
    (64, 16, 1, 1, 0.5, None, 9),                   # one expert
    (64, 24, 4, 4, 3.0, (8, 0.3), 300),             # every expert chosen, enough rows for the large tiles
    (256, 128, 4, 2, 1.0, (128, 1.0), 400),         # the grouped product that fetches whole slices
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,ff,count,top,limit,shared,tokens", ROUTED_SHAPES)
def test_experts_on_weighted_inputs_with_a_shared_expert_part(dtype, width, ff, count, top, limit, shared, tokens):
    from llm_runtime_study_amd.parts import PartSpec, create

    shared_spec = None if shared is None else PartSpec("swiglu", {"hidden_size": width, "intermediate_size": shared[0], "activation": "clamped",
                                                                  "alpha": 1.702, "limit": shared[1]})
    part = create("feed_forward", PartSpec("routed_experts", {
        "hidden_size": width, "intermediate_size": ff, "num_experts": count, "top": top, "rule": "sigmoid_scores", "activation": "clamped_gated",
        "activation_alpha": 1.702, "activation_limit": limit, "weight_on": "input", "shared": shared_spec}))
    w = part_weights(part, 20)
    for name in w:                                   # projections large enough that the clamps bite for a good share of the features
        if name.endswith("gate.weight") or name.endswith("up.weight") or name.endswith("gate_proj.weight") or name.endswith("up_proj.weight"):
            w[name] = (w[name] * 1.5).to(torch.bfloat16).double()
    named = bound(part, w, dtype)
    mlp = configs.experts(ff, limit, count, top, shared)
    x = bf16_values(tokens, width, seed=31)
    margins = []
    want = plain.routed_ff(x, named, mlp, margins)
    harness = PartHarness([], dtype, max_step_tokens=512)
    ctx = harness.context([(harness.cache.admit("a"), [0] * tokens)])
    residual = torch.full((tokens, width), 0.25, dtype=torch.float32, device="cuda")
    part.forward(ctx, x.to(dtype).cuda(), residual)
    torch.cuda.synchronize()
    got = residual.cpu().double() - 0.25
    if dtype == torch.float32:
        close(got, want, dtype, f32=1e-4)
    else:
        # rows whose choice is not a close call (the router's product is bfloat16 x bfloat16 into float32 either way)
        sure = torch.tensor([m > 1e-3 for m in margins]) if margins else torch.ones(tokens, dtype=torch.bool)
        close(got[sure], want[sure], dtype, bf16=2e-2)
    # the norm of a layer that normalises outputs, applied by the kernel that adds the sums up
    from llm_runtime_study_amd.parts import PartSpec as Spec

    norm = create("norm", Spec("rmsnorm", {"size": width, "eps": 1e-5}))
    norm_weight = (1.0 + bf16_values(width, scale=0.1, seed=5)).to(torch.bfloat16).double()
    norm.bind({"weight": norm_weight.to(torch.bfloat16).cuda()}, dtype)
    residual.fill_(0.25)
    part.forward(ctx, x.to(dtype).cuda(), residual, output_norm=norm)
    torch.cuda.synchronize()
    normed = plain.unit_rms(want, 1e-5) * norm_weight
    got = residual.cpu().double() - 0.25
    if dtype == torch.float32:
        close(got, normed, dtype, f32=2e-4)


def test_small_kernels_of_the_design():
    from llm_runtime_study_amd.kernels import ops

    g = torch.Generator().manual_seed(3)
    # a learned vector per position, added to the stream
    table = torch.randn(50, 40, generator=g).to(torch.bfloat16)
    ids = torch.tensor([49, 0, 7, 7, 13], dtype=torch.int32)
    h = torch.randn(5, 40, generator=g)
    for t in (table, table.float()):
        out = h.clone().cuda()
        ops.add_gathered(out, t.cuda(), ids.cuda())
        torch.testing.assert_close(out.cpu(), h + table.float()[ids.long()])
    # a factor on the logits
    x = torch.randn(7, 33, generator=g)
    out = x.clone().cuda()
    ops.scale_values(out, 0.3)
    torch.testing.assert_close(out.cpu(), x * 0.3)
    # the clamped gated activation, values on both sides of the limits
    gu = (3.0 * torch.randn(9, 2 * 14, generator=g))
    gate, up = gu[:, :14].double(), gu[:, 14:].double()
    gt = torch.clamp(gate, max=1.3)
    want = gt * plain.logistic(1.702 * gt) * (torch.clamp(up, -1.3, 1.3) + 1.0)
    for dtype in DTYPES:
        src = gu.to(dtype)
        out = torch.empty(9, 14, dtype=dtype, device="cuda")
        ops.gated_clamped(out, src.cuda(), 1.702, 1.3)
        gate, up = src[:, :14].double(), src[:, 14:].double()
        gt = torch.clamp(gate, max=1.3)
        want = gt * plain.logistic(1.702 * gt) * (torch.clamp(up, -1.3, 1.3) + 1.0)
        close(out, want, dtype, f32=1e-5, bf16=1e-2)
    # one gate value a head
    out = torch.randn(6, 3 * 10, generator=g)
    gates = torch.randn(6, 3, generator=g)
    got = out.clone().cuda()
    ops.sigmoid_gate(got, gates.cuda())
    torch.testing.assert_close(got.cpu(), out * torch.sigmoid(gates).repeat_interleave(10, 1))


# ------------------------------------------------------------------------------------- whole models
RAW = {"odd": configs.ODD, "cores": configs.CORES, "ones": configs.ONES, "awkward": configs.AWKWARD}
MODEL_LENGTHS = {"odd": [70, 33, 9, 1, 52, 17, 66], "cores": [150, 64, 2, 97, 33], "ones": [40, 1, 65, 16, 5], "awkward": [90, 31, 3, 48, 17]}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for number, (name, raw) in enumerate(RAW.items()):
        folder = configs.write_folder(raw, 160 + number, tmp_path_factory.mktemp(f"felosun_{name}"))
        tensors, _ = plain.load_model_dir(folder)
        rng = np.random.default_rng(121 + number)
        requests = {f"{name}{i}": rng.integers(0, raw["vocab"], n).tolist() for i, n in enumerate(MODEL_LENGTHS[name])}
        want, margins = {}, []
        for key, tokens in requests.items():
            want[key] = plain.forward(tensors, raw, tokens, margins=margins)
        out[name] = (folder, raw, requests, want)
    return out


def check(got, want, dtype):
    """float32: every row within 1e-4 of the plain row as a whole (relative L2; a row whose expert choice is a close call may
    differ, so one row in fifty may be off) and no logit of the others further off than 3e-4 of the row's largest.  bfloat16:
    these models are a few dozen values wide and choose experts, which is a discrete choice that a rounding can turn (and the
    token's row, and those that attend to it, with it): 80 rows in 100 within 3 % as a whole, and none off by more than its
    own length."""
    errors = np.array([float((row.double() - want[key][position]).norm() / want[key][position].norm())
                       for key, rows in got.items() for position, row in rows.items()])
    if dtype == "float32":
        assert np.mean(errors < 1e-4) >= 0.98, f"{np.mean(errors < 1e-4):.3f} of the rows are close, the worst is off by {errors.max():.3g}"
        return len(errors)
    assert np.mean(errors < 3e-2) >= 0.8 and errors.max() < 1.0, f"{np.mean(errors < 3e-2):.2f} of the rows are close, the worst is off by {errors.max():.3g}"
    return len(errors)


def test_the_stream_after_every_layer_run(models):
    """One step function call on a whole prompt in float32, the stream read after every run of a layer (a layer that shares
    weights counts each time) against the plain implementation's."""
    from llm_runtime_study_amd.engine import trace
    from llm_runtime_study_amd.engine.step import StepEntry

    for name in ("odd", "ones"):
        folder, raw, requests, _ = models[name]
        tokens = requests[f"{name}2"]
        tensors, _ = plain.load_model_dir(folder)
        streams = []
        plain.forward(tensors, raw, tokens, streams)
        runner = trace.make_runner(folder, "float32", 128, 16)
        seen = []
        for layer in runner.model.layers:
            inner = layer.forward

            def watched(ctx, h, *args, _inner=inner, **kwargs):
                result = _inner(ctx, h, *args, **kwargs)
                seen.append(h.detach().clone())
                return result

            layer.forward = watched
        runner.step([StepEntry(runner.cache.admit("r"), tokens, [len(tokens) - 1])])
        torch.cuda.synchronize()
        assert len(seen) == len(streams) == len(raw["layers"])
        for mine, theirs in zip(seen, streams):
            torch.testing.assert_close(mine[:len(tokens)].cpu().double(), theirs, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(RAW))
def test_whole_then_last_tokens_one_by_one_then_portions(models, name, dtype, tmp_path):
    folder, raw, requests, want = models[name]
    longest = max(round64(len(t)) for t in requests.values())
    steps = traces.whole(requests)
    got = traces.collect(steps, run_replay(folder, dtype, steps, longest, tmp_path / "whole"), raw["vocab"])
    assert check(got, want, dtype) == sum(len(t) for t in requests.values())
    steps = traces.prefill_then_decode(requests, tail=50)        # longer than the windows: they pass over decoded tokens
    check(traces.collect(steps, run_replay(folder, dtype, steps, longest, tmp_path / "tail"), raw["vocab"]), want, dtype)
    steps = traces.portions(requests)
    check(traces.collect(steps, run_replay(folder, dtype, steps, longest, tmp_path / "portions", page_size=32), raw["vocab"]), want, dtype)
    few = {key: tokens for key, tokens in requests.items() if len(tokens) < 70}
    steps = traces.portions(few, sizes=(2, 2, 3, 2))
    check(traces.collect(steps, run_replay(folder, dtype, steps, longest, tmp_path / "twos"), raw["vocab"]), want, dtype)


def test_cuts_batch_mates_and_pages_change_no_bit_in_float32(models, tmp_path):
    """float32 sums depend on the position alone: the same rows under every cutting, to the bit."""
    folder, raw, requests, _ = models["odd"]
    longest = max(round64(len(t)) for t in requests.values())
    steps = traces.whole(requests)
    whole = traces.collect(steps, run_replay(folder, "float32", steps, longest, tmp_path / "whole"), raw["vocab"])
    steps, peak = traces.mixed(requests, seed=8, max_live=4, max_tokens=2 * longest)
    mixed = traces.collect(steps, run_replay(folder, "float32", steps, peak, tmp_path / "mixed", page_size=32), raw["vocab"])
    steps = traces.portions(requests, sizes=(3, 2, 19, 2))
    cut = traces.collect(steps, run_replay(folder, "float32", steps, longest, tmp_path / "cut"), raw["vocab"])
    compared = 0
    for key, rows in mixed.items():
        for position, row in rows.items():
            assert torch.equal(row, whole[key][position]) and torch.equal(cut[key][position], row), (key, position)
            compared += 1
    assert compared > 40


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,seed", [("odd", 0), ("odd", 1), ("cores", 2), ("ones", 3), ("awkward", 6)])
def test_mixed_steps_with_pages_and_slots_used_again(models, name, seed, dtype, tmp_path):
    folder, raw, requests, want = models[name]
    budget = 2 * max(round64(len(t)) for t in requests.values())
    steps, peak = traces.mixed(requests, seed=seed, max_live=4, max_tokens=budget)
    assert max(len(s["entries"]) for s in steps) >= 3
    got = traces.collect(steps, run_replay(folder, dtype, steps, peak, tmp_path), raw["vocab"])
    assert check(got, want, dtype) > 30
    assert peak < sum(round64(len(t)) for t in requests.values())


@pytest.mark.parametrize("name", ["odd", "cores"])
def test_the_engines_path_of_graphs_and_recorded_steps(models, name, tmp_path):
    """On a stream of the runner's own with graphs on: single-token steps are graph replays, shapes that come back are
    launched from their recorded plan."""
    folder, raw, requests, want = models[name]
    longest = max(round64(len(t)) for t in requests.values())
    seen = {}
    steps = traces.prefill_then_decode(requests, tail=40)
    out = run_replay(folder, "float32", steps, longest, tmp_path / "tail", as_the_engine=True, counters=seen)
    check(traces.collect(steps, out, raw["vocab"]), want, "float32")
    assert seen["graph_replays"] >= 20 * (len(requests) - 2)
    steps, peak = traces.mixed(requests, seed=5, max_live=4, max_tokens=2 * longest)
    out = run_replay(folder, "bfloat16", steps, peak, tmp_path / "mixed", as_the_engine=True, counters=seen)
    check(traces.collect(steps, out, raw["vocab"]), want, "bfloat16")
    steps = traces.portions(requests, sizes=(16, 16, 16, 2))
    out = run_replay(folder, "float32", steps, longest, tmp_path / "portions", as_the_engine=True, counters=seen)
    check(traces.collect(steps, out, raw["vocab"]), want, "float32")
    assert seen["plan_replays"] >= 10


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_wider_model_through_the_products_for_many_rows(tmp_path, dtype):
    """Width 512 and prompts of 330 and 140 tokens: the projections of a prompt are products of hundreds of rows (the vendor
    library's in bfloat16), the experts get enough rows for the large tiles, the window of 150 lies inside the longer prompt."""
    raw = configs.WIDE
    folder = configs.write_folder(raw, 21, tmp_path / "wide")
    tensors, _ = plain.load_model_dir(folder)
    rng = np.random.default_rng(4)
    requests = {"long": rng.integers(0, raw["vocab"], 330).tolist(), "short": rng.integers(0, raw["vocab"], 140).tolist()}
    want = {key: plain.forward(tensors, raw, tokens) for key, tokens in requests.items()}
    steps = [{"step": 0, "entries": [{"id": key, "tokens": tokens[:-6], "want": list(range(0, len(tokens) - 6, 7))} for key, tokens in requests.items()], "end": []}]
    for i in range(6, 0, -1):
        steps.append({"step": len(steps), "entries": [{"id": key, "tokens": [tokens[-i]], "want": [0]} for key, tokens in requests.items()],
                      "end": list(requests) if i == 1 else []})
    got = traces.collect(steps, run_replay(folder, dtype, steps, 512, tmp_path / "o"), raw["vocab"])
    assert check(got, want, dtype) > 70


def test_bfloat16_path_follows_float32_at_real_layer_sizes():
    """Two layers at the sizes of a real model's (width 1,024, 16 heads of 128 on 8 key groups, a window of 512 with 8 kept
    positions, 2 of 8 experts of 384 and a shared one, a vocabulary of 8,000): the bfloat16 path with everything it uses at that
    size (graphs, the vendor's products for many rows, the grouped products' large tiles, key splits, the prefill kernel for
    heads of 128 with capped scores, values stored as runs) against the float32 path of the same weights, over prompts in two
    portions beside decoding requests and decode steps.  Experts are a discrete choice, so a share of the rows may differ."""
    from llm_runtime_study_amd.benchmarks.shapes import SHAPES, felosun_like
    from llm_runtime_study_amd.cache import CacheManager
    from llm_runtime_study_amd.config import config_from_dict, spec_for
    from llm_runtime_study_amd.engine.step import ModelRunner, StepEntry
    from llm_runtime_study_amd.models import DecoderModel
    from llm_runtime_study_amd.weights import random_init

    raw = felosun_like(dict(SHAPES["0.6b"], vocab_size=8000), 2, experts=8, top=2, window=512, positions=2048)
    cfg = config_from_dict(raw)
    device = torch.device("cuda", 0)
    weights = random_init.device_weights(DecoderModel(spec_for(cfg)), 0, torch.bfloat16, device, "scaled")
    rng = np.random.default_rng(1)
    prompts = [rng.integers(0, cfg.vocab_size, n).tolist() for n in (700, 33, 1500, 257, 64, 5, 1023, 90)]
    tails = [rng.integers(0, cfg.vocab_size, 14).tolist() for _ in prompts]
    logits_of = {}
    for dtype in (torch.float32, torch.bfloat16):
        model = DecoderModel(spec_for(cfg))
        model.bind(weights, dtype)
        cache = CacheManager(model.cache_needs(), page_size=16, num_pages=400, max_requests=8, max_seq_len=2048, dtype=dtype, device=device)
        runner = ModelRunner(model, cache, max_step_tokens=2048, dtype=dtype, device=device, use_graph=dtype == torch.bfloat16)
        rows = []
        with torch.cuda.stream(torch.cuda.Stream(device)):
            caches = [cache.admit(i) for i in range(len(prompts))]
            fed = {}
            for i, prompt in enumerate(prompts):
                # the first half of the prompt beside one token of every earlier request, then the rest alone
                half = len(prompt) // 2
                decoding = [StepEntry(caches[j], [tails[j][fed[j]]], [0]) for j in sorted(fed)]
                for j in fed:
                    fed[j] += 1
                mixed = runner.step(decoding + [StepEntry(caches[i], prompt[:half], [half - 1])])
                rows.append(mixed.float().cpu())
                rows.append(runner.step([StepEntry(caches[i], prompt[half:], [0, len(prompt) - half - 1])]).float().cpu())
                fed[i] = 0
            for _ in range(6):
                rows.append(runner.step([StepEntry(caches[j], [tails[j][fed[j]]], [0]) for j in sorted(fed)]).float().cpu())
                for j in fed:
                    fed[j] += 1
            if dtype == torch.bfloat16:
                assert runner.graph_replays >= 3
                runner.drop_graphs()
        logits_of[dtype] = torch.cat(rows)
        cache.check_invariants()
        del runner, cache, model
    exact, fast = logits_of[torch.float32], logits_of[torch.bfloat16]
    assert exact.shape == fast.shape and exact.shape[0] > 80
    error = (exact - fast).norm(dim=1) / exact.norm(dim=1)
    assert (error < 3e-2).float().mean() >= 0.9 and error.median() < 1.5e-2, f"median {error.median():.3g}, {(error < 3e-2).float().mean():.2f} of the rows close"


# ------------------------------------------------------------------------------------- planted inputs
WINDOW, KEPT = 21, 3


def planted_model(tmp_path, layer):
    """A model of one layer whose attention's query matrix is its key matrix behind a swap of the two halves of the stream:
    the query of token B is the key of token A when A's embedding is B's with its halves swapped (no biases, no learned
    positions).  Both are unit vectors of the same direction then, so the match scores dim * scale, which towers over every
    other score: a B sees an A, and adds A's value to the stream, exactly when A is visible from B.  Token 0 is A, token 1 B."""
    raw = configs.model(50, 32, 1e-6, 704, 1.0, 1.0, [layer])

    def edit(tensors):
        k = tensors["l0.mix.k"]
        tensors["l0.mix.q"] = torch.cat((k[:, 16:], k[:, :16]), 1).contiguous()
        for name in ("l0.mix.q.b", "l0.mix.k.b", "l0.mix.sink"):
            if name in tensors:
                tensors[name].zero_()
        tensors["pos"].zero_()
        embed = tensors["embed"]
        embed[0] = torch.cat((embed[1, 16:], embed[1, :16]))

    return raw, configs.write_folder(raw, 77, tmp_path / "planted", edit=edit)


def planted_requests(raw, places, length, seed=2):
    """{label: tokens} with an A at `first` and a B at `asked` for every (label, first, asked) in `places`."""
    rng = np.random.default_rng(seed)
    requests, asked = {}, {}
    for label, first, second in places:
        tokens = rng.integers(2, raw["vocab"], length).tolist()
        tokens[first], tokens[second] = 0, 1
        requests[label], asked[label] = tokens, second
    return requests, asked


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_keys_on_either_side_of_the_windows_edge_and_of_the_kept_positions(tmp_path, dtype):
    layer = configs.windowed(2, 2, 32, 32, 0.5, mask=(WINDOW, KEPT))
    raw, folder = planted_model(tmp_path, layer)
    tensors, _ = plain.load_model_dir(folder)
    places = []
    for label, first in (("edge", 40), ("early", 5), ("page", 31)):
        places += [(f"{label}_in", first, first + WINDOW - 1), (f"{label}_out", first, first + WINDOW)]
    # the kept positions: the last of them is seen from far away, the one behind it is not; and from a page's first token
    places += [("kept_in", KEPT - 1, 100), ("kept_out", KEPT, 100), ("first_in", 0, 64), ("first_out", KEPT, 64)]
    requests, asked = planted_requests(raw, places, 120)
    want = {key: plain.forward(tensors, raw, tokens) for key, tokens in requests.items()}
    for label in ("edge", "early", "page", "kept", "first"):           # the planted key matters: the two rows differ as a whole
        inside, outside = want[f"{label}_in"][asked[f"{label}_in"]], want[f"{label}_out"][asked[f"{label}_out"]]
        assert (inside - outside).norm() > 0.3 * inside.norm(), label
    for steps in (traces.whole(requests), traces.prefill_then_decode(requests, tail=90), traces.portions(requests, sizes=(5, 2, 30, 3, 17))):
        got = traces.collect(steps, run_replay(folder, dtype, steps, 128, tmp_path / f"o{len(steps)}"), raw["vocab"])
        for key, position in asked.items():
            assert position in got[key]
        check(got, want, dtype)
        for key, position in asked.items():                       # the rows that matter, one by one
            row, ref = got[key][position].double(), want[key][position]
            assert (row - ref).norm() < (1e-4 if dtype == "float32" else 5e-2) * ref.norm(), (key, position)
    steps, peak = traces.mixed(requests, seed=3, max_live=4, max_tokens=384)
    for step in steps:                                           # the rows that matter are asked for in every schedule
        for entry in step["entries"]:
            place = asked[entry["id"]] - entry["_at"]
            if 0 <= place < len(entry["tokens"]) and place not in entry["want"]:
                entry["want"] = sorted(entry["want"] + [place])
    got = traces.collect(steps, run_replay(folder, dtype, steps, peak, tmp_path / "mixed"), raw["vocab"])
    assert all(asked[key] in got[key] for key in asked)
    check(got, want, dtype)
    for key, position in asked.items():
        row, ref = got[key][position].double(), want[key][position]
        assert (row - ref).norm() < (1e-4 if dtype == "float32" else 5e-2) * ref.norm(), (key, position)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_key_far_back_among_hundreds(tmp_path, dtype):
    """Capped attention over the whole context, a quarter of every head rotated and stretched: the one matching key lies 600
    positions back, in the prompt's first page, and is found from a prompt's portion and from a single decoded token."""
    layer = configs.capped(2, 2, 32, 32, 0.5, rot=(1e4, 8, 2.0), softcap=12.0)
    raw, folder = planted_model(tmp_path, layer)
    tensors, _ = plain.load_model_dir(folder)
    requests, asked = planted_requests(raw, [("with", 7, 607), ("decoded", 15, 650)], 660)
    without = list(requests["with"])
    without[7] = 9
    requests["without"], asked["without"] = without, 607
    want = {key: plain.forward(tensors, raw, tokens) for key, tokens in requests.items()}
    assert (want["with"][607] - want["without"][607]).norm() > 0.3 * want["with"][607].norm()
    steps = []
    for number, (key, tokens) in enumerate(requests.items()):
        cut = 640 if key == "decoded" else 300
        steps.append({"step": len(steps), "entries": [{"id": key, "tokens": tokens[:cut], "want": [cut - 1]}], "end": []})
        if key == "decoded":
            for i in range(cut, 660):
                steps.append({"step": len(steps), "entries": [{"id": key, "tokens": [tokens[i]], "want": [0]}], "end": [key] if i == 659 else []})
        else:
            steps.append({"step": len(steps), "entries": [{"id": key, "tokens": tokens[cut:], "want": list(range(300, 360 - 0))}], "end": [key]})
    got = traces.collect(steps, run_replay(folder, dtype, steps, 704, tmp_path / "o"), raw["vocab"])
    assert 607 in got["with"] and 607 in got["without"] and 650 in got["decoded"]
    check(got, want, dtype)
    for key, position in asked.items():
        row, ref = got[key][position].double(), want[key][position]
        assert (row - ref).norm() < (1e-4 if dtype == "float32" else 5e-2) * ref.norm(), (key, position)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_beside_a_second_request(models, dtype, tmp_path):
    """240 tokens one by one behind a prompt of ten, a second request's tokens beside them: windows pass over decoded tokens,
    pages are given back while the request runs."""
    folder, raw, _, _ = models["cores"]
    tensors, _ = plain.load_model_dir(folder)
    rng = np.random.default_rng(17)
    requests = {"x": rng.integers(0, raw["vocab"], 250).tolist(), "y": rng.integers(0, raw["vocab"], 120).tolist()}
    want = {key: plain.forward(tensors, raw, tokens) for key, tokens in requests.items()}
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": requests["x"][:10], "want": [9]}, {"id": "y", "tokens": requests["y"][:3], "want": [2]}], "end": []}]
    for i in range(10, 250):
        entries = [{"id": "x", "tokens": [requests["x"][i]], "want": [0]}]
        j = i - 7
        if j < 120:
            entries.append({"id": "y", "tokens": [requests["y"][j]], "want": [0]})
        steps.append({"step": len(steps), "entries": entries, "end": (["y"] if j == 119 else []) + (["x"] if i == 249 else [])})
    got = traces.collect(steps, run_replay(folder, dtype, steps, 384, tmp_path / "o"), raw["vocab"])
    assert 249 in got["x"] and 119 in got["y"]
    check(got, want, dtype)


# ------------------------------------------------------------------------------------- generation
def test_greedy_generation_through_engine_and_scheduler(models):
    """Three prompts on two slots (the third waits and takes a freed slot and its pages), prompts fed in portions of at most 16
    tokens beside decoding requests: the tokens are the plain implementation's own greedy continuation."""
    from llm_runtime_study_amd import Engine

    folder, raw, requests, _ = models["odd"]
    tensors, _ = plain.load_model_dir(folder)
    prompts = [requests["odd2"], requests["odd6"][:30], requests["odd1"]]
    want = []
    for prompt in prompts:
        ids = list(prompt)
        for _ in range(6):
            ids.append(int(plain.forward(tensors, raw, ids)[-1].argmax()))
        want.append(ids[len(prompt):])
    engine = Engine.from_model_dir(folder, dtype="float32", max_seq_len=128, max_batch_size=2, max_num_batched_tokens=16)
    assert engine.generate_tokens(prompts, max_new_tokens=6) == want
    assert engine.cache_manager.active_requests == 0


def test_command_line_and_trace_run_as_programs(models, tmp_path):
    """The two programs, each a process of its own, find the architecture by the folder's config.json: greedy tokens from the
    command line (token ids in, token ids out, random weights from a seed as well), and a mixed replay through bin/trace_run."""
    import os
    import subprocess
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parents[1]
    env = dict(os.environ, PYTHONPATH=str(root))
    folder, raw, requests, want = models["awkward"]
    tensors, _ = plain.load_model_dir(folder)
    prompt = requests["awkward2"]
    ids = list(prompt)
    for _ in range(5):
        ids.append(int(plain.forward(tensors, raw, ids)[-1].argmax()))
    proc = subprocess.run([sys.executable, "-m", "llm_runtime_study_amd", "--model", str(folder), "--prompt-ids", ",".join(map(str, prompt)),
                           "--max-new-tokens", "5", "--dtype", "float32", "--max-seq-len", "64", "--no-metrics"],
                          capture_output=True, text=True, timeout=300, env=env, cwd=tmp_path)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [int(t) for t in proc.stdout.split()] == ids[len(prompt):]
    only_config = tmp_path / "only_config"
    only_config.mkdir()
    (only_config / "config.json").write_text((folder / "config.json").read_text())
    proc = subprocess.run([sys.executable, "-m", "llm_runtime_study_amd", "--model", str(only_config), "--random-weights", "3", "--prompt-ids", "1,2,3",
                           "--max-new-tokens", "4", "--max-seq-len", "64", "--no-metrics"], capture_output=True, text=True, timeout=300, env=env, cwd=tmp_path)
    assert proc.returncode == 0 and len(proc.stdout.split()) == 4, proc.stderr[-2000:]
    steps, peak = traces.mixed(requests, seed=9, max_live=3)
    out = tmp_path / "replayed"
    proc = subprocess.run([sys.executable, str(root / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32", "--out", str(out),
                           "--max-tokens", str(peak)], input=traces.strip(steps), capture_output=True, text=True, timeout=300, env=env, cwd=tmp_path)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [line for line in proc.stdout.splitlines() if line.startswith("done ")] == [f"done {s['step']}" for s in steps]
    check(traces.collect(steps, out, raw["vocab"]), want, "float32")
