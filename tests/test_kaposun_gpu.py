"""Kaposun on the GPU against the plain implementation (tests/plain/kaposun.py): each mechanism alone (requests of unequal
length stepped side by side, slots and pages given back and used again), then whole models of the tests' own sizes under
every way of cutting their requests into steps, keys planted on either side of a window's edge and of the kept first
positions, a key far back among hundreds, a state that must last hundreds of tokens, and greedy generation through Engine
and scheduler."""

import math

import numpy as np
import pytest
import torch

from tests import kaposun_configs as configs
from tests import traces
from tests.plain import kaposun as plain
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
    name = name.removesuffix(".weight").replace("_proj", "").replace("_conv", ".conv").replace("_norm", ".norm")
    return name.replace("conv.bias", "conv.b")


def part_weights(part, seed, ranks=(5, 9)):
    """Random tensors of bfloat16 values for a part, by the part's own names; sizes left to the checkpoint are `ranks`."""
    out = {}
    for number, (name, spec) in enumerate(part.tensors().items()):
        rank = ranks[1] if ".g1" in short(name) or ".g2" in short(name) or short(name) in ("g1", "g2") else ranks[0]
        shape = tuple(rank if size == -1 else size for size in spec.shape)
        if spec.role == "norm":
            out[name] = 1.0 + bf16_values(*shape, scale=0.1, seed=seed + number)
            out[name] = out[name].to(torch.bfloat16).double()
        elif spec.role == "bias":
            out[name] = bf16_values(*shape, scale=0.5, seed=seed + number)
        else:
            out[name] = bf16_values(*shape, scale=1.0 / math.sqrt(shape[-1]), seed=seed + number)
    return out


def bound(part, w, dtype):
    part.bind({name: t.to(torch.bfloat16).cuda() for name, t in w.items()}, dtype)
    return {short(name): t for name, t in w.items()}


SCHEDULE = [[("a", 15), ("b", 1)], [("a", 1), ("b", 17)], [("b", 16), ("a", 2)], [("a", 33)], [("a", 1), ("b", 1)], [("b", 5), ("a", 18)],
            [("c", 3)], [("c", 16)], [("c", 1), ("a", 1)], [("a", 1), ("c", 2)]]
LENGTHS = {"a": 72, "b": 40, "c": 22}


def step_through(part, dtype, inputs, width, schedule=SCHEDULE, release_before=(6, "b"), page_size=16):
    """The rows a mixer gives for `inputs` {key: [n, width]} when their tokens arrive as `schedule` says: portions beside
    single tokens, portions that end inside, at and just past pages and the scan's chunk of 16 tokens; before step
    `release_before[0]` the request release_before[1] ends and the next admitted takes its slot (and pages)."""
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
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,groups,state,e,taps,parts", [(4, 2, 24, 40, 3, 2), (2, 2, 64, 64, 4, 1), (3, 1, 128, 16, 2, 3), (1, 1, 10, 7, 1, 1),
                                                             (6, 3, 48, 32, 4, 6), (2, 1, 256, 8, 5, 4), (20, 4, 16, 64, 2, 1)])
def test_state_space_part(dtype, heads, groups, state, e, taps, parts):
    from llm_runtime_study_amd.parts import PartSpec, create

    width = 48
    part = create("mixer", PartSpec("state_space", {"hidden_size": width, "num_heads": heads, "num_groups": groups, "state_size": state, "value_dim": e,
                                                   "conv_taps": taps, "norm_parts": parts, "norm_eps": 1e-5}))
    w = part_weights(part, 10)
    w["A_log"] = (w["A_log"] - 1.5).to(torch.bfloat16).double()       # slow decays: what a token wrote is still there dozens of tokens on
    named = bound(part, w, dtype)
    inputs = {key: bf16_values(n, width, seed=100 + i) for i, (key, n) in enumerate(LENGTHS.items())}
    want = {key: plain.state_space(x, named, heads=heads, groups=groups, state=state, e=e, taps=taps, parts=parts, eps=1e-5) for key, x in inputs.items()}
    got, live = step_through(part, dtype, inputs, width)
    for key in inputs:
        close(got[key], want[key][:got[key].shape[0]], dtype, f32=5e-5, bf16=2e-2)
    assert live["c"].slot == 1            # c took the slot b gave back: its state row read as zeros again


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,groups,d,e,taps,ranks", [(4, 2, 24, 40, 3, (5, 9)), (2, 2, 64, 64, 4, (16, 16)), (3, 1, 128, 16, 2, (1, 3)), (1, 1, 10, 7, 1, (4, 2)),
                                                         (2, 1, 256, 128, 5, (24, 8))])
def test_delta_rule_with_channel_decays_part(dtype, heads, groups, d, e, taps, ranks):
    from llm_runtime_study_amd.parts import PartSpec, create

    width = 48
    part = create("mixer", PartSpec("gated_delta_rule", {"hidden_size": width, "num_heads": heads, "num_kv_heads": groups, "head_dim": d, "value_dim": e,
                                                        "conv_taps": taps, "norm_eps": 1e-5, "channel_decay": True}))
    w = part_weights(part, 30, ranks)
    w["A_log"] = (w["A_log"] - 2.0).to(torch.bfloat16).double()
    named = bound(part, w, dtype)
    assert (part.decay_rank, part.gate_rank) == ranks
    inputs = {key: bf16_values(n, width, seed=200 + i) for i, (key, n) in enumerate(LENGTHS.items())}
    want = {key: plain.delta_rule_channel_decay(x, named, heads=heads, groups=groups, d=d, e=e, eps=1e-5) for key, x in inputs.items()}
    got, live = step_through(part, dtype, inputs, width)
    for key in inputs:
        close(got[key], want[key][:got[key].shape[0]], dtype, f32=5e-5, bf16=2e-2)
    assert live["c"].slot == 1


ATTENTION_SHAPES = [
    # heads, kv, d, e, scale, rot (base, dims, stretch), window, kept, gated
    (4, 2, 16, 24, 0.3, (500.0, 8, 4.0), None, 0, False),        # values wider than keys, part of a head rotated, stretched
    (6, 2, 32, 16, 0.2, None, 9, 3, True),                       # a window shorter than a page, three kept, gated
    (2, 1, 64, 64, 0.125, (1e4, 64, 1.0), None, 0, False),       # the matrix cores' shape
    (4, 4, 64, 64, 0.125, None, 20, 0, True),                    # ... behind a window that keeps nothing
    (2, 2, 128, 128, 0.09, None, 21, 18, True),                  # kept positions that reach into the second page
    (1, 1, 8, 8, 0.35, (100.0, 8, 2.0), 1, 0, False),            # a window of one
    (3, 1, 48, 40, 0.15, (1e6, 48, 2.0), 30, 30, False),         # as many kept as the window holds
    (4, 2, 64, 64, 0.125, (1e4, 32, 2.0), 24, 5, True),          # the matrix cores' shape with kept positions, half a head rotated
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,groups,d,e,scale,rot,window,kept,gated", ATTENTION_SHAPES)
def test_attention_normalised_over_the_projection_part(dtype, heads, groups, d, e, scale, rot, window, kept, gated):
    from llm_runtime_study_amd.parts import PartSpec, create

    width = 56
    position = PartSpec("none") if rot is None else PartSpec("rope_half", {"rotary_dim": rot[1], "theta": rot[0], "factor": rot[2]})
    part = create("mixer", PartSpec("gqa_attention", {"hidden_size": width, "num_heads": heads, "num_kv_heads": groups, "head_dim": d, "value_dim": e,
                                                     "position": position, "qk_norm": True, "qk_norm_eps": 1e-3, "norm_over": "projection", "scale": scale,
                                                     "window": window, "keep_first": kept, "output_gate": gated}))
    named = bound(part, part_weights(part, 50), dtype)
    assert ("g" in named) == gated and named["q.norm"].shape == (heads * d,)
    inputs = {key: bf16_values(n, width, seed=300 + i) for i, (key, n) in enumerate(LENGTHS.items())}
    want = {key: plain.softmax_attention(x, named, heads=heads, groups=groups, d=d, e=e, eps=1e-3, scale=scale, rot=rot, window=window, kept=kept, gated=gated)
            for key, x in inputs.items()}
    for page_size in (16, 4):
        got, live = step_through(part, dtype, inputs, width, page_size=page_size)
        for key in inputs:
            close(got[key], want[key][:got[key].shape[0]], dtype, f32=5e-5, bf16=2e-2)
    if window is not None and window < 40:
        first_kept_pages = -(-kept // 4)
        assert live["a"].first_live[0] > first_kept_pages         # pages between the kept positions and the window went back
        assert all(page >= 0 for page in live["a"].tables[0][:first_kept_pages])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("scales", [(0.8, 1.5), (1.0, 1.0)])
def test_two_mixers_side_by_side_part(dtype, scales):
    from llm_runtime_study_amd.parts import BothNeeds, PartSpec, create

    width = 40
    left = PartSpec("gqa_attention", {"hidden_size": width, "num_heads": 2, "num_kv_heads": 1, "head_dim": 32, "value_dim": 16, "qk_norm": True,
                                     "qk_norm_eps": 1e-5, "norm_over": "projection", "scale": 0.2, "window": 9, "keep_first": 3, "output_gate": True})
    right = PartSpec("gated_delta_rule", {"hidden_size": width, "num_heads": 4, "num_kv_heads": 2, "head_dim": 24, "value_dim": 8, "conv_taps": 2,
                                         "norm_eps": 1e-5, "channel_decay": True})
    part = create("mixer", PartSpec("side_by_side", {"left": left, "right": right, "left_scale": scales[0], "right_scale": scales[1]}))
    assert isinstance(part.cache_need(), BothNeeds)
    named = bound(part, part_weights(part, 70), dtype)
    inputs = {key: bf16_values(n, width, seed=400 + i) for i, (key, n) in enumerate(LENGTHS.items())}
    want = {}
    for key, x in inputs.items():
        a = plain.softmax_attention(x, plain.under(named, "left."), heads=2, groups=1, d=32, e=16, eps=1e-5, scale=0.2, window=9, kept=3, gated=True)
        b = plain.delta_rule_channel_decay(x, plain.under(named, "right."), heads=4, groups=2, d=24, e=8, eps=1e-5)
        want[key] = scales[0] * a + scales[1] * b
    got, _ = step_through(part, dtype, inputs, width)
    for key in inputs:
        close(got[key], want[key][:got[key].shape[0]], dtype, f32=5e-5, bf16=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["gelu", "gelu_tanh"])
def test_dense_feed_forward_part(dtype, kind):
    from llm_runtime_study_amd.parts import PartSpec, create

    width, ff, rows = 72, 136, 21
    part = create("feed_forward", PartSpec("dense_mlp", {"hidden_size": width, "intermediate_size": ff, "activation": kind}))
    named = bound(part, part_weights(part, 90), dtype)
    x = bf16_values(rows, width, scale=2.0, seed=5)
    hidden = x @ named["up"].T
    act = plain.gelu_exact(hidden) if kind == "gelu" else torch.nn.functional.gelu(hidden, approximate="tanh")
    harness = PartHarness([], dtype)
    ctx = harness.context([(harness.cache.admit("a"), [0] * rows)])
    out = torch.full((rows, width), 0.25, dtype=torch.float32, device="cuda")
    part.forward(ctx, x.to(dtype).cuda(), out)
    close(out - 0.25, act @ named["down"].T, dtype, f32=3e-5, bf16=1.5e-2)
    part.forward(ctx, x.to(dtype).cuda(), out, accumulate=False)
    close(out, act @ named["down"].T, dtype, f32=3e-5, bf16=1.5e-2)


@pytest.mark.parametrize("cols", [136, 135, 4096, 8200])
def test_sum_into_the_stream_leaves_the_next_norm(cols):
    """Rows of a multiple of four values up to 8,192 go through the kernel that keeps them in registers, the others through
    the plain one."""
    from llm_runtime_study_amd.kernels import ops

    h, y = torch.randn(9, cols), 3 * torch.randn(9, cols)
    weight = (1 + 0.2 * torch.randn(cols)).to(torch.bfloat16).float()
    want = h.double() + 0.3 * y.double()
    for dtype in DTYPES:
        stream, normed = h.clone().cuda(), torch.empty(9, cols, dtype=dtype, device="cuda")
        ops.axpby(stream, stream, 1.0, y.cuda(), 0.3, weight.cuda(), 1e-3, normed)
        torch.testing.assert_close(stream.cpu().double(), want, rtol=1e-6, atol=1e-6)
        close(normed, plain.unit_rms(want, 1e-3) * weight.double(), dtype, f32=1e-5, bf16=5e-3)
    out = torch.empty(9, cols, device="cuda")
    ops.axpby(out, h.cuda(), 0.8, y.cuda(), 1.5)
    torch.testing.assert_close(out.cpu().double(), 0.8 * h.double() + 1.5 * y.double(), rtol=1e-6, atol=1e-6)


# ------------------------------------------------------------------------------------- whole models
MODEL_LENGTHS = {"odd": [1, 5, 23, 64, 97, 130, 33, 16], "cores": [3, 40, 64, 129, 210, 18], "ones": [2, 17, 48, 65, 150, 31, 9], "self_loop": [4, 70, 31, 120, 2],
                 "awkward": [7, 50, 1, 100, 33, 140]}
RAW = {"odd": configs.ODD, "cores": configs.CORES, "ones": configs.ONES, "self_loop": configs.SELF_LOOP, "awkward": configs.AWKWARD}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for number, (name, raw) in enumerate(RAW.items()):
        folder = configs.write_folder(raw, 60 + number, tmp_path_factory.mktemp(f"kaposun_{name}"), ranks=(3 + 2 * number, 4 + number))
        _, tensors = plain.load_folder(folder)
        rng = np.random.default_rng(21 + number)
        requests = {f"{name}{i}": rng.integers(0, raw["vocab"], n).tolist() for i, n in enumerate(MODEL_LENGTHS[name])}
        want = {key: plain.forward(raw, tensors, tokens) for key, tokens in requests.items()}
        out[name] = (folder, raw, requests, want)
    return out


def check(got, want, dtype):
    """float32: every row within 3e-5 of the plain row as a whole (relative L2) and no logit further off than 1e-4 of the
    row's largest (the logits of these models run to dozens, and a state carried through hundreds of float32 updates
    rounds).  bfloat16: these models are a few dozen values wide, so a single row's rounding is larger than a real
    model's: 9 rows in 10 within 3 % as a whole and every row within 20 %."""
    errors = np.array([float((row.double() - want[key][position]).norm() / want[key][position].norm())
                       for key, rows in got.items() for position, row in rows.items()])
    if dtype == "float32":
        worst = max(float((row.double() - want[key][position]).abs().max() / want[key][position].abs().max())
                    for key, rows in got.items() for position, row in rows.items())
        assert errors.max() < 3e-5 and worst < 1e-4, f"the worst row is off by {errors.max():.3g} as a whole, the worst logit by {worst:.3g} of its row's largest"
        return len(errors)
    assert np.mean(errors < 3e-2) >= 0.9 and errors.max() < 0.2, f"{np.mean(errors < 3e-2):.2f} of the rows are close, the worst is off by {errors.max():.3g}"
    return len(errors)


def test_the_stream_after_every_layer_run(models):
    """One step function call on a whole prompt in float32, the stream read after every run of a layer (a looped layer
    counts each time) against the plain implementation's."""
    from llm_runtime_study_amd.engine import trace
    from llm_runtime_study_amd.engine.step import StepEntry

    for name in ("odd", "self_loop"):
        folder, raw, requests, _ = models[name]
        tokens = requests[f"{name}2"]
        _, tensors = plain.load_folder(folder)
        streams = []
        plain.forward(raw, tensors, tokens, streams)
        runner = trace.make_runner(folder, "float32", 64, 16)
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
        assert len(seen) == len(streams) == len(plain.layer_order(raw))
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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,seed", [("odd", 0), ("odd", 1), ("cores", 2), ("ones", 3), ("self_loop", 4), ("awkward", 6)])
def test_mixed_steps_with_pages_and_slots_used_again(models, name, seed, dtype, tmp_path):
    folder, raw, requests, want = models[name]
    budget = 2 * max(round64(len(t)) for t in requests.values())
    steps, peak = traces.mixed(requests, seed=seed, max_live=4, max_tokens=budget)
    assert max(len(s["entries"]) for s in steps) >= 3
    got = traces.collect(steps, run_replay(folder, dtype, steps, peak, tmp_path), raw["vocab"])
    assert check(got, want, dtype) > 40
    assert peak < sum(round64(len(t)) for t in requests.values())


@pytest.mark.parametrize("name", ["odd", "cores"])
def test_the_engines_path_of_graphs_and_recorded_steps(models, name, tmp_path):
    """On a stream of the runner's own with graphs on: single-token steps are graph replays, shapes that come back are
    launched from their recorded plan; a layer with state must see every step exactly once."""
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
    library's in bfloat16), the window of 150 lies inside the longer prompt, heads of 64 and 96."""
    raw = configs.WIDE
    folder = configs.write_folder(raw, 21, tmp_path / "wide", ranks=(16, 24))
    _, tensors = plain.load_folder(folder)
    rng = np.random.default_rng(4)
    requests = {"long": rng.integers(0, raw["vocab"], 330).tolist(), "short": rng.integers(0, raw["vocab"], 140).tolist()}
    want = {key: plain.forward(raw, tensors, tokens) for key, tokens in requests.items()}
    steps = [{"step": 0, "entries": [{"id": key, "tokens": tokens[:-6], "want": list(range(0, len(tokens) - 6, 7))} for key, tokens in requests.items()], "end": []}]
    for i in range(6, 0, -1):
        steps.append({"step": len(steps), "entries": [{"id": key, "tokens": [tokens[-i]], "want": [0]} for key, tokens in requests.items()],
                      "end": list(requests) if i == 1 else []})
    got = traces.collect(steps, run_replay(folder, dtype, steps, 512, tmp_path / "o"), raw["vocab"])
    assert check(got, want, dtype) > 70


# ------------------------------------------------------------------------------------- planted inputs
WINDOW, KEPT = 21, 3


def planted_model(tmp_path, layer):
    """A model of one layer whose attention's query matrix is its key matrix behind a swap of the two halves of the stream:
    the query of token B is the key of token A when A's embedding is B's with its halves swapped (the layer's norm weighs
    all channels alike, so it keeps the swap).  The match's score towers over every other, so a B sees an A, and adds A's
    value to the stream, exactly when A is visible from B.  Token 0 is A, token 1 is B."""
    raw = configs.model(50, 32, 1e-6, 1.0, [layer])
    prefix = "l0.mix.left." if layer["type"] == "parallel" else "l0.mix."

    def edit(tensors):
        k = tensors[prefix + "k"]
        tensors[prefix + "q"] = torch.cat((k[:, 16:], k[:, :16]), 1).contiguous()
        tensors[prefix + "q.norm"].fill_(1.0)
        tensors[prefix + "k.norm"].fill_(1.0)
        tensors["l0.norm1"].fill_(1.0)
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
    layer = configs.parallel(configs.attention_sizes(2, 2, 32, 32, 2.0, mask=(WINDOW, KEPT)), (2, 1, 8, 8, 2), 1.0, 0.3)
    raw, folder = planted_model(tmp_path, layer)
    _, tensors = plain.load_folder(folder)
    places = []
    for label, first in (("edge", 40), ("early", 5), ("page", 31)):
        places += [(f"{label}_in", first, first + WINDOW - 1), (f"{label}_out", first, first + WINDOW)]
    # the kept positions: the last of them is seen from far away, the one behind it is not; and from a page's first token
    places += [("kept_in", KEPT - 1, 100), ("kept_out", KEPT, 100), ("first_in", 0, 64), ("first_out", KEPT, 64)]
    requests, asked = planted_requests(raw, places, 120)
    want = {key: plain.forward(raw, tensors, tokens) for key, tokens in requests.items()}
    for label in ("edge", "early", "page", "kept", "first"):           # the planted key matters: the two rows differ as a whole
        inside, outside = want[f"{label}_in"][asked[f"{label}_in"]], want[f"{label}_out"][asked[f"{label}_out"]]
        assert (inside - outside).norm() > 0.3 * inside.norm(), label
    for steps in (traces.whole(requests), traces.prefill_then_decode(requests, tail=90), traces.portions(requests, sizes=(5, 2, 30, 3, 17))):
        got = traces.collect(steps, run_replay(folder, dtype, steps, 128, tmp_path / f"o{len(steps)}"), raw["vocab"])
        for key, position in asked.items():
            assert position in got[key]
        check(got, want, dtype)
    steps, peak = traces.mixed(requests, seed=3, max_live=4, max_tokens=384)
    for step in steps:                                           # the rows that matter are asked for in every schedule
        for entry in step["entries"]:
            place = asked[entry["id"]] - entry["_at"]
            if 0 <= place < len(entry["tokens"]) and place not in entry["want"]:
                entry["want"] = sorted(entry["want"] + [place])
    got = traces.collect(steps, run_replay(folder, dtype, steps, peak, tmp_path / "mixed"), raw["vocab"])
    assert all(asked[key] in got[key] for key in asked)
    check(got, want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_key_far_back_among_hundreds(tmp_path, dtype):
    """Attention over the whole context, a quarter of every head rotated: the one matching key lies 600 positions back, in the
    prompt's first page, and is found from a prompt's portion and from a single decoded token."""
    layer = configs.attention(2, 2, 32, 24, 2.0, rot=(1e4, 8, 2.0))
    raw, folder = planted_model(tmp_path, layer)
    _, tensors = plain.load_folder(folder)
    requests, asked = planted_requests(raw, [("with", 7, 607), ("decoded", 15, 650)], 660)
    without = list(requests["with"])
    without[7] = 9
    requests["without"], asked["without"] = without, 607
    want = {key: plain.forward(raw, tensors, tokens) for key, tokens in requests.items()}
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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_states_that_last_hundreds_of_tokens(tmp_path, dtype):
    """State space and delta layers that hardly decay behind a window of two tokens: the only way from a token to one far
    behind it is the state, and what the first tokens wrote still shapes the output dozens of tokens on, so a state that is
    lost, cleared or mixed up at any step's edge shows in the rows behind it."""
    raw = configs.model(90, 48, 1e-5, 0.6, [
        configs.mamba(3, 1, 16, 16, 3, 1, mlp=None),
        configs.parallel(configs.attention_sizes(2, 1, 16, 16, 0.25, mask=(2,)), (3, 3, 8, 16, 4), 0.2, 1.0, mlp=configs.dense(32)),
        configs.mamba(2, 2, 24, 8, 2, 2, mlp=configs.dense(16))], loop=(0, 2, 2))

    def edit(tensors):
        for name in tensors:
            if name.endswith("A_log"):
                tensors[name].fill_(-6.0)

    folder = configs.write_folder(raw, 5, tmp_path / "lasting", edit=edit)
    _, tensors = plain.load_folder(folder)
    rng = np.random.default_rng(8)
    base = rng.integers(0, raw["vocab"], 520).tolist()
    other = list(base)
    other[:3] = [(t + 1) % raw["vocab"] for t in base[:3]]
    requests = {"x": base, "y": other}
    want = {key: plain.forward(raw, tensors, tokens) for key, tokens in requests.items()}
    assert (want["x"][60] - want["y"][60]).norm() > 1e-3 * want["x"][60].norm()      # the first three tokens are remembered
    steps, at = [], 0
    for number, n in enumerate([300, 2, 100, 1, 1, 64, 16, 33, 1, 1, 1]):
        entries = [{"id": key, "tokens": tokens[at:at + n], "want": list(range(max(0, n - 8), n))} for key, tokens in requests.items()]
        steps.append({"step": number, "entries": entries, "end": ["x", "y"] if at + n == 520 else []})
        at += n
    assert at == 520
    got = traces.collect(steps, run_replay(folder, dtype, steps, 1088, tmp_path / "o"), raw["vocab"])
    check(got, want, dtype)
    # long decoding: 200 tokens one by one behind a short prompt
    tail = {"x": base[:230]}
    steps = traces.prefill_then_decode(tail, tail=200)
    got = traces.collect(steps, run_replay(folder, dtype, steps, 256, tmp_path / "tail"), raw["vocab"])
    check(got, {"x": want["x"][:230]}, dtype)


# ------------------------------------------------------------------------------------- generation
def test_greedy_generation_through_engine_and_scheduler(models):
    """Three prompts on two slots (the third waits and takes a freed slot, its state rows and pages), prompts fed in portions
    of at most 16 tokens beside decoding requests: the tokens are the plain implementation's own greedy continuation."""
    from llm_runtime_study_amd import Engine

    folder, raw, requests, _ = models["odd"]
    _, tensors = plain.load_folder(folder)
    prompts = [requests["odd2"], requests["odd6"][:30], requests["odd1"]]
    want = []
    for prompt in prompts:
        ids = list(prompt)
        for _ in range(6):
            ids.append(int(plain.forward(raw, tensors, ids)[-1].argmax()))
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
    folder, raw, requests, want = models["self_loop"]
    _, tensors = plain.load_folder(folder)
    prompt = requests["self_loop2"]
    ids = list(prompt)
    for _ in range(5):
        ids.append(int(plain.forward(raw, tensors, ids)[-1].argmax()))
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
