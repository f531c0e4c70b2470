"""Nobodra on the GPU against the plain implementation (tests/plain/nobodra.py): each new mechanism alone, then whole
models of the tests' own sizes under every way of cutting their requests into steps, a key planted on either side
of a window's edge, a memory that must last hundreds of tokens, and greedy generation through Engine and scheduler.

Routing is a discrete choice: a bfloat16 run may rate two experts the other way round than the float64 plain forward
where their logits nearly tie.  float32 runs are compared row by row without exception; bfloat16 runs row by row
for models in which every expert runs (no choice), and by the share of rows within tolerance where experts are chosen.
"""

import math

import numpy as np
import pytest
import torch

from tests import nobodra_configs as configs
from tests import traces
from tests.plain import nobodra as plain
from tests.test_parts_gpu import PartHarness, close
from tests.test_replay_gpu import compare, round64, run_replay

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def bf16_values(*shape, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(*shape, generator=g)).to(torch.bfloat16).double()


# ------------------------------------------------------------------------------------- mechanisms alone
def test_norm_of_an_output_is_added_to_the_stream():
    from llm_runtime_study_amd.kernels import ops
    from llm_runtime_study_amd.parts import PartSpec, create

    part = create("norm", PartSpec("rmsnorm", {"size": 72, "eps": 0.02, "unit_offset": True}))
    stored = bf16_values(72, scale=0.3, seed=1)
    part.bind({"weight": stored.to(torch.bfloat16).cuda()}, torch.bfloat16)
    h, y = torch.randn(5, 72), 3 * torch.randn(5, 72)
    got = h.clone().cuda()
    part.add_normed(None, got, y.cuda())
    torch.testing.assert_close(got.cpu().double(), h.double() + plain.stream_norm(y.double(), stored, 0.02), rtol=1e-5, atol=1e-5)
    rounded = torch.empty(5, 72, dtype=torch.bfloat16, device="cuda")
    ops.round_rows(rounded, h.cuda())
    assert torch.equal(rounded.cpu(), h.to(torch.bfloat16))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,groups,d,e,taps", [(4, 2, 24, 40, 3), (2, 2, 64, 64, 4), (3, 1, 128, 16, 2), (1, 1, 10, 7, 1), (2, 1, 256, 128, 5)])
def test_gated_delta_rule_part(dtype, heads, groups, d, e, taps):
    """Two requests whose tokens arrive in steps of unequal sizes (a portion beside a single token, portions that end
    inside, at and just past the scan's chunk of 16 tokens), a slot given back and used again: every output row against
    the whole-sequence recurrence."""
    from llm_runtime_study_amd.kernels import ops
    from llm_runtime_study_amd.parts import PartSpec, create

    width = 48
    part = create("mixer", PartSpec("gated_delta_rule", {"hidden_size": width, "num_heads": heads, "num_kv_heads": groups, "head_dim": d,
                                                        "value_dim": e, "conv_taps": taps, "norm_eps": 1e-5}))
    shapes = {name: spec.shape for name, spec in part.tensors().items()}
    w = {name: bf16_values(*shape, scale=1.0 / math.sqrt(shape[-1]) if len(shape) == 2 else 0.5, seed=i) for i, (name, shape) in enumerate(shapes.items())}
    w["A_log"] = (w["A_log"] - 2.0).to(torch.bfloat16).double()      # decays near one: what a token wrote is still there dozens of tokens on
    w["norm.weight"] = (w["norm.weight"] + 1.0).to(torch.bfloat16).double()
    part.bind({name: t.to(torch.bfloat16).cuda() for name, t in w.items()}, dtype)
    assert part.state_floats() == heads * ops.library().lrs_delta_state_rows(d) * 16 * e + (taps - 1) * (2 * groups * d + heads * e)
    named = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "q.conv": "q_conv.weight", "k.conv": "k_conv.weight",
             "v.conv": "v_conv.weight", "b": "b_proj.weight", "a": "a_proj.weight", "A_log": "A_log", "dt_bias": "dt_bias", "g": "g_proj.weight",
             "norm": "norm.weight", "o": "o_proj.weight"}
    harness = PartHarness([part.cache_need()], dtype)
    inputs = {"a": bf16_values(70, width, seed=100), "b": bf16_values(40, width, seed=101), "c": bf16_values(19, width, seed=102)}
    want = {key: plain.gated_delta_rule(x, {short: w[long] for short, long in named.items()}, heads=heads, groups=groups, d=d, e=e, eps=1e-5)
            for key, x in inputs.items()}
    live, at, got = {}, {key: 0 for key in inputs}, {key: [] for key in inputs}
    schedule = [[("a", 15), ("b", 1)], [("a", 1), ("b", 17)], [("b", 16), ("a", 2)], [("a", 33)], [("a", 1), ("b", 1)], [("b", 5), ("a", 18)],
                [("c", 3)], [("c", 16)]]
    for number, step in enumerate(schedule):
        if number == 6:
            harness.cache.release(live.pop("b"))       # c takes the slot that b held: its row must read as zeros again
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
    for key in inputs:
        rows = torch.cat(got[key])
        close(rows, want[key][:rows.shape[0]], dtype, f32=5e-5, bf16=2e-2)
    assert live["c"].slot == 1


def moe_weights(width, ff, count, seed):
    ups = [bf16_values(ff, width, scale=1 / math.sqrt(width), seed=seed + 2 * e) for e in range(count)]
    downs = [bf16_values(width, ff, scale=1 / math.sqrt(ff), seed=seed + 2 * e + 1) for e in range(count)]
    return ups, downs


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,ff,count,top,tokens", [(64, 48, 6, 2, 50), (128, 64, 70, 3, 200), (128, 128, 8, 8, 33), (40, 24, 5, 1, 7), (320, 64, 16, 4, 1),
                                                       (128, 192, 3, 2, 400), (72, 40, 2, 2, 260), (256, 320, 4, 2, 600), (512, 96, 2, 1, 700)])
def test_grouped_expert_products_with_given_choices(dtype, width, ff, count, top, tokens):
    """The sort by expert, the two grouped products and the weighted sum, with the choices given (no routing decision to
    differ in): float32 on the vector units, bfloat16 on the matrix cores where the shape allows."""
    from llm_runtime_study_amd.kernels import ops

    ups, downs = moe_weights(width, ff, count, 10)
    x = bf16_values(tokens, width, seed=3)
    g = torch.Generator().manual_seed(4)
    ids = torch.stack([torch.randperm(count, generator=g)[:top] for _ in range(tokens)]).to(torch.int32)
    share = torch.softmax(torch.randn(tokens, top, generator=g), -1)
    want = torch.zeros(tokens, width, dtype=torch.float64)
    for t in range(tokens):
        for c in range(top):
            e = int(ids[t, c])
            want[t] += share[t, c].double() * (torch.relu(ups[e] @ x[t]).pow(2) @ downs[e].T)
    tile, tiles = ops.moe_tile_rows(tokens * top, count), ops.moe_max_tiles(tokens * top, count)
    assert tile == (128 if tokens >= 260 else 32)       # steps that bring every expert 48 rows and more use the larger tiles
    rows = tiles * tile
    sorted_pairs, place = torch.empty(rows, dtype=torch.int32, device="cuda"), torch.empty(tokens * top, dtype=torch.int32, device="cuda")
    tile_expert = torch.empty(tiles, dtype=torch.int32, device="cuda")
    ops.moe_align(ids.cuda(), count, sorted_pairs, place, tile_expert)
    listed = sorted_pairs.cpu()
    assert sorted(listed[listed >= 0].tolist()) == list(range(tokens * top))
    for number, e in enumerate(tile_expert.cpu().tolist()):       # every tile holds pairs of its one expert only
        inside = listed[number * tile:(number + 1) * tile]
        assert all(int(ids.view(-1)[p]) == e for p in inside[inside >= 0].tolist()) and (e >= 0 or (inside < 0).all())
    hidden = torch.empty(rows, ff, dtype=dtype, device="cuda")
    ops.moe_experts(hidden, x.to(dtype).cuda(), torch.stack(ups).to(dtype).cuda(), sorted_pairs, tile_expert, tile, top, gather=True, relu_squared=True)
    outputs = torch.empty(rows, width, dtype=torch.float32, device="cuda")
    ops.moe_experts(outputs, hidden, torch.stack(downs).to(dtype).cuda(), sorted_pairs, tile_expert, tile, top, gather=False, relu_squared=False)
    got = torch.ones(tokens, width, dtype=torch.float32, device="cuda")
    ops.moe_combine(got, outputs, place, share.cuda(), None)
    close(got - 1.0, want, dtype, f32=2e-5, bf16=1.5e-2)
    stored = bf16_values(width, scale=0.2, seed=9)
    got = torch.ones(tokens, width, dtype=torch.float32, device="cuda")
    ops.moe_combine(got, outputs, place, share.cuda(), (1.0 + stored).float().cuda(), 1e-5)
    close(got - 1.0, plain.stream_norm(want, stored, 1e-5), dtype, f32=2e-5, bf16=1.5e-2)


@pytest.mark.parametrize("count,top", [(6, 2), (70, 3), (5, 5), (130, 1), (64, 64)])
def test_routing_picks_the_largest_logits(count, top):
    from llm_runtime_study_amd.kernels import ops

    g = torch.Generator().manual_seed(count)
    logits, bias = torch.randn(37, count + 3, generator=g), torch.randn(count, generator=g)
    logits[5, :count] = 0.25
    bias_free = torch.zeros(count)
    for b in (bias, bias_free):
        ids = torch.empty(37, top, dtype=torch.int32, device="cuda")
        weights = torch.empty(37, top, dtype=torch.float32, device="cuda")
        ops.moe_route(logits.cuda()[:, :count], b.cuda(), ids, weights)
        values, where = (logits[:, :count] + b).topk(top, -1)
        rows = [r for r in range(37) if not (r == 5 and b is bias_free)]
        assert torch.equal(ids.cpu()[rows].long(), where[rows])
        torch.testing.assert_close(weights.cpu(), torch.softmax(values, -1), rtol=1e-5, atol=1e-6)
    assert ids.cpu()[5].tolist() == list(range(top))         # equal logits: the lowest indices


@pytest.mark.parametrize("dtype", DTYPES)
def test_routed_experts_part(dtype):
    from llm_runtime_study_amd.parts import PartSpec, create

    width, ff, count, top, tokens = 128, 64, 12, 3, 90
    part = create("feed_forward", PartSpec("routed_experts", {"hidden_size": width, "intermediate_size": ff, "num_experts": count, "top": top,
                                                              "router_bias": True}))
    ups, downs = moe_weights(width, ff, count, 20)
    router, bias = bf16_values(count, width, scale=0.3, seed=7), bf16_values(count, seed=8)
    w = {"router.weight": router, "router.bias": bias}
    for e in range(count):
        w[f"experts.{e}.up.weight"], w[f"experts.{e}.down.weight"] = ups[e], downs[e]
    assert set(w) == set(part.tensors())
    part.bind({name: t.to(torch.bfloat16).cuda() for name, t in w.items()}, dtype)
    x = bf16_values(tokens, width, seed=5)
    margins = []
    want = plain.routed_experts(x, router, bias, ups, downs, top, margins)
    harness = PartHarness([], dtype)
    ctx = harness.context([(harness.cache.admit("a"), [0] * tokens)])
    got = torch.zeros(tokens, width, dtype=torch.float32, device="cuda")
    part.forward(ctx, x.to(dtype).cuda(), got)
    sure = [t for t in range(tokens) if margins[t] > 1e-3]
    assert len(sure) > 0.9 * tokens
    close(got[sure], want[sure], dtype, f32=2e-5, bf16=1.5e-2)


# ------------------------------------------------------------------------------------- whole models
LENGTHS = {"routed": [1, 5, 23, 64, 97, 130, 33, 16], "dense": [2, 17, 48, 65, 150, 31, 9], "cores": [3, 40, 64, 129, 210, 18]}
RAW = {"routed": configs.ROUTED, "dense": configs.DENSE, "cores": configs.CORES}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for number, (name, raw) in enumerate(RAW.items()):
        folder = configs.write_folder(raw, 40 + number, tmp_path_factory.mktemp(f"nobodra_{name}"))
        _, weights = plain.load_model_dir(folder)
        rng = np.random.default_rng(11 + number)
        requests = {f"{name}{i}": rng.integers(0, raw["vocab"], n).tolist() for i, n in enumerate(LENGTHS[name])}
        want = {key: plain.forward(weights, raw, tokens) for key, tokens in requests.items()}
        out[name] = (folder, raw, requests, want)
    return out


def check(got, want, dtype, name="dense"):
    """float32: every row closely (see tests/test_replay_gpu.py: compare).  bfloat16 where no expert is chosen: 9 rows in 10
    within 3 % as a whole and every row within 20 % (these models are a few dozen values wide, and the norm that follows
    every sublayer magnifies the rounding of an output that happens to be small: the mean is 1 %, single rows reach 10 %,
    in whole prompts and in single tokens alike); bfloat16 with chosen experts: at least 85 of 100 rows within 3 %, none
    wildly off."""
    if dtype == "float32":
        return compare(got, want, dtype)
    errors = np.array([float((row.double() - want[key][position]).norm() / want[key][position].norm())
                       for key, rows in got.items() for position, row in rows.items()])
    close_rows, most = np.mean(errors < 3e-2), (0.85, 0.5) if name == "routed" else (0.9, 0.2)
    assert close_rows >= most[0] and errors.max() < most[1], f"{close_rows:.2f} of the rows are close, the worst is off by {errors.max():.3g}"
    return len(errors)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(RAW))
def test_whole_then_last_tokens_one_by_one_then_portions(models, name, dtype, tmp_path):
    folder, raw, requests, want = models[name]
    longest = max(round64(len(t)) for t in requests.values())
    steps = traces.whole(requests)
    got = traces.collect(steps, run_replay(folder, dtype, steps, longest, tmp_path / "whole"), raw["vocab"])
    assert check(got, want, dtype, name) == sum(len(t) for t in requests.values())
    steps = traces.prefill_then_decode(requests, tail=40)        # longer than two of the windows: they pass over decoded tokens
    check(traces.collect(steps, run_replay(folder, dtype, steps, longest, tmp_path / "tail"), raw["vocab"]), want, dtype, name)
    steps = traces.portions(requests)
    check(traces.collect(steps, run_replay(folder, dtype, steps, longest, tmp_path / "portions", page_size=32), raw["vocab"]), want, dtype, name)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,seed", [("routed", 0), ("routed", 1), ("dense", 2), ("cores", 3)])
def test_mixed_steps_with_pages_and_slots_used_again(models, name, seed, dtype, tmp_path):
    folder, raw, requests, want = models[name]
    budget = 2 * max(round64(len(t)) for t in requests.values())
    steps, peak = traces.mixed(requests, seed=seed, max_live=4, max_tokens=budget)
    assert max(len(s["entries"]) for s in steps) >= 3
    got = traces.collect(steps, run_replay(folder, dtype, steps, peak, tmp_path), raw["vocab"])
    assert check(got, want, dtype, name) > 50
    assert peak < sum(round64(len(t)) for t in requests.values())


@pytest.mark.parametrize("name", ["routed", "dense"])
def test_the_engines_path_of_graphs_and_recorded_steps(models, name, tmp_path):
    """On a stream of the runner's own with graphs on: single-token steps are graph replays, shapes that come back are
    launched from their recorded plan; a layer with state must see every step exactly once."""
    folder, raw, requests, want = models[name]
    longest = max(round64(len(t)) for t in requests.values())
    seen = {}
    steps = traces.prefill_then_decode(requests, tail=40)
    out = run_replay(folder, "float32", steps, longest, tmp_path / "tail", as_the_engine=True, counters=seen)
    check(traces.collect(steps, out, raw["vocab"]), want, "float32", name)
    assert seen["graph_replays"] >= 20 * (len(requests) - 2)
    steps, peak = traces.mixed(requests, seed=5, max_live=4, max_tokens=2 * longest)
    out = run_replay(folder, "bfloat16" if name == "dense" else "float32", steps, peak, tmp_path / "mixed", as_the_engine=True, counters=seen)
    check(traces.collect(steps, out, raw["vocab"]), want, "bfloat16" if name == "dense" else "float32", name)
    steps = traces.portions(requests, sizes=(16, 16, 16, 2))
    out = run_replay(folder, "float32", steps, longest, tmp_path / "portions", as_the_engine=True, counters=seen)
    check(traces.collect(steps, out, raw["vocab"]), want, "float32", name)
    assert seen["plan_replays"] >= 10


def test_cuts_change_no_bit_in_float32(models, tmp_path):
    folder, raw, requests, _ = models["routed"]
    a, b = traces.whole(requests), traces.portions(requests)
    ga = traces.collect(a, run_replay(folder, "float32", a, 192, tmp_path / "w"), raw["vocab"])
    gb = traces.collect(b, run_replay(folder, "float32", b, 192, tmp_path / "p"), raw["vocab"])
    for key in ga:
        for position in ga[key]:
            assert torch.equal(ga[key][position], gb[key][position]), f"{key}@{position}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_wider_model_through_the_products_for_many_rows(tmp_path, dtype):
    """Width 512 and prompts of 330 and 140 tokens: the projections of a prompt are products of hundreds of rows (the
    vendor library's in bfloat16), the experts get dozens to hundreds of rows each (large tiles), heads of 64 and 128."""
    raw = configs.WIDE
    folder = configs.write_folder(raw, 21, tmp_path / "wide")
    _, weights = plain.load_model_dir(folder)
    rng = np.random.default_rng(4)
    requests = {"long": rng.integers(0, raw["vocab"], 330).tolist(), "short": rng.integers(0, raw["vocab"], 140).tolist()}
    want = {key: plain.forward(weights, raw, tokens) for key, tokens in requests.items()}
    steps = [{"step": 0, "entries": [{"id": key, "tokens": tokens[:-6], "want": list(range(0, len(tokens) - 6, 7))} for key, tokens in requests.items()], "end": []}]
    for i in range(6, 0, -1):
        steps.append({"step": len(steps), "entries": [{"id": key, "tokens": [tokens[-i]], "want": [0]} for key, tokens in requests.items()],
                      "end": list(requests) if i == 1 else []})
    got = traces.collect(steps, run_replay(folder, dtype, steps, 512, tmp_path / "o"), raw["vocab"])
    assert check(got, want, dtype, "routed") > 70


# ------------------------------------------------------------------------------------- planted inputs
WINDOW = 21


def planted_model(tmp_path):
    """One attention layer (window 21, one head per key group, no rotation) whose query matrix is its key matrix
    behind a swap of the two halves of the stream: the query of token B is the key of token A when A's embedding is
    B's with its halves swapped.  With a score scale of 3 the match takes all the weight, so a B sees an A, and adds
    A's value to the stream, exactly when A lies inside its window.  Token 0 is A, token 1 is B."""
    raw = configs.model(50, 32, 1e-6, [configs.attention(2, 2, 16, 3.0, window=WINDOW, rot=None, mlp=None)])

    def edit(tensors):
        k = tensors["l0.mix.k"]
        tensors["l0.mix.q"] = torch.cat((k[:, 16:], k[:, :16]), 1)
        tensors["l0.mix.q.norm"].fill_(1.0)
        tensors["l0.mix.k.norm"].fill_(1.0)
        embed = tensors["embed"]
        embed[0] = torch.cat((embed[1, 16:], embed[1, :16]))

    return raw, configs.write_folder(raw, 77, tmp_path / "planted", edit)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_key_on_either_side_of_the_windows_edge(tmp_path, dtype):
    raw, folder = planted_model(tmp_path)
    _, weights = plain.load_model_dir(folder)
    rng = np.random.default_rng(2)
    requests, asked = {}, {}
    for label, first in (("edge", 40), ("early", 3), ("page", 31)):
        for distance in (WINDOW - 1, WINDOW):
            tokens = rng.integers(2, raw["vocab"], 120).tolist()
            tokens[first], tokens[first + distance] = 0, 1
            requests[f"{label}{distance}"], asked[f"{label}{distance}"] = tokens, first + distance
    want = {key: plain.forward(weights, raw, tokens) for key, tokens in requests.items()}
    for label in ("edge", "early", "page"):           # the planted key matters: the two rows differ as a whole
        inside, outside = want[f"{label}{WINDOW - 1}"][asked[f"{label}{WINDOW - 1}"]], want[f"{label}{WINDOW}"][asked[f"{label}{WINDOW}"]]
        assert (inside - outside).norm() > 0.3 * inside.norm()
    for steps in (traces.whole(requests), traces.prefill_then_decode(requests, tail=90), traces.portions(requests, sizes=(5, 2, 30, 3, 17))):
        got = traces.collect(steps, run_replay(folder, dtype, steps, 128, tmp_path / f"o{len(steps)}"), raw["vocab"])
        for key, position in asked.items():
            assert position in got[key]
        check(got, want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_memory_that_lasts_hundreds_of_tokens(tmp_path, dtype):
    """Delta layers that hardly decay (and no attention at all): the only way from one token to a later one is the state,
    and what the first tokens wrote still shapes the output dozens of tokens on, so a state that is lost, cleared or mixed
    up at any step's edge shows in the rows behind it."""
    raw = configs.model(90, 48, 1e-5, [configs.delta(2, 1, 16, 24, 3, None), configs.delta(3, 3, 8, 16, 4, configs.experts(16, 2, 2))])

    def edit(tensors):
        for layer in (0, 1):
            tensors[f"l{layer}.mix.A_log"].fill_(-7.0)

    folder = configs.write_folder(raw, 5, tmp_path / "lasting", edit)
    _, weights = plain.load_model_dir(folder)
    rng = np.random.default_rng(8)
    base = rng.integers(0, raw["vocab"], 520).tolist()
    other = list(base)
    other[:3] = [(t + 1) % raw["vocab"] for t in base[:3]]
    requests = {"x": base, "y": other}
    want = {key: plain.forward(weights, raw, tokens) for key, tokens in requests.items()}
    assert (want["x"][40] - want["y"][40]).norm() > 1e-3 * want["x"][40].norm()      # the first three tokens are remembered
    steps, at = [], 0
    for number, n in enumerate([300, 2, 100, 1, 1, 64, 16, 33, 1, 1, 1]):
        entries = [{"id": key, "tokens": tokens[at:at + n], "want": list(range(max(0, n - 8), n))} for key, tokens in requests.items()]
        steps.append({"step": number, "entries": entries, "end": ["x", "y"] if at + n == 520 else []})
        at += n
    assert at == 520
    got = traces.collect(steps, run_replay(folder, dtype, steps, 1088, tmp_path / "o"), raw["vocab"])
    check(got, want, dtype)


# ------------------------------------------------------------------------------------- generation
def test_greedy_generation_through_engine_and_scheduler(models):
    """Three prompts on two slots (the third waits and takes a freed slot and its state row), prompts fed in portions of
    at most 16 tokens beside decoding requests: the tokens are the plain implementation's own greedy continuation."""
    from llm_runtime_study_amd import Engine

    folder, raw, requests, _ = models["dense"]
    _, weights = plain.load_model_dir(folder)
    prompts = [requests["dense1"], requests["dense2"][:30], requests["dense0"]]
    want = []
    for prompt in prompts:
        ids = list(prompt)
        for _ in range(6):
            ids.append(int(plain.forward(weights, raw, ids)[-1].argmax()))
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
    folder, raw, requests, want = models["routed"]
    _, weights = plain.load_model_dir(folder)
    prompt = requests["routed2"]
    ids = list(prompt)
    for _ in range(5):
        ids.append(int(plain.forward(weights, raw, ids)[-1].argmax()))
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
    few = dict(list(requests.items())[2:6])
    steps, peak = traces.mixed(few, seed=9, max_live=3)
    out = tmp_path / "replayed"
    proc = subprocess.run([sys.executable, str(root / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32", "--out", str(out),
                           "--max-tokens", str(peak)], input=traces.strip(steps), capture_output=True, text=True, timeout=300, env=env, cwd=tmp_path)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [line for line in proc.stdout.splitlines() if line.startswith("done ")] == [f"done {s['step']}" for s in steps]
    compare(traces.collect(steps, out, raw["vocab"]), want, "float32")
