"""Napizen on the GPU against the plain implementation (tests/plain/napizen.py): each mechanism alone, then whole models
of the tests' own sizes under every way of cutting their requests into steps, a far key that must be found among hundreds,
a sink that takes most of the weight, and greedy generation through Engine and scheduler.

Routing is a discrete choice: a bfloat16 run may rate two experts (or two groups) the other way round than the float64
plain forward where their scores nearly tie.  float32 runs are compared row by row without exception; bfloat16 runs by
the share of rows within tolerance where experts are chosen.
"""

import math

import numpy as np
import pytest
import torch

from tests import napizen_configs as configs
from tests import traces
from tests.plain import napizen as plain
from tests.test_parts_gpu import PartHarness, close
from tests.test_replay_gpu import compare, round64, run_replay

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def bf16_values(*shape, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(*shape, generator=g)).to(torch.bfloat16).double()


# ------------------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("width", [48, 256, 2050])
def test_layer_norm_of_rows_and_of_the_sum(width):
    from llm_runtime_study_amd.parts import PartSpec, create

    part = create("norm", PartSpec("layernorm", {"size": width, "eps": 0.03}))
    weight = bf16_values(width, scale=0.3, seed=1) + 1.0
    part.bind({"weight": weight.to(torch.bfloat16).cuda()}, torch.bfloat16)
    weight = weight.to(torch.bfloat16).double()
    h, y = 2.0 + torch.randn(7, width), 3 * torch.randn(7, width)       # a mean far from zero: a norm that left it in would show
    harness = PartHarness([], torch.float32)
    ctx = harness.context([(harness.cache.admit("a"), [0] * 7)])
    got = part.forward(ctx, h.cuda())
    torch.testing.assert_close(got.cpu().double(), plain.centred_norm(h.double(), weight, 0.03), rtol=1e-5, atol=1e-5)
    rows = torch.tensor([5, 0, 5], dtype=torch.int32)
    got = part.forward(ctx, h.cuda(), rows=rows.cuda(), count=3)
    torch.testing.assert_close(got.cpu().double(), plain.centred_norm(h.double()[rows.long()], weight, 0.03), rtol=1e-5, atol=1e-5)
    stream, rounded = h.clone().cuda(), torch.empty(7, width, dtype=torch.bfloat16, device="cuda")
    part.scale_add_normed(ctx, stream, y.cuda(), 1.75, rounded=rounded)
    want = plain.centred_norm(1.75 * h.double() + y.double(), weight, 0.03)
    torch.testing.assert_close(stream.cpu().double(), want, rtol=1e-5, atol=1e-5)
    assert torch.equal(rounded.cpu(), stream.cpu().to(torch.bfloat16))


@pytest.mark.parametrize("dims,base,scaling", [(8, 10000.0, (8.0, 64, 16.0, 2.0)), (16, 2e5, (6.0, 1024, 24.0, 2.0)), (2, 30.0, None), (64, 1e4, (40.0, 4096, 32.0, 1.0))])
def test_rotation_tables_of_neighbouring_pairs(dims, base, scaling):
    from llm_runtime_study_amd.parts import PartSpec, create

    rot = {"dims": dims, "base": base}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    part = create("position", PartSpec("rope_interleaved", {"rotary_dim": dims, "theta": base, "scaling": rot.get("scaling")}))
    harness = PartHarness([], torch.float32, max_step_tokens=2048)
    request = harness.cache.admit("a")
    harness.cache.extend(request, 900)                      # the step's tokens stand at positions 900..1099
    ctx = harness.context([(request, [0] * 200)])
    cos, sin = part.tables(ctx)
    assert part.tables(ctx)[0] is cos                       # made once a step
    rates, factor = plain.pair_rates(rot)
    angle = torch.arange(900, 1100, dtype=torch.float64)[:, None] * torch.tensor(rates, dtype=torch.float64)
    # float32 angles of a thousand radians carry errors of 1e-4
    torch.testing.assert_close(cos.cpu().double(), angle.cos() * factor, rtol=0, atol=3e-4)
    torch.testing.assert_close(sin.cpu().double(), angle.sin() * factor, rtol=0, atol=3e-4)


@pytest.mark.parametrize("count,top,groups,scale", [(6, 2, (2, 1), 1.5), (9, 3, (3, 2), 2.5), (8, 3, (4, 2), 2.25), (70, 2, (70, 5), 0.5), (4, 1, (4, 4), 1.0),
                                                    (3, 3, None, 1.0), (130, 5, (10, 4), 3.0), (64, 64, None, 1.0), (256, 8, (8, 4), 2.5), (12, 4, (6, 2), 1.0)])
def test_routing_by_sigmoid_scores_among_the_best_groups(count, top, groups, scale):
    """Corrections well below zero make choice scores negative: an expert of a dropped group must count as minus infinity,
    not as zero.  Rows whose choice the plain implementation calls close are left out, the others agree exactly."""
    from llm_runtime_study_amd.kernels import ops

    g = torch.Generator().manual_seed(count)
    tokens = 60
    logits, correction = 2 * torch.randn(tokens, count + 3, generator=g), torch.randn(count, generator=g) - 1.5
    router = {"experts": count, "top": top, "scale": scale}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    margins = []
    chosen, shares = plain.choose_experts(logits[:, :count].double(), correction.double(), router, margins)
    rule = ops.RouteRule("sigmoid", *(groups or (0, 0)), scale)
    ids = torch.empty(tokens, top, dtype=torch.int32, device="cuda")
    weights = torch.empty(tokens, top, dtype=torch.float32, device="cuda")
    ops.moe_route(logits.cuda()[:, :count], correction.cuda(), ids, weights, rule=rule)
    sure = [t for t in range(tokens) if margins[t] > 1e-5]
    assert len(sure) > 0.9 * tokens
    for t in sure:
        assert ids[t].tolist() == chosen[t], f"token {t}"
        torch.testing.assert_close(weights[t].cpu().double(), torch.tensor(shares[t], dtype=torch.float64), rtol=1e-5, atol=1e-6)
    if True:                                                 # the one-launch form for steps of few tokens chooses the same
        few = min(tokens, ops.ROUTE_ALIGN_TOKENS)
        tile, tiles = ops.moe_tile_rows(few * top, count), ops.moe_max_tiles(few * top, count)
        lists = [torch.empty(n, dtype=torch.int32, device="cuda") for n in (tiles * tile, few * top, tiles)]
        ids2, weights2 = torch.empty(few, top, dtype=torch.int32, device="cuda"), torch.empty(few, top, dtype=torch.float32, device="cuda")
        ops.moe_route_align(logits.cuda()[:few, :count], correction.cuda(), ids2, weights2, *lists, rule=rule)
        assert torch.equal(ids2, ids[:few]) and torch.equal(weights2, weights[:few])


def expert_weights(width, ff, count, seed):
    return {f"experts.{e}.{name}.weight": bf16_values(*shape, scale=1 / math.sqrt(shape[1]), seed=seed + 3 * e + i)
            for e in range(count) for i, (name, shape) in enumerate((("gate", (ff, width)), ("up", (ff, width)), ("down", (width, ff))))}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,ff,count,top,groups,tokens", [(64, 48, 6, 2, (3, 2), 50), (128, 64, 12, 3, (4, 2), 90), (128, 128, 8, 8, None, 33), (40, 24, 5, 1, None, 7),
                                                             (320, 64, 16, 4, (4, 3), 1), (128, 192, 4, 2, (2, 1), 400)])
def test_routed_gated_experts_part(dtype, width, ff, count, top, groups, tokens):
    from llm_runtime_study_amd.parts import PartSpec, create

    part = create("feed_forward", PartSpec("routed_experts", {
        "hidden_size": width, "intermediate_size": ff, "num_experts": count, "top": top, "router_bias": True, "bias_name": "correction",
        "activation": "silu_gated", "rule": "sigmoid", "groups": groups[0] if groups else 0, "keep": groups[1] if groups else 0, "weight_scale": 1.75}))
    w = expert_weights(width, ff, count, 20)
    w["router.weight"], w["correction"] = bf16_values(count, width, scale=0.3, seed=7), (bf16_values(count, seed=8) - 1.0).to(torch.bfloat16).double()
    assert set(w) == set(part.tensors())
    part.bind({name: t.to(torch.bfloat16).cuda() for name, t in w.items()}, dtype)
    x = bf16_values(tokens, width, seed=5)
    short = {"router": w["router.weight"], "correction": w["correction"]}
    short.update({f"e{e}.{name}": w[f"experts.{e}.{name}.weight"] for e in range(count) for name in ("gate", "up", "down")})
    router = {"experts": count, "top": top, "scale": 1.75}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    margins = []
    want = plain.routed_ff(x, short, {"router": router}, margins)
    harness = PartHarness([], dtype, max_step_tokens=512)
    ctx = harness.context([(harness.cache.admit("a"), [0] * tokens)])
    got = torch.zeros(tokens, width, dtype=torch.float32, device="cuda")
    part.forward(ctx, x.to(dtype).cuda(), got)
    sure = [t for t in range(tokens) if margins[t] > (1e-4 if dtype == torch.float32 else 2e-2)]
    assert len(sure) > 0.7 * tokens
    close(got[sure], want[sure], dtype, f32=2e-5, bf16=1.5e-2)


def latent_part(width, heads, d, r, e, c, scale, rot, dtype, seed, edit=None):
    from llm_runtime_study_amd.parts import PartSpec, create

    position = PartSpec("rope_interleaved", {"rotary_dim": r, "theta": rot["base"], "scaling": rot.get("scaling")})
    part = create("mixer", PartSpec("latent_attention", {"hidden_size": width, "num_heads": heads, "head_dim": d, "rot_dim": r, "value_dim": e, "kv_rank": c,
                                                        "position": position, "norm_eps": 1e-5, "scale": scale, "sink": True, "gate": True}))
    w = {name: bf16_values(*spec.shape, scale=1.0 / math.sqrt(spec.shape[-1]) if len(spec.shape) == 2 else 0.5, seed=seed + i)
         for i, (name, spec) in enumerate(part.tensors().items())}
    w["dkv_norm.weight"] = (w["dkv_norm.weight"] + 1.0).to(torch.bfloat16).double()
    if edit is not None:
        edit(w)
    part.bind({name: t.to(torch.bfloat16).cuda() for name, t in w.items()}, dtype)
    named = {"q": "q_proj.weight", "dkv": "dkv_proj.weight", "dkv.norm": "dkv_norm.weight", "uk": "uk_proj.weight", "uv": "uv_proj.weight", "sink": "sink",
             "g": "g_proj.weight", "o": "o_proj.weight"}
    m = {"heads": heads, "dim": d, "rot_dim": r, "vdim": e, "kv_rank": c, "scale": scale, "rot": rot}
    return part, {short: w[long] for short, long in named.items()}, m


SCALED = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,d,r,e,c,scaling", [(3, 16, 8, 24, 40, SCALED), (1, 8, 2, 8, 8, None), (4, 64, 32, 64, 96, SCALED), (16, 32, 16, 32, 64, None),
                                                   (2, 128, 64, 128, 256, None), (5, 24, 4, 10, 20, None), (8, 128, 64, 128, 512, SCALED)])
def test_latent_attention_part_in_portions(dtype, heads, d, r, e, c, scaling):
    """Three requests whose tokens arrive in steps of unequal sizes (portions beside single tokens, portions that end inside,
    at and just past a page's edge, two tokens), a request's pages given back and used again by the next: every output row
    against the whole-sequence plain mixer.  The page is 16 tokens, the cache holds few."""
    width = 64
    rot = {"base": 10000.0, "dims": r}
    if scaling is not None:
        rot["scaling"] = scaling
    part, w, m = latent_part(width, heads, d, r, e, c, 0.3 / math.sqrt(d + r) * 4, rot, dtype, seed=3)
    need = part.cache_need()
    # float32 keeps one row a position and nothing else; bfloat16 keeps the latent values once more, a column's keys side by side
    columns = c if dtype == torch.bfloat16 and (c + r) % 8 == 0 else 0
    assert need.head_dim == c + r and need.value_dim == columns
    harness = PartHarness([need], dtype, max_step_tokens=160)
    assert harness.cache.layer_caches[0].k_pages.shape[1:] == (1, 16, c + r)
    assert (harness.cache.layer_caches[0].v_pages is None) if not columns else harness.cache.layer_caches[0].v_pages.shape[1:] == (1, c, 16)
    inputs = {"a": bf16_values(81, width, seed=100), "b": bf16_values(47, width, seed=101), "c": bf16_values(35, width, seed=102)}
    want = {key: plain.latent_attention(x, w, m, 1e-5) for key, x in inputs.items()}
    live, at, got = {}, {key: 0 for key in inputs}, {key: [] for key in inputs}
    schedule = [[("a", 15), ("b", 1)], [("a", 1), ("b", 17)], [("b", 14), ("a", 2)], [("a", 33)], [("a", 1), ("b", 1)], [("b", 14), ("a", 29)],
                [("c", 3)], [("c", 16), ("a", 0)], [("c", 1)], [("c", 13)], [("c", 2)]]
    for number, step in enumerate(schedule):
        if number == 6:
            assert at["b"] == 47
            harness.cache.release(live.pop("b"))       # c takes pages that b held
        step = [(key, n) for key, n in step if n]
        entries = []
        for key, n in step:
            if key not in live:
                live[key] = harness.cache.admit(key)
            entries.append((live[key], [0] * n))
        ctx = harness.context(entries)
        x = torch.cat([inputs[key][at[key]:at[key] + n] for key, n in step]).to(dtype).cuda()
        out = torch.zeros(x.shape[0], width, dtype=torch.float32, device="cuda")
        part.forward(ctx, x, out, harness.cache.layer_caches[0])
        row = 0
        for key, n in step:
            got[key].append(out[row:row + n].cpu())
            row, at[key] = row + n, at[key] + n
    for key in inputs:
        assert at[key] == len(inputs[key])
        close(torch.cat(got[key]), want[key], dtype, f32=3e-5, bf16=3e-2)
    # stored instead of added: the same rows over whatever the buffer held
    request = harness.cache.admit("d")
    ctx = harness.context([(request, [0] * 9)])
    out = torch.full((9, width), 7.0, dtype=torch.float32, device="cuda")
    part.forward(ctx, inputs["c"][:9].to(dtype).cuda(), out, harness.cache.layer_caches[0], accumulate=False)
    close(out, want["c"][:9], dtype, f32=3e-5, bf16=3e-2)


def answering(w, heads, d, r, width):
    """Edits a latent mixer's weights so that a token's plain query is the (unnormalised) plain key of the token whose input
    is its own with the two halves of the stream swapped: the latent norm's weight is 1, a head's key is the first d latent
    values, its plain query rows are the first d rows of the down projection behind a swap of the halves, and its rotated
    query rows are zero.  The matched score is about d times the scale, every other one a random number of size sqrt(d)."""
    down = w["dkv_proj.weight"]
    w["dkv_norm.weight"] = torch.ones_like(w["dkv_norm.weight"])
    swapped = torch.cat((down[:d, width // 2:], down[:d, :width // 2]), 1)
    q = torch.zeros_like(w["q_proj.weight"])
    for h in range(heads):
        q[h * (d + r):h * (d + r) + d] = swapped
    w["q_proj.weight"] = q
    eye = torch.zeros_like(w["uk_proj.weight"]).view(heads, d, -1)
    for h in range(heads):
        eye[h, :, :d] = torch.eye(d, dtype=eye.dtype)
    w["uk_proj.weight"] = eye.view(heads * d, -1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("planted,last", [(0, 699), (3, 512), (255, 256), (256, 700), (15, 16), (16, 17), (400, 401), (127, 640), (128, 640)])
def test_a_far_key_is_found_among_hundreds(dtype, planted, last):
    """The last token's query answers one planted position's key and no other: its output is that position's value, which
    no other position holds.  The key is planted at the very start, far back, at the edges of pages and of the kernels' key
    tiles, and right before the query; most of the prompt comes whole, the last tokens one by one."""
    width, heads, d, r, e, c = 64, 2, 64, 8, 12, 80
    part, w, m = latent_part(width, heads, d, r, e, c, 1.0, {"base": 10000.0, "dims": r}, dtype, seed=11, edit=lambda w: answering(w, heads, d, r, width))
    x = bf16_values(last + 1, width, seed=50)
    x[planted] = torch.cat((x[last, width // 2:], x[last, :width // 2]))
    shares = []
    want = plain.latent_attention(x, w, m, 1e-5, shares)
    for h, i, share in shares:
        if i == last:
            assert float(share[planted]) > 0.95                      # the planted key takes the weight
    harness = PartHarness([part.cache_need()], dtype, max_step_tokens=768)
    request = harness.cache.admit("a")
    head = max(1, last - 5)
    rows = []
    for first, n in [(0, head)] + [(i, 1) for i in range(head, last + 1)]:
        ctx = harness.context([(request, [0] * n)])
        out = torch.zeros(n, width, dtype=torch.float32, device="cuda")
        part.forward(ctx, x[first:first + n].to(dtype).cuda(), out, harness.cache.layer_caches[0])
        rows.append(out.cpu())
    close(torch.cat(rows)[last], want[last], dtype, f32=3e-5, bf16=4e-2)
    # and as the last token of a portion of two, behind the rest in one step, in the pages that the first request gives back
    harness.cache.release(request)
    other = harness.cache.admit("b")
    for first, n in ((0, last - 1), (last - 1, 2)):
        ctx = harness.context([(other, [0] * n)])
        out = torch.zeros(n, width, dtype=torch.float32, device="cuda")
        part.forward(ctx, x[first:first + n].to(dtype).cuda(), out, harness.cache.layer_caches[0])
    close(out[-1], want[last], dtype, f32=3e-5, bf16=4e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_sink_that_takes_weight(dtype):
    """Sinks well above and well below the scores: leaving the sink out, counting it twice, or scaling it with the scores
    would show in every row."""
    width, heads, d, r, e, c = 64, 2, 16, 8, 12, 24

    def edit(w):
        w["sink"] = torch.tensor([4.0, -3.0], dtype=torch.float64)

    part, w, m = latent_part(width, heads, d, r, e, c, 1.5, {"base": 50.0, "dims": r}, dtype, seed=21, edit=edit)
    x = bf16_values(300, width, seed=60)
    want = plain.latent_attention(x, w, m, 1e-5)
    without = plain.latent_attention(x, dict(w, sink=torch.full((2,), -80.0, dtype=torch.float64)), m, 1e-5)
    assert (without - want).norm() > 0.05 * want.norm()
    harness = PartHarness([part.cache_need()], dtype, max_step_tokens=320)
    request = harness.cache.admit("a")
    rows = []
    for first, n in [(0, 290)] + [(i, 1) for i in range(290, 300)]:
        ctx = harness.context([(request, [0] * n)])
        out = torch.zeros(n, width, dtype=torch.float32, device="cuda")
        part.forward(ctx, x[first:first + n].to(dtype).cuda(), out, harness.cache.layer_caches[0])
        rows.append(out.cpu())
    close(torch.cat(rows), want, dtype, f32=3e-5, bf16=4e-2)


def test_soft_cap_of_the_logits():
    from llm_runtime_study_amd.parts import PartSpec, create

    part = create("transform", PartSpec("soft_cap", {"cap": 7.5}))
    x = 20 * torch.randn(5, 333)
    got = x.clone().cuda()
    part.forward(None, got)
    torch.testing.assert_close(got.cpu().double(), 7.5 * torch.tanh(x.double() / 7.5), rtol=1e-5, atol=1e-5)
    assert got.abs().max() <= 7.5


# ------------------------------------------------------------------------------------- whole models
LENGTHS = {"mixed": [1, 5, 23, 64, 97, 130, 33, 16], "plain": [2, 17, 48, 65, 150, 31, 9], "cores": [3, 40, 64, 129, 210, 18]}
RAW = {"mixed": configs.MIXED, "plain": configs.PLAIN, "cores": configs.CORES}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for number, (name, raw) in enumerate(RAW.items()):
        folder = configs.write_folder(raw, 60 + number, tmp_path_factory.mktemp(f"napizen_{name}"))
        _, weights = plain.load_model_dir(folder)
        rng = np.random.default_rng(21 + number)
        requests = {f"{name}{i}": rng.integers(0, raw["vocab"], n).tolist() for i, n in enumerate(LENGTHS[name])}
        want = {key: plain.forward(weights, raw, tokens) for key, tokens in requests.items()}
        out[name] = (folder, raw, requests, want)
    return out


def check(got, want, dtype):
    """float32: every row closely (see tests/test_replay_gpu.py: compare).  bfloat16: experts are chosen, and a choice that
    falls the other way (a whole group of experts, in places) changes a row as a whole and every row of that request behind it: at
    least 85 of 100 rows within 3 %, none unrelated to the plain row."""
    if dtype == "float32":
        return compare(got, want, dtype)
    errors = np.array([float((row.double() - want[key][position]).norm() / want[key][position].norm())
                       for key, rows in got.items() for position, row in rows.items()])
    close_rows = np.mean(errors < 3e-2)
    assert close_rows >= 0.85 and errors.max() < 1.0, f"{close_rows:.2f} of the rows are close, the worst is off by {errors.max():.3g}"
    return len(errors)


def test_the_stream_after_every_layer(models):
    """float32, one prompt whole: the residual stream behind each layer against the plain implementation's."""
    from llm_runtime_study_amd.engine import trace
    from llm_runtime_study_amd.engine.step import StepEntry

    folder, raw, requests, _ = models["mixed"]
    _, weights = plain.load_model_dir(folder)
    tokens = requests["mixed4"]
    streams = []
    plain.forward(weights, raw, tokens, streams)
    runner = trace.make_runner(folder, "float32", 128)
    runner.use_plans = False
    kept = []
    for layer in runner.model.layers:
        def watched(ctx, h, cache, given=None, inner=layer.forward):
            out = inner(ctx, h, cache, given=given)
            kept.append(h.clone())
            return out
        layer.forward = watched
    request = runner.cache.admit("a")
    runner.step([StepEntry(request, tokens, [0])])
    assert len(kept) == len(streams)
    for got, want in zip(kept, streams):
        torch.testing.assert_close(got.cpu().double(), want, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(RAW))
def test_whole_then_last_tokens_one_by_one_then_portions(models, name, dtype, tmp_path):
    folder, raw, requests, want = models[name]
    longest = max(round64(len(t)) for t in requests.values())
    steps = traces.whole(requests)
    got = traces.collect(steps, run_replay(folder, dtype, steps, longest, tmp_path / "whole"), raw["vocab"])
    assert check(got, want, dtype) == sum(len(t) for t in requests.values())
    steps = traces.prefill_then_decode(requests, tail=40)
    check(traces.collect(steps, run_replay(folder, dtype, steps, longest, tmp_path / "tail"), raw["vocab"]), want, dtype)
    steps = traces.portions(requests)
    check(traces.collect(steps, run_replay(folder, dtype, steps, longest, tmp_path / "portions", page_size=32), raw["vocab"]), want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,seed", [("mixed", 0), ("mixed", 1), ("plain", 2), ("cores", 3)])
def test_mixed_steps_with_pages_and_slots_used_again(models, name, seed, dtype, tmp_path):
    folder, raw, requests, want = models[name]
    budget = 2 * max(round64(len(t)) for t in requests.values())
    steps, peak = traces.mixed(requests, seed=seed, max_live=4, max_tokens=budget)
    assert max(len(s["entries"]) for s in steps) >= 3
    got = traces.collect(steps, run_replay(folder, dtype, steps, peak, tmp_path), raw["vocab"])
    assert check(got, want, dtype) > 50
    assert peak < sum(round64(len(t)) for t in requests.values())


@pytest.mark.parametrize("name", ["mixed", "cores"])
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


def test_cuts_change_no_bit_in_float32(models, tmp_path):
    folder, raw, requests, _ = models["mixed"]
    a, b = traces.whole(requests), traces.portions(requests)
    ga = traces.collect(a, run_replay(folder, "float32", a, 192, tmp_path / "w"), raw["vocab"])
    gb = traces.collect(b, run_replay(folder, "float32", b, 192, tmp_path / "p"), raw["vocab"])
    for key in ga:
        for position in ga[key]:
            assert torch.equal(ga[key][position], gb[key][position]), f"{key}@{position}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_wider_model_through_the_products_for_many_rows(tmp_path, dtype):
    """Width 512 and prompts of 330 and 140 tokens: the projections of a prompt are products of hundreds of rows (the
    vendor library's in bfloat16), the experts get dozens to hundreds of rows each (large tiles)."""
    raw = configs.WIDE
    folder = configs.write_folder(raw, 31, tmp_path / "wide")
    _, weights = plain.load_model_dir(folder)
    rng = np.random.default_rng(4)
    requests = {"long": rng.integers(0, raw["vocab"], 330).tolist(), "short": rng.integers(0, raw["vocab"], 140).tolist()}
    want = {key: plain.forward(weights, raw, tokens) for key, tokens in requests.items()}
    steps = [{"step": 0, "entries": [{"id": key, "tokens": tokens[:-6], "want": list(range(0, len(tokens) - 6, 7))} for key, tokens in requests.items()], "end": []}]
    for i in range(6, 0, -1):
        steps.append({"step": len(steps), "entries": [{"id": key, "tokens": [tokens[-i]], "want": [0]} for key, tokens in requests.items()],
                      "end": list(requests) if i == 1 else []})
    got = traces.collect(steps, run_replay(folder, dtype, steps, 512, tmp_path / "o"), raw["vocab"])
    assert check(got, want, dtype) > 70


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_layer_without_feed_forward_whose_second_norm_is_stored(tmp_path, dtype):
    """Such a layer has no second update, and folders of random weights hold no second norm for it.  A checkpoint that holds
    one all the same is taken to mean h = norm2(alpha * h): both kinds of folder against the plain implementation."""
    raw = configs.MIXED

    def edit(tensors):
        tensors["l2.norm2"] = (tensors["l2.norm1"].float() * 0.7 + 0.4).to(torch.bfloat16)

    rng = np.random.default_rng(13)
    requests = {"p": rng.integers(0, raw["vocab"], 70).tolist(), "q": rng.integers(0, raw["vocab"], 33).tolist()}
    rows = {}
    for name, change in (("without", None), ("with", edit)):
        folder = configs.write_folder(raw, 71, tmp_path / name, change)
        _, weights = plain.load_model_dir(folder)
        assert ("l2.norm2" in weights) == (change is not None)
        want = {key: plain.forward(weights, raw, tokens) for key, tokens in requests.items()}
        steps = traces.portions(requests, sizes=(9, 2, 30, 1, 1))
        got = traces.collect(steps, run_replay(folder, dtype, steps, 128, tmp_path / f"o_{name}"), raw["vocab"])
        check(got, want, dtype)
        rows[name] = want["p"][-1]
    assert (rows["with"] - rows["without"]).norm() > 0.05 * rows["without"].norm()      # the stored norm matters


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(models, dtype, tmp_path):
    """A prompt of 20 tokens and 300 more one by one, beside a second request that starts later."""
    folder, raw, _, _ = models["mixed"]
    _, weights = plain.load_model_dir(folder)
    rng = np.random.default_rng(9)
    requests = {"x": rng.integers(0, raw["vocab"], 320).tolist(), "y": rng.integers(0, raw["vocab"], 150).tolist()}
    want = {key: plain.forward(weights, raw, tokens) for key, tokens in requests.items()}
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": requests["x"][:20], "want": [19]}], "end": []}]
    for i in range(20, 320):
        entries = [{"id": "x", "tokens": [requests["x"][i]], "want": [0]}]
        if i >= 170:
            entries.append({"id": "y", "tokens": [requests["y"][i - 170]], "want": [0]})
        steps.append({"step": len(steps), "entries": entries, "end": ["x", "y"] if i == 319 else []})
    got = traces.collect(steps, run_replay(folder, dtype, steps, 512, tmp_path / "o"), raw["vocab"])
    assert check(got, want, dtype) == 1 + 300 + 150


# ------------------------------------------------------------------------------------- generation
def test_greedy_generation_through_engine_and_scheduler(models):
    """Three prompts on two slots (the third waits and takes a freed slot and its pages), prompts fed in portions of at most
    16 tokens beside decoding requests: the tokens are the plain implementation's own greedy continuation."""
    from llm_runtime_study_amd import Engine

    folder, raw, requests, _ = models["plain"]
    _, weights = plain.load_model_dir(folder)
    prompts = [requests["plain1"], requests["plain2"][:30], requests["plain0"]]
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
    folder, raw, requests, want = models["mixed"]
    _, weights = plain.load_model_dir(folder)
    prompt = requests["mixed2"]
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
