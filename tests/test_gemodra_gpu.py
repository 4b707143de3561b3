"""Gemodra through the engine against the plain implementation (``plain_gemodra.py``,
float64, whole sequences, one function per mechanism, keys and values of every head formed
from the latent vectors).

float32 runs are held to the plain logits row by row (root mean square of the difference
over the vocabulary, means taken off, relative to the logits' own spread); every schedule,
cut and batch is held to the same bound.  A bfloat16 run chooses experts from a rounded
input: where two choice scores are closer than that rounding a token goes to another expert
than in float64, and the test weights are drawn with routers far from flat on purpose, so
single rows may differ visibly (measured: one row in some hundreds, by as much as the
logits' own spread).  bfloat16 rows are therefore held to the plain logits by their median
and their ninth decile, and only a few in a hundred may be far off; and how a bfloat16
request was cut and batched must not show beyond rounding: every schedule is held to the
whole prompts' run in the same way."""

import copy
import math

import pytest
import torch

import engine_util as eu
import gemodra_util as gu
import plain_gemodra as plain

pytestmark = pytest.mark.gpu

F32_BOUND = 1e-4
BF16_MEDIAN, BF16_DECILE = 0.04, 0.12
BF16_FAR, BF16_FAR_SHARE = 0.3, 0.03          # rows further off than this, and how many may be
BF16_BETWEEN_MEDIAN, BF16_BETWEEN_DECILE = 0.02, 0.06


def build(cfg, seed=0, dtype="float32", tensors=None):
    from zig_ai_amd.engine import DecoderModel
    d, tensors = gu.folder(cfg, seed, tensors)
    return DecoderModel.from_folder(d, dtype), tensors


def runner_for(model, page_size=4, tokens=256, slots=4, graphs=True):
    from zig_ai_amd.engine import ModelRunner
    return ModelRunner(model, page_size=page_size, num_pages=max(1, -(-tokens // page_size)),
                       num_slots=slots, use_graphs=graphs)


def plain_logits(cfg, tensors, prompts):
    return [plain.forward(cfg, tensors, p).float() for p in prompts]


def worst(got, want):
    return float(gu.row_error(got, want).max())


def assert_bfloat16_close(got, want, what=None):
    e = gu.row_error(got, want)
    found = (float(e.median()), float(e.quantile(0.9)), float((e > BF16_FAR).double().mean()))
    assert found[0] < BF16_MEDIAN and found[1] < BF16_DECILE and found[2] <= BF16_FAR_SHARE, \
        (what, found)


def assert_bfloat16_same_run(got, base, what=None):
    e = gu.row_error(got, base)
    found = (float(e.median()), float(e.quantile(0.9)))
    assert found[0] < BF16_BETWEEN_MEDIAN and found[1] < BF16_BETWEEN_DECILE, (what, found)


# ----------------------------------------------------------- each mechanism alone
SMALL = gu.plain_latent(heads=2, dim=8, vdim=8, kv_rank=16, q_rank=8)
ALONE = {
    "rotated": gu.one_layer("latent_attention", gu.latent(), side=0, softcap=0.0),
    "rotated, a part of the part turned": gu.one_layer(
        "latent_attention", gu.latent(heads=2, dim=24, vdim=8, kv_rank=40, q_rank=16, rot_dim=16,
                                      rot_dims=6, base=40.0), side=0, softcap=0.0),
    "rotated, one head, two rotated elements": gu.one_layer(
        "latent_attention", gu.latent(heads=1, dim=40, vdim=48, kv_rank=24, q_rank=8, rot_dim=2),
        side=0, softcap=0.0),
    "rotated, many heads": gu.one_layer(
        "latent_attention", gu.latent(heads=40, dim=8, vdim=8, kv_rank=72, q_rank=16, rot_dim=8),
        side=0, softcap=0.0, width=64),
    "unrotated": gu.one_layer("latent_attention_2", gu.plain_latent(), side=0, softcap=0.0),
    "unrotated, one head": gu.one_layer("latent_attention_2", gu.plain_latent(
        heads=1, dim=16, vdim=40, kv_rank=8, q_rank=32), side=0, softcap=0.0),
    "unrotated, a wide latent": gu.one_layer("latent_attention_2", gu.plain_latent(
        heads=3, dim=16, vdim=16, kv_rank=320, q_rank=16), side=0, softcap=0.0, width=64),
    "experts in groups": gu.one_layer("latent_attention_2", SMALL, gu.moe(
        ff=16, experts=9, identity=3, top=3, groups=(4, 2), shared=0), side=0, softcap=0.0),
    "experts, no groups, a shared one": gu.one_layer("latent_attention_2", SMALL, gu.moe(
        ff=24, experts=5, identity=0, top=2, shared=40), side=0, softcap=0.0),
    "all outputs chosen": gu.one_layer("latent_attention_2", SMALL, gu.moe(
        ff=8, experts=2, identity=1, top=3, shared=0, scale=0.7), side=0, softcap=0.0),
    "identity outputs only": gu.one_layer("latent_attention_2", SMALL, gu.moe(
        experts=0, identity=4, top=2, groups=(2, 1), shared=8), side=0, softcap=0.0),
    "one group kept": gu.one_layer("latent_attention_2", SMALL, gu.moe(
        ff=16, experts=6, identity=2, top=2, groups=(4, 1), shared=0), side=0, softcap=0.0),
    "token input": gu.one_layer("latent_attention_2", SMALL, None, side=12, softcap=0.0),
    "capped logits": gu.one_layer("latent_attention_2", SMALL, None, side=0, softcap=1.5),
}


@pytest.mark.parametrize("name", sorted(ALONE))
def test_mechanism_alone(name):
    cfg = ALONE[name]
    model, tensors = build(cfg, seed=3)
    prompts = [gu.tokens(70, cfg["vocab"], 1), gu.tokens(5, cfg["vocab"], 2)]
    want = plain_logits(cfg, tensors, prompts)
    runner = runner_for(model)
    got = eu.run_schedule(runner, prompts, eu.whole([len(p) for p in prompts]))
    for g, w in zip(got, want):
        assert worst(g, w) < F32_BOUND
    # the same, token by token from the first token on: the cache alone
    got = eu.run_schedule(runner, prompts, eu.bulk_then_single([len(p) for p in prompts], tail=10 ** 6))
    for g, w in zip(got, want):
        assert worst(g, w) < F32_BOUND


def test_every_mechanism_counts():
    """The plain implementation without one mechanism is far from the one with it: the
    weights make each of them visible, so the comparisons above can fail."""
    cfg = gu.TINY_ALL
    tensors = gu.make_tensors(cfg, seed=3)
    prompt = gu.tokens(40, cfg["vocab"], 1)
    want = plain.forward(cfg, tensors, prompt).float()

    def changed(edit_cfg=None, edit_tensors=None):
        c, t = copy.deepcopy(cfg), dict(tensors)
        if edit_cfg:
            edit_cfg(c)
        if edit_tensors:
            edit_tensors(t)
        return worst(plain.forward(c, t, prompt).float(), want)

    def no_sink(t):
        for i in range(4):
            t[f"l{i}.mix.sink"] = torch.full_like(t[f"l{i}.mix.sink"], -60.0)

    def no_correction(t):
        for i in (0, 1, 3):
            t[f"l{i}.mlp.correction"] = torch.zeros_like(t[f"l{i}.mlp.correction"])

    def no_groups(c):
        for i in (0, 3):
            del c["layers"][i]["mlp"]["router"]["groups"]

    def no_side(c):
        del c["token_side"]

    def no_cap(c):
        del c["logit_softcap"]

    def other_base(c):
        c["layers"][0]["mixer"]["rot"]["base"] = 3000.0

    def no_shared_gate(t):
        t["l0.mlp.shared.sg"] = torch.zeros_like(t["l0.mlp.shared.sg"])

    def no_embed_norm(t):
        t["embed.norm"] = torch.ones_like(t["embed.norm"])

    for name, kw in (("sink", {"edit_tensors": no_sink}), ("correction", {"edit_tensors": no_correction}),
                     ("groups", {"edit_cfg": no_groups}), ("token input", {"edit_cfg": no_side}),
                     ("cap", {"edit_cfg": no_cap}), ("base", {"edit_cfg": other_base}),
                     ("shared gate", {"edit_tensors": no_shared_gate}),
                     ("embedding norm", {"edit_tensors": no_embed_norm})):
        assert changed(**kw) > 0.02, name


# ------------------------------- sizes that are multiples of nothing the kernels like
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_awkward_sizes(dtype):
    cfg = gu.config([
        gu.layer("latent_attention", gu.latent(heads=3, dim=12, vdim=20, kv_rank=28, q_rank=12,
                                               rot_dim=6, base=77.0),
                 gu.moe(ff=20, experts=7, identity=2, top=3, groups=(3, 2), shared=12)),
        gu.layer("latent_attention_2", gu.plain_latent(heads=7, dim=10, vdim=6, kv_rank=18, q_rank=14),
                 gu.moe(ff=12, experts=2, identity=0, top=1, shared=0)),
        gu.layer("latent_attention", gu.latent(heads=70, dim=8, vdim=8, kv_rank=16, q_rank=24,
                                               rot_dim=8), None),
    ], width=36, vocab=53, side=6, softcap=9.0, mult=0.7)
    model, tensors = build(cfg, seed=17, dtype=dtype)
    lengths = [50, 3, 21]
    prompts = [gu.tokens(n, cfg["vocab"], 30 + i) for i, n in enumerate(lengths)]
    want = plain_logits(cfg, tensors, prompts)
    base = None
    for name, schedule in (("whole", eu.whole(lengths)),
                           ("portions", eu.changing_portions(lengths, seed=2)),
                           ("mixed", eu.mixed(lengths, seed=3, max_live=3, decode_tail=8))):
        got = eu.run_schedule(runner_for(model, page_size=8, tokens=128, slots=3), prompts, schedule)
        if dtype == "float32":
            for g, w in zip(got, want):
                assert worst(g, w) < F32_BOUND, name
        else:
            assert_bfloat16_close(torch.cat(got), torch.cat(want), name)
            base = base or got
            assert_bfloat16_same_run(torch.cat(got), torch.cat(base), name)


# -------------------------------------------------------- schedules of whole models
LENGTHS = [150, 37, 9, 1, 75, 130, 2]


def schedules(lengths):
    return {
        "whole": eu.whole(lengths),
        "bulk + tail": eu.bulk_then_single(lengths, tail=40),
        "portions": eu.changing_portions(lengths, seed=1),
        "portions of two": eu.changing_portions(lengths, seed=0, sizes=(2, 2, 3, 2, 17)),
        "mixed": eu.mixed(lengths, seed=2, max_live=4, decode_tail=20),
        "mixed, three live": eu.mixed(lengths, seed=5, max_live=3, decode_tail=45),
    }


@pytest.mark.parametrize("which", ["all", "other"])
@pytest.mark.parametrize("page_size", [4, 16])
def test_schedules_float32(which, page_size):
    cfg = gu.TINY_ALL if which == "all" else gu.TINY_OTHER
    model, tensors = build(cfg, seed=11)
    prompts = [gu.tokens(n, cfg["vocab"], 20 + i) for i, n in enumerate(LENGTHS)]
    want = plain_logits(cfg, tensors, prompts)
    for name, schedule in schedules(LENGTHS).items():
        # a pool for the most tokens live at any time: pages are used again
        peak = eu.peak_tokens(LENGTHS, schedule, round_to=max(16, page_size))
        runner = runner_for(model, page_size=page_size, tokens=peak, slots=4)
        got = eu.run_schedule(runner, prompts, schedule)
        for i, (g, w) in enumerate(zip(got, want)):
            assert worst(g, w) < F32_BOUND, (name, i)
        if "mixed" in name:
            assert runner.cache.pages_reused > 0
        assert len(runner.cache.requests) == 0


@pytest.mark.parametrize("which", ["all", "other"])
def test_schedules_bfloat16(which):
    cfg = gu.TINY_ALL if which == "all" else gu.TINY_OTHER
    model, tensors = build(cfg, seed=11, dtype="bfloat16")
    prompts = [gu.tokens(n, cfg["vocab"], 20 + i) for i, n in enumerate(LENGTHS)]
    want = plain_logits(cfg, tensors, prompts)
    base = None
    for name, schedule in schedules(LENGTHS).items():
        peak = eu.peak_tokens(LENGTHS, schedule, round_to=16)
        runner = runner_for(model, page_size=16, tokens=peak, slots=4)
        got = eu.run_schedule(runner, prompts, schedule)
        assert_bfloat16_close(torch.cat(got), torch.cat(want), name)
        if base is None:
            base = got
        assert_bfloat16_same_run(torch.cat(got), torch.cat(base), name)


# ------------------------------------------------ configurations drawn at random
@pytest.mark.parametrize("seed", range(10))
def test_random_configurations(seed):
    cfg = gu.random_config(seed)
    lengths = [70, 1, 33, 12, 2]
    prompts = [gu.tokens(n, cfg["vocab"], 90 + i) for i, n in enumerate(lengths)]
    model, tensors = build(cfg, seed=seed)
    want = plain_logits(cfg, tensors, prompts)
    for name, schedule in (("whole", eu.whole(lengths)),
                           ("portions", eu.changing_portions(lengths, seed=seed)),
                           ("mixed", eu.mixed(lengths, seed=seed, max_live=3, decode_tail=9))):
        peak = eu.peak_tokens(lengths, schedule, round_to=16)
        runner = runner_for(model, page_size=4 if seed % 2 else 16, tokens=peak, slots=3)
        got = eu.run_schedule(runner, prompts, schedule)
        for i, (g, w) in enumerate(zip(got, want)):
            assert worst(g, w) < 3 * F32_BOUND, (name, i, cfg)
    # the same model in bfloat16 runs (odd widths fall back to 32-bit weights) and agrees
    # with itself across schedules
    model16, _ = build(cfg, seed=seed, dtype="bfloat16")
    base = None
    for schedule in (eu.whole(lengths), eu.mixed(lengths, seed=seed, max_live=3, decode_tail=9)):
        got = eu.run_schedule(runner_for(model16, page_size=16, tokens=256, slots=3), prompts, schedule)
        assert all(torch.isfinite(g).all() for g in got)
        base = base or got
        assert_bfloat16_same_run(torch.cat(got), torch.cat(base), cfg)


# --------------------------------- the causal edge, with scores that stand out
def sharp_cfg(kind):
    # a scale that makes the softmax all but choose one key: a key wrongly seen or wrongly
    # hidden then takes or loses nearly all of a query's weight
    mixer = gu.latent(heads=2, dim=16, vdim=16, kv_rank=24, q_rank=16, rot_dim=8, base=100.0,
                      scale=3.0) if kind == "latent_attention" else \
        gu.plain_latent(heads=2, dim=16, vdim=16, kv_rank=24, q_rank=16, scale=3.0)
    return gu.one_layer(kind, mixer, None, side=0, softcap=0.0)


def plain_with_reach(cfg, tensors, prompt, reach):
    """The plain model with every query seeing one key fewer (-1: not itself) or one more
    (+1: its successor too) than it should."""
    real = plain.latent_attention
    plain.latent_attention = lambda *a, **k: real(*a, reach=reach, **k)
    try:
        return plain.forward(cfg, tensors, prompt).float()
    finally:
        plain.latent_attention = real


@pytest.mark.parametrize("kind", ["latent_attention", "latent_attention_2"])
def test_causal_edge(kind):
    cfg = sharp_cfg(kind)
    model, tensors = build(cfg, seed=5)
    n = 90
    prompts = [gu.tokens(n, cfg["vocab"], 7)]
    want = plain_logits(cfg, tensors, prompts)[0]
    # the test can see an edge that is one token off
    for reach in (-1, 1):
        assert worst(plain_with_reach(cfg, tensors, prompts[0], reach), want) > 0.05
    for page_size in (4, 16):
        for name, schedule in (("whole", eu.whole([n])),
                               ("decoded", eu.bulk_then_single([n], tail=n - 3)),
                               ("portions", eu.changing_portions([n], sizes=(5, 2, 16, 3, 17, 15, 1)))):
            runner = runner_for(model, page_size=page_size, tokens=128)
            got = eu.run_schedule(runner, prompts, schedule)[0]
            assert worst(got, want) < 1e-3, (name, page_size)


# ----------------------------------------------------------------- far tokens count
def far_prompt(cfg, tensors, n, place):
    """A prompt of ``n`` tokens and the same with another token at ``place``, made so that the
    last rows of the plain logits differ clearly: the body repeats three ids, the token at
    ``place`` occurs nowhere else, and the last eight tokens are one id whose queries it
    draws (both found by trying the ids kept aside for this)."""
    V = cfg["vocab"]
    body = [t % 3 for t in gu.tokens(n, V, 3)]
    best = None
    for tail in range(V - 16, V - 8):
        for cand in range(V - 8, V):
            a = list(body)
            a[-8:] = [tail] * 8
            b = list(a)
            a[place] = cand
            wa, wb = plain.forward(cfg, tensors, a).float(), plain.forward(cfg, tensors, b).float()
            d = worst(wb[-8:], wa[-8:])
            if best is None or d > best[0]:
                best = (d, a, b, wa, wb)
            if d > 0.1:
                return best
    return best


@pytest.mark.parametrize("kind", ["latent_attention", "latent_attention_2"])
def test_far_tokens_reach_the_end(kind):
    cfg = sharp_cfg(kind)
    tensors = gu.make_tensors(cfg, seed=9)
    tensors["l0.mix.sink"] = torch.full_like(tensors["l0.mix.sink"], -4.0)
    model, tensors = build(cfg, tensors=tensors)
    n = 600
    d, a, b, wa, wb = far_prompt(cfg, tensors, n, place=1)
    assert d > 0.02           # the second token still shows at the end, among hundreds
    for prompt, want in ((a, wa), (b, wb)):
        for page_size, schedule in ((16, eu.whole([n])), (4, eu.bulk_then_single([n], tail=40)),
                                    (16, eu.changing_portions([n], sizes=(33, 2, 64, 17, 200)))):
            got = eu.run_schedule(runner_for(model, page_size=page_size, tokens=640), [prompt],
                                  schedule)[0]
            assert worst(got, want) < F32_BOUND
    # nothing is left of a request whose pages are taken again: b after a in the same pool
    runner = runner_for(model, page_size=16, tokens=640, slots=1)
    for prompt, want in ((a, wa), (b, wb), (a, wa)):
        got = eu.run_schedule(runner, [prompt], eu.bulk_then_single([n], tail=5))[0]
        assert worst(got, want) < F32_BOUND
    assert runner.cache.pages_reused > 0


# --------------------------------------------------------------------- the sink
@pytest.mark.parametrize("kind", ["latent_attention", "latent_attention_2"])
def test_sinks_that_take_most_of_the_weight(kind):
    cfg = sharp_cfg(kind)
    cfg["layers"][0]["mixer"]["scale"] = 0.2
    tensors = gu.make_tensors(cfg, seed=2)
    tensors["l0.mix.sink"] = torch.tensor([3.0, -1.0])
    model, tensors = build(cfg, tensors=tensors)
    lengths = [60, 3]
    prompts = [gu.tokens(n, cfg["vocab"], 4 + i) for i, n in enumerate(lengths)]
    want = plain_logits(cfg, tensors, prompts)
    # a sink that is scaled like a score, or given to the other head, shows
    for other in (torch.tensor([3.0 * 0.2, -0.2]), torch.tensor([-1.0, 3.0])):
        t2 = dict(tensors)
        t2["l0.mix.sink"] = other
        assert worst(plain.forward(cfg, t2, prompts[0]).float(), want[0]) > 0.02
    for schedule in (eu.whole(lengths), eu.bulk_then_single(lengths, tail=30),
                     eu.changing_portions(lengths, sizes=(2, 7, 16))):
        got = eu.run_schedule(runner_for(model), prompts, schedule)
        for g, w in zip(got, want):
            assert worst(g, w) < F32_BOUND


# -------------------------- a long context: ranges of keys, merged, with the sink once
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_context_in_ranges(dtype):
    from zig_ai_amd.kernels import ops
    cfg = gu.config([gu.layer("latent_attention", gu.latent(heads=2, dim=16, vdim=16, kv_rank=64,
                                                            q_rank=16, rot_dim=16, base=1e4), None),
                     gu.layer("latent_attention_2", gu.plain_latent(), None)], side=8)
    model, tensors = build(cfg, seed=4, dtype=dtype)
    n = 1500
    prompts = [gu.tokens(n, cfg["vocab"], 1), gu.tokens(30, cfg["vocab"], 2)]
    want = plain_logits(cfg, tensors, prompts)
    runner = runner_for(model, page_size=16, tokens=1600, graphs=False)
    wants = [list(range(n - 90, n)), list(range(30))]
    steps = [([(0, 0, n - 80)], [])]
    # the long request decodes beside the short one's portions and single tokens
    steps += [([(0, n - 80 + i, n - 79 + i)] + ([(1, 3 * i, 3 * i + 3)] if i < 10 else []),
               [1] if i == 9 else []) for i in range(80)]
    steps[-1] = (steps[-1][0], [0])
    ops.form_log = []
    try:
        got = eu.run_schedule(runner, prompts, steps, wants=wants)
        cut = [r for r in (ops.form_log or []) if r.get("op") == "attention" and r.get("nsplit", 1) > 1]
    finally:
        ops.form_log = None
    if dtype == "float32":
        assert worst(got[0], want[0][n - 90:]) < F32_BOUND
        assert worst(got[1], want[1]) < F32_BOUND
    else:
        assert_bfloat16_close(torch.cat(got), torch.cat([want[0][n - 90:], want[1]]))


# ------------------------------------------------------------------- long decoding
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype):
    cfg = gu.TINY_ALL
    model, tensors = build(cfg, seed=21, dtype=dtype)
    n = 330
    prompts = [gu.tokens(n, cfg["vocab"], 5)]
    want = plain_logits(cfg, tensors, prompts)[0]
    runner = runner_for(model, page_size=16, tokens=512)       # decode steps replay from graphs
    got = eu.run_schedule(runner, prompts, eu.bulk_then_single([n], tail=300))[0]
    if dtype == "float32":
        assert worst(got, want) < F32_BOUND
    else:
        assert_bfloat16_close(got, want)


# ------------------------------------------- unequal requests together and alone
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_batch_against_each_alone(dtype):
    cfg = gu.TINY_ALL
    model, tensors = build(cfg, seed=2, dtype=dtype)
    lengths = [64, 3, 41, 17]
    prompts = [gu.tokens(n, cfg["vocab"], 40 + i) for i, n in enumerate(lengths)]
    alone = eu.run_schedule(runner_for(model, tokens=256), prompts, eu.whole(lengths))
    together = [([(i, 0, n) for i, n in enumerate(lengths)], list(range(len(lengths))))]
    got = eu.run_schedule(runner_for(model, tokens=256), prompts, together)
    if dtype == "float32":
        assert worst(torch.cat(got), torch.cat(alone)) < F32_BOUND
    else:
        assert_bfloat16_same_run(torch.cat(got), torch.cat(alone))


# ----------------------------------- sizes at which the products run on the matrix cores
def test_wider_model_bfloat16():
    mixer = gu.latent(heads=8, dim=32, vdim=48, kv_rank=128, q_rank=96, rot_dim=32, base=1e5)
    cfg = gu.config([gu.layer("latent_attention", mixer, gu.moe(ff=64, experts=6, identity=2, top=3,
                                                                groups=(4, 2), shared=128)),
                     gu.layer("latent_attention_2", gu.plain_latent(heads=4, dim=64, vdim=32,
                                                                    kv_rank=256, q_rank=64),
                              gu.moe(ff=128, experts=8, identity=0, top=2, shared=0))],
                    width=256, vocab=300, side=32)
    model, tensors = build(cfg, seed=6, dtype="bfloat16")
    lengths = [200, 70, 3]
    prompts = [gu.tokens(n, cfg["vocab"], 50 + i) for i, n in enumerate(lengths)]
    want = plain_logits(cfg, tensors, prompts)
    base = None
    for name, schedule in (("whole", eu.whole(lengths)),
                           ("bulk + tail", eu.bulk_then_single(lengths, tail=60)),
                           ("portions", eu.changing_portions(lengths, seed=3)),
                           ("mixed", eu.mixed(lengths, seed=1, max_live=3, decode_tail=30))):
        runner = runner_for(model, page_size=16, tokens=512, slots=3)
        got = eu.run_schedule(runner, prompts, schedule)
        assert_bfloat16_close(torch.cat(got), torch.cat(want), name)
        base = base or got
        assert_bfloat16_same_run(torch.cat(got), torch.cat(base), name)


# ------------------------------------------- generation through engine and scheduler
def test_greedy_generation():
    from zig_ai_amd.engine import Engine
    cfg = gu.TINY_ALL
    d, tensors = gu.folder(cfg, seed=8)
    engine = Engine(d, dtype="float32", page_size=4, num_pages=128, max_num_seqs=3,
                    max_num_batched_tokens=48, chunk_size=20, max_model_len=256)
    prompts = [gu.tokens(n, cfg["vocab"], 60 + i) for i, n in enumerate([33, 5, 70, 12, 1])]
    outs = engine.generate(prompts, max_new_tokens=20, temperature=0.0)
    assert all(len(o) == 20 for o in outs)
    for p, o in zip(prompts, outs):
        # every chosen token is the plain implementation's choice for the same history
        logits = plain.forward(cfg, tensors, p + o)
        for j, tok in enumerate(o):
            row = logits[len(p) + j - 1]
            assert float(row.max() - row[tok]) <= 1e-3 * float(row.abs().max()), (j, tok)
    assert len(engine.runner.cache.requests) == 0
    engine.runner.cache.check()


def test_generation_bfloat16_runs_through_graphs():
    from zig_ai_amd.engine import Engine
    cfg = gu.TINY_OTHER
    d, tensors = gu.folder(cfg, seed=8)
    engine = Engine(d, dtype="bfloat16", page_size=16, num_pages=64, max_num_seqs=4,
                    max_model_len=256)
    assert engine.runner.graphs is not None        # every part can be recorded
    prompts = [gu.tokens(n, cfg["vocab"], 80 + i) for i, n in enumerate([40, 7, 19])]
    outs = engine.generate(prompts, max_new_tokens=24, temperature=0.0)
    assert all(len(o) == 24 for o in outs)
    good = total = 0
    for p, o in zip(prompts, outs):
        logits = plain.forward(cfg, tensors, p + o)
        for j, tok in enumerate(o):
            row = logits[len(p) + j - 1]
            spread = float(row.max() - row.min())
            good += float(row.max() - row[tok]) <= 0.1 * spread
            total += 1
    # (a token routed to another expert than in float64 may pick another word; rare)
    assert good >= 0.9 * total, (good, total)


def test_trace_replay_and_command_line(tmp_path):
    import json
    import os
    import subprocess
    import sys
    import numpy as np
    cfg = gu.TINY_ALL
    d, tensors = gu.folder(cfg, seed=8)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    prompt, other = gu.tokens(40, cfg["vocab"], 3), gu.tokens(11, cfg["vocab"], 4)
    want = plain.forward(cfg, tensors, prompt).float()
    want_other = plain.forward(cfg, tensors, other).float()
    # portions of one request beside another's, single tokens, a step in which nothing is asked
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": prompt[:25], "want": [3, 24]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": prompt[25:27], "want": []},
                                     {"id": "b", "tokens": other[:10], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": other[10:], "want": [0]},
                                     {"id": "a", "tokens": prompt[27:], "want": [12]}], "end": ["a", "b"]}]
    out = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", d,
                          "--dtype", "float32", "--out", str(tmp_path), "--max-tokens", "128"],
                         input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
                         capture_output=True, timeout=600)
    assert out.returncode == 0, out.stderr[-2000:]
    assert [l for l in out.stdout.split("\n") if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    first = torch.from_numpy(np.fromfile(tmp_path / "0.f32", dtype="<f4").reshape(2, -1))
    last = torch.from_numpy(np.fromfile(tmp_path / "2.f32", dtype="<f4").reshape(2, -1))
    assert not (tmp_path / "1.f32").exists()
    assert worst(torch.cat([first, last[1:]]), want[[3, 24, 39]]) < F32_BOUND
    assert worst(last[:1], want_other[[10]]) < F32_BOUND
    gen = subprocess.run([sys.executable, "-m", "zig_ai_amd", "--model", d, "--dtype", "float32",
                          "--prompt-ids", ",".join(map(str, prompt[:9])), "-n", "5",
                          "--temperature", "0", "--json"], cwd=root, text=True, capture_output=True,
                         timeout=600)
    assert gen.returncode == 0, gen.stderr[-2000:]
    outputs = json.loads(gen.stdout.strip().split("\n")[-1])["outputs"]
    assert len(outputs) == 1 and len(outputs[0]) == 5
    logits = plain.forward(cfg, tensors, prompt[:9] + outputs[0])
    for j, tok in enumerate(outputs[0]):
        row = logits[9 + j - 1]
        assert float(row.max() - row[tok]) <= 1e-3 * float(row.abs().max()), (j, tok)


# ------------------------------------------------------------------ kernels alone
def _route_plain(logits, correction, router):
    n = logits.shape[1]
    t = {"x.router": torch.eye(n, dtype=torch.float64), "x.correction": correction}
    return plain.route(logits.double(), t, "x.", router)


@pytest.mark.parametrize("n,top,groups,scale", [(12, 3, (4, 2), 1.5), (16, 4, (4, 3), 2.0),
                                                (7, 7, None, 1.0), (6, 1, (6, 1), 0.5),
                                                (64, 6, (8, 3), 1.0), (9, 2, (1, 1), 1.0),
                                                (300, 8, (10, 4), 2.5)])
def test_router_kernel(n, top, groups, scale):
    from zig_ai_amd.kernels import ops
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(n + top)
    T = 200
    # a few extra columns behind the router's outputs, as the shared expert's gate is
    logits = torch.randn(T, n + 3, generator=g) * 2.0
    router = {"top": top, "scale": scale}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    # corrections that push every choice score below zero in half of the cases: an output
    # that may not be chosen counts as minus infinity, not as zero
    for shift in (0.0, -3.0):
        correction = torch.randn(n, generator=g) * 0.2 + shift
        chosen, weight = ops.route_topk(logits.to(dev), n, top, correction.to(dev),
                                        groups[0] if groups else 0, groups[1] if groups else 0,
                                        scale, "softmax", False)
        want_c, want_w = _route_plain(logits[:, :n], correction.double(), router)
        got = {(t, int(e)): float(w) for t in range(T)
               for e, w in zip(chosen[t].cpu(), weight[t].cpu())}
        assert len(got) == T * top                      # a row's experts differ
        for t in range(T):
            for e, w in zip(want_c[t].tolist(), want_w[t].tolist()):
                assert (t, e) in got, (t, e, shift)
                assert abs(got[(t, e)] - w) < 1e-6 + 1e-5 * abs(w)


def _latent_attention_case(dtype, H, W, R, requests, page_size, per_item, seed):
    """A paged cache of rows ``[latent | rotated part]`` for ``requests`` = [(cached, new)],
    folded queries for the new tokens, the step's arrays, and what the attention should give
    (float64, with a sink a head)."""
    g = torch.Generator().manual_seed(seed)
    n_pages = sum(-(-(c + n) // page_size) for c, n in requests) + 3
    order = torch.randperm(n_pages, generator=g).tolist()
    plane = torch.zeros(n_pages, 1, page_size, W)
    most = max(-(-(c + n) // page_size) for c, n in requests)
    table = torch.full((len(requests), most + 1), -1, dtype=torch.int32)
    scale = 1.7 * W ** -0.5
    sink = torch.randn(H, generator=g) * 1.5
    qs, positions, items, want = [], [], [], []
    row = 0
    for s, (cached, new) in enumerate(requests):
        keys = (torch.randn(cached + new, W, generator=g)).to(dtype).float()
        for p in range(-(-(cached + new) // page_size)):
            page = order.pop()
            table[s, p] = page
            chunk = keys[p * page_size:(p + 1) * page_size]
            plane[page, 0, :chunk.shape[0]] = chunk
        q = torch.randn(new, H, W, generator=g).to(dtype).float()
        qs.append(q)
        positions += list(range(cached, cached + new))
        for a in range(0, new, per_item):
            items.append((s, row + a, min(per_item, new - a)))
        row += new
        for i in range(new):
            k = keys[:cached + i + 1].double()
            sc = torch.einsum("hw,jw->hj", q[i].double(), k) * scale
            top = torch.maximum(sc.max(dim=1, keepdim=True).values, sink.double()[:, None])
            e = torch.exp(sc - top)
            pr = e / (e.sum(dim=1, keepdim=True) + torch.exp(sink.double()[:, None] - top))
            want.append(pr @ k[:, :R])
    dev = torch.device("cuda")
    mk = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    return (torch.cat(qs).to(dtype).to(dev), plane.to(dtype).to(dev), table.to(dev), mk(positions),
            mk([i[0] for i in items]), mk([i[1] for i in items]), mk([i[2] for i in items]),
            len(items), scale, sink.to(dev), torch.stack(want))


@pytest.mark.parametrize("H,W,R,page_size", [(3, 40, 32, 4), (16, 576, 512, 16), (8, 160, 128, 16),
                                             (4, 96, 96, 16), (5, 48, 24, 8), (40, 80, 72, 16),
                                             (1, 264, 256, 32)])
def test_latent_attention_kernels(H, W, R, page_size):
    from zig_ai_amd.kernels import ops
    # prompt portions behind cached tokens, a first portion, single tokens, one token alone
    requests = [(70, 9), (0, 45), (133, 1), (0, 1), (31, 2)]
    for dtype, waves_list in ((torch.float32, (0,)), (torch.bfloat16, (0, 4))):
        for waves in waves_list:
            most = ops.LATENT_MFMA_ROWS if waves else ops.LATENT_MAX_ROWS
            per_item = max(1, most // min(H, most))
            q, plane, table, pos, iseq, irow, icnt, n, scale, sink, want = _latent_attention_case(
                dtype, H, W, R, requests, page_size, per_item, seed=H + W)
            for keys, nsplit in ((0, 1), (64, 3)):
                got = ops.latent_attention(q, plane, R, table, pos, iseq, irow, icnt, n, scale, sink,
                                           keys, nsplit, waves).cpu().double()
                tol = 2e-5 if dtype == torch.float32 else 2e-2
                assert float((got - want).abs().max()) < tol, (dtype, waves, nsplit)
    # single tokens only: a wave a workgroup
    requests = [(200, 1), (0, 1), (63, 1), (64, 1)]
    q, plane, table, pos, iseq, irow, icnt, n, scale, sink, want = _latent_attention_case(
        torch.bfloat16, H, W, R, requests, page_size, 1, seed=7)
    for keys, nsplit in ((0, 1), (64, 4), (128, 2)):
        got = ops.latent_attention(q, plane, R, table, pos, iseq, irow, icnt, n, scale, sink, keys,
                                   nsplit, 1).cpu().double()
        assert float((got - want).abs().max()) < 2e-2, nsplit


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,N,K,mode", [(3, 24, 16, None), (8, 128, 64, "element"), (5, 40, 32, "head"),
                                        (1, 8, 320, "element"), (40, 72, 8, None)])
def test_head_linear_kernel(dtype, H, N, K, mode):
    from zig_ai_amd.kernels import ops
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(H * N + K)
    T = 37
    x = torch.randn(T, H, K + 8, generator=g).to(dtype)
    w = (torch.randn(H, N, K, generator=g) * K ** -0.5).to(dtype)
    gate = torch.randn(T, 16 + (H if mode == "head" else H * N), generator=g).to(dtype)
    got = ops.head_linear(x.to(dev), 8, w.to(dev), gate=gate.to(dev) if mode else None, gate_col=16,
                          gate_mode=mode).cpu().double()
    want = torch.einsum("thk,hnk->thn", x[:, :, 8:].double(), w.double())
    if mode == "head":
        want = want * torch.sigmoid(gate[:, 16:].double())[:, :, None]
    elif mode == "element":
        want = want * torch.sigmoid(gate[:, 16:].double()).view(T, H, N)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert float((got - want).abs().max()) < tol * max(1.0, float(want.abs().max()))


def test_token_side_kernels():
    from zig_ai_amd.kernels import ops
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(1)
    T, dim, V, width = 19, 12, 50, 40
    gate = torch.randn(T, dim, generator=g) * 2
    table = torch.randn(V, 5 * dim, generator=g)
    ids = torch.randint(0, V, (T,), generator=g, dtype=torch.int32)
    got = ops.table_gate(gate.to(dev), ids.to(dev), table.to(dev), 3 * dim, "gelu_tanh").cpu().double()
    want = plain.gelu_tanh(gate.double()) * table.double()[ids.long()][:, 3 * dim:4 * dim]
    assert float((got - want).abs().max()) < 1e-5
    stream = torch.randn(T, width, generator=g)
    y = torch.randn(T, width, generator=g) * 3
    w = torch.randn(width, generator=g)
    res = stream.to(dev).clone()
    ops.normed_add_(res, y.to(dev), w.to(dev), 1e-3, 0.3)
    want = stream.double() + 0.3 * plain.rms_norm(y.double(), w.double(), 1e-3)
    assert float((res.cpu().double() - want).abs().max()) < 1e-5
    z = torch.randn(T, width, generator=g) * 20
    got = ops.softcap_(z.to(dev).clone(), 7.0).cpu().double()
    assert float((got - 7.0 * torch.tanh(z.double() / 7.0)).abs().max()) < 1e-5
