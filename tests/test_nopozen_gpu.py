"""Nopozen through the engine against the plain implementation (``plain_nopozen.py``,
float64, one function per mechanism).

float32 runs are held to the plain logits row by row (root mean square of the difference
over the vocabulary, relative to the logits' own spread): measured 1e-6 to 1e-5, bound
1e-4; every schedule, cut and batch is held to it.  bfloat16 rows are held to the plain
logits by their median, their ninth decile and the share of rows that are far off (the
weights here are drawn sharp on purpose, and a router whose two best logits lie within
rounding of each other sends a token to another expert: such a row is far off, and rows
behind it in a recurrent layer with it), and every schedule to the whole prompts' run: how a
request was cut and batched must not show beyond rounding."""

import pytest
import torch

import engine_util as eu
import nopozen_util as nu
import plain_nopozen as plain

pytestmark = pytest.mark.gpu

F32_BOUND = 1e-4
BF16_MEDIAN, BF16_DECILE, BF16_WORST = 0.04, 0.1, 0.5
BF16_FAR_SHARE = 0.03            # of rows beyond BF16_WORST
BF16_BETWEEN_MEDIAN, BF16_BETWEEN_WORST = 0.02, 0.2


def build(cfg, seed=0, dtype="float32", tensors=None):
    from zig_ai_amd.engine import DecoderModel
    d, tensors = nu.folder(cfg, seed, tensors)
    return DecoderModel.from_folder(d, dtype), tensors


def runner_for(model, page_size=4, tokens=256, slots=4, graphs=True):
    from zig_ai_amd.engine import ModelRunner
    return ModelRunner(model, page_size=page_size, num_pages=max(1, -(-tokens // page_size)),
                       num_slots=slots, use_graphs=graphs)


def plain_logits(cfg, tensors, prompts):
    return [plain.forward(cfg, tensors, p)[0].float() for p in prompts]


def worst(got, want):
    return float(nu.row_error(got, want).max())


def assert_bfloat16_close(got, want, what=None):
    e = nu.row_error(got, want)
    found = (float(e.median()), float(e.quantile(0.9)), float((e > BF16_WORST).double().mean()))
    assert found[0] < BF16_MEDIAN and found[1] < BF16_DECILE and found[2] <= BF16_FAR_SHARE, \
        (what, found)


def assert_bfloat16_same(got, base, what=None):
    """Two bfloat16 runs of the same requests, cut or batched differently."""
    e = nu.row_error(got, base)
    found = (float(e.median()), float((e > BF16_BETWEEN_WORST).double().mean()))
    assert found[0] < BF16_BETWEEN_MEDIAN and found[1] <= BF16_FAR_SHARE, (what, found)


# ----------------------------------------------------------- each mechanism alone
ALONE = {
    "lightning": nu.one_layer("lightning", nu.lightning()),
    "lightning, wide, no decay and a fast one": nu.one_layer(
        "lightning", nu.lightning(heads=2, dim=40, vdim=72, decay=[1.0, 0.25])),
    "attention": nu.one_layer("attention", nu.attention()),
    "attention, one kv head, chunk of five": nu.one_layer(
        "attention", nu.attention(heads=8, kv_heads=1, dim=32, vdim=16, scale=0.4, chunk=5,
                                  rot_dims=16, scaling=(8.0, 1.0, 4.0, 64))),
    "attention, no frequency scaling, one chunk for all": nu.one_layer(
        "attention", nu.attention(heads=2, kv_heads=2, dim=24, chunk=4096, scaling=None)),
    "attention, no rotation, no chunks": nu.one_layer(
        "attention", nu.attention(heads=2, kv_heads=1, dim=16, chunk=0, rot_dims=0)),
    "sizes that are multiples of nothing": nu.config([
        nu.layer("attention", nu.attention(heads=3, kv_heads=1, dim=20, vdim=12, chunk=9, rot_dims=6),
                 nu.dense(20)),
        nu.layer("lightning", nu.lightning(heads=5, dim=12, vdim=20), nu.moe(ff=12, experts=7, top=3)),
        nu.layer("attention_2", nu.attention_2(heads=3, kv_heads=3, dim=10, vdim=28, conv=2, rot_dims=6),
                 nu.dense(44)),
        nu.layer("attention", nu.attention(heads=2, kv_heads=2, dim=6, vdim=6, chunk=4, rot_dims=6),
                 None)], width=36, vocab=53, loop=(1, 3, 2)),
    "attention, forty heads on one key head": nu.one_layer(
        "attention", nu.attention(heads=40, kv_heads=1, dim=8, vdim=8, chunk=30, rot_dims=4)),
    "attention_2, sixty-six heads on two key heads": nu.one_layer(
        "attention_2", nu.attention_2(heads=66, kv_heads=2, dim=8, vdim=8, conv=3, rot_dims=8)),
    "attention_2": nu.one_layer("attention_2", nu.attention_2()),
    "attention_2, one tap, whole rotation": nu.one_layer(
        "attention_2", nu.attention_2(heads=2, kv_heads=2, dim=16, vdim=16, conv=1, rot_dims=16)),
    "attention_2, eight taps, one kv head": nu.one_layer(
        "attention_2", nu.attention_2(heads=5, kv_heads=1, dim=32, vdim=8, conv=8, rot_dims=2)),
    "dense": nu.one_layer("lightning", nu.lightning(), nu.dense()),
    "experts": nu.one_layer("lightning", nu.lightning(), nu.moe()),
    "experts, one of one": nu.one_layer("attention", nu.attention(), nu.moe(ff=40, experts=1, top=1)),
    "experts, all of four": nu.one_layer("attention_2", nu.attention_2(), nu.moe(ff=8, experts=4, top=4)),
    "loop of one layer, three times": nu.one_layer("lightning", nu.lightning(), nu.dense(16),
                                                   loop=(0, 1, 3)),
    "loop of an attention_2 layer, twice": nu.one_layer("attention_2", nu.attention_2(), None,
                                                       loop=(0, 1, 2)),
}


@pytest.mark.parametrize("name", sorted(ALONE))
def test_mechanism_alone(name):
    cfg = ALONE[name]
    model, tensors = build(cfg, seed=3)
    prompts = [nu.tokens(70, cfg["vocab"], 1), nu.tokens(5, cfg["vocab"], 2)]
    want = plain_logits(cfg, tensors, prompts)
    runner = runner_for(model)
    got = eu.run_schedule(runner, prompts, eu.whole([len(p) for p in prompts]))
    for g, w in zip(got, want):
        assert worst(g, w) < F32_BOUND
    # the same, token by token from the first token on: the state and the cache alone
    got = eu.run_schedule(runner, prompts, eu.bulk_then_single([len(p) for p in prompts], tail=10 ** 6))
    for g, w in zip(got, want):
        assert worst(g, w) < F32_BOUND


def test_every_mechanism_matters():
    """The plain implementation with one mechanism changed is far from itself: what the
    engine is held to would notice each of them."""
    cfg = nu.TINY_ALL
    tensors = nu.make_tensors(cfg, seed=4)
    prompt = nu.tokens(60, cfg["vocab"], 3)
    want = plain.forward(cfg, tensors, prompt)[0].float()

    def changed(edit):
        import copy
        c = copy.deepcopy(cfg)
        t = dict(tensors)
        edit(c, t)
        return worst(plain.forward(c, t, prompt)[0].float(), want)

    def chunk(c, t): c["layers"][0]["mixer"]["mask"]["size"] += 1
    def scaling(c, t): del c["layers"][0]["mixer"]["rot"]["scaling"]
    def taps(c, t): t["l2.mix.k.conv"] = t["l2.mix.k.conv"].flip(1)
    def router_bias(c, t): t["l1.mlp.router.b"] = torch.zeros_like(t["l1.mlp.router.b"])
    def loop_in(c, t): t["loop.in"] = t["loop.in"].roll(c["width"], 1)
    def decay(c, t): c["layers"][1]["mixer"]["decay"][2] = 0.9
    def gate(c, t): t["l0.mix.g"] = -t["l0.mix.g"]
    for edit in (chunk, scaling, taps, router_bias, loop_in, decay, gate):
        assert changed(edit) > 0.02, edit.__name__


def test_streams_after_every_layer_run():
    cfg = nu.TINY_ALL
    model, tensors = build(cfg, seed=4)
    prompt = nu.tokens(21, cfg["vocab"], 3)
    _, streams = plain.forward(cfg, tensors, prompt)
    from zig_ai_amd.engine import StepEntry
    runner = runner_for(model)
    runner.admit("a")
    taps = []
    runner.step([StepEntry("a", prompt, [])], taps=taps)
    assert len(taps) == len(streams) + 1 == 12       # the embedding, then eleven layer runs
    for i, s in enumerate(streams):
        got = taps[i + 1]["stream"].double().cpu()
        assert float((got - s).abs().max()) < 1e-4 * float(s.abs().max()), i


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


CONFIGS = {"all": nu.TINY_ALL, "other": nu.TINY_OTHER, "loop once": nu.TINY_LOOP_ONCE,
           "loop twice": nu.TINY_LOOP_TWICE}


@pytest.mark.parametrize("which", ["all", "other", "loop once", "loop twice"])
@pytest.mark.parametrize("page_size", [4, 16])
def test_schedules_float32(which, page_size):
    cfg = CONFIGS[which]
    model, tensors = build(cfg, seed=11)
    prompts = [nu.tokens(n, cfg["vocab"], 20 + i) for i, n in enumerate(LENGTHS)]
    want = plain_logits(cfg, tensors, prompts)
    for name, schedule in schedules(LENGTHS).items():
        # a pool for the most tokens live at any time: pages and slots are used again
        peak = eu.peak_tokens(LENGTHS, schedule, round_to=max(16, page_size))
        runner = runner_for(model, page_size=page_size, tokens=peak, slots=4)
        got = eu.run_schedule(runner, prompts, schedule)
        for i, (g, w) in enumerate(zip(got, want)):
            assert worst(g, w) < F32_BOUND, (name, i)
        if "mixed" in name:
            assert runner.cache.pages_reused > 0
        assert len(runner.cache.requests) == 0
        runner.cache.check()


@pytest.mark.parametrize("which", ["all", "other"])
def test_schedules_bfloat16(which):
    cfg = CONFIGS[which]
    model, tensors = build(cfg, seed=11, dtype="bfloat16")
    prompts = [nu.tokens(n, cfg["vocab"], 20 + i) for i, n in enumerate(LENGTHS)]
    want = plain_logits(cfg, tensors, prompts)
    base = None
    for name, schedule in schedules(LENGTHS).items():
        peak = eu.peak_tokens(LENGTHS, schedule, round_to=16)
        got = eu.run_schedule(runner_for(model, page_size=16, tokens=peak), prompts, schedule)
        assert_bfloat16_close(torch.cat(got), torch.cat(want), name)
        base = base or got
        assert_bfloat16_same(torch.cat(got), torch.cat(base), name)


def test_sizes_that_are_multiples_of_nothing_in_bfloat16():
    cfg = ALONE["sizes that are multiples of nothing"]
    model, tensors = build(cfg, seed=13, dtype="bfloat16")
    lengths = [60, 21, 2]
    prompts = [nu.tokens(n, cfg["vocab"], 70 + i) for i, n in enumerate(lengths)]
    want = plain_logits(cfg, tensors, prompts)
    base = None
    for name, schedule in (("whole", eu.whole(lengths)), ("bulk + tail", eu.bulk_then_single(lengths, tail=20)),
                           ("mixed", eu.mixed(lengths, seed=3, max_live=3, decode_tail=10))):
        got = eu.run_schedule(runner_for(model, page_size=16, tokens=256), prompts, schedule)
        assert_bfloat16_close(torch.cat(got), torch.cat(want), name)
        base = base or got
        assert_bfloat16_same(torch.cat(got), torch.cat(base), name)


@pytest.mark.parametrize("seed", range(10))
def test_random_configurations(seed):
    cfg = nu.random_config(seed)
    model, tensors = build(cfg, seed=seed)
    lengths = [90, 1, 23, 2]
    prompts = [nu.tokens(n, cfg["vocab"], 30 + i) for i, n in enumerate(lengths)]
    want = plain_logits(cfg, tensors, prompts)
    for name, schedule in (("whole", eu.whole(lengths)),
                           ("portions", eu.changing_portions(lengths, seed=seed)),
                           ("mixed", eu.mixed(lengths, seed=seed, max_live=3, decode_tail=15))):
        peak = eu.peak_tokens(lengths, schedule, round_to=16)
        got = eu.run_schedule(runner_for(model, page_size=4, tokens=peak, slots=3), prompts, schedule)
        for i, (g, w) in enumerate(zip(got, want)):
            assert worst(g, w) < F32_BOUND, (seed, name, i)


# ------------------------------------------------ a key just inside and just outside
def edge_model(kind, dtype, dim, chunk=0):
    """One attention layer whose last query puts all but all of its weight on ONE key: the
    token 299 wherever it stands.  A key that is wrongly seen, or wrongly not seen, moves
    the result by its whole size."""
    if kind == "attention":
        mixer = nu.attention(heads=2, kv_heads=1, dim=dim, scale=1.0, chunk=chunk, rot_dims=2,
                             base=1e6, scaling=None)
    else:
        mixer = nu.attention_2(heads=2, kv_heads=1, dim=dim, vdim=dim, scale=1.0, conv=1,
                               rot_dims=2, base=1e6)
    cfg = nu.one_layer(kind, mixer, None, width=64, vocab=300)
    t = nu.make_tensors(cfg, seed=7)
    t["l0.norm1"] = torch.ones_like(t["l0.norm1"])
    # token 299 is the one to find and token 298 the one that asks: the key's LAST element
    # (not rotated) reads the stream's first channel, where 299 is long and every other token
    # is zero; the queries' last elements read the second channel, where only 298 is not zero
    t["embed"][:, :2] = 0.0
    for tok, ch in ((299, 0), (298, 1)):
        t["embed"][tok] = 0.0
        t["embed"][tok, ch] = 8.0
    t["l0.mix.k"][dim - 1, :] = 0.0
    t["l0.mix.k"][dim - 1, 0] = 3.0
    for h in range(2):
        t["l0.mix.q"][h * dim + dim - 1, :] = 0.0
        t["l0.mix.q"][h * dim + dim - 1, 1] = 3.0
    if kind == "attention":
        for n in ("q", "k"):
            t[f"l0.mix.{n}.b"] = torch.zeros_like(t[f"l0.mix.{n}.b"])
            t[f"l0.mix.{n}.norm"] = torch.full_like(t[f"l0.mix.{n}.norm"], 1.5)
    else:
        for n in ("q", "k", "v"):
            t[f"l0.mix.{n}.conv"] = torch.ones_like(t[f"l0.mix.{n}.conv"])
    t["l0.mix.o"] *= 4.0
    return cfg, {k: v.to(torch.bfloat16).float() for k, v in t.items()}


@pytest.mark.parametrize("dtype,dim", [("float32", 16), ("bfloat16", 64), ("bfloat16", 128),
                                       ("bfloat16", 24)])
def test_chunk_edges(dtype, dim):
    chunk = 48
    cfg, tensors = edge_model("attention", dtype, dim, chunk)
    model, _ = build(cfg, tensors=tensors, dtype=dtype)
    n = 200
    asks = 150                                           # chunk 3: positions 144..191
    for place, seen in ((143, False), (144, True), (145, True), (149, True), (150, True),
                        (96, False), (0, False)):
        prompt = [t % 298 for t in nu.tokens(n, 298, place)]
        prompt[place] = 299
        if place != asks:
            prompt[asks] = 298
        other = list(prompt)
        other[place] = 5 if place != asks else 6          # the same prompt without the key
        want = plain.forward(cfg, tensors, prompt)[0].float()
        moved = worst(plain.forward(cfg, tensors, other)[0].float()[asks:asks + 1], want[asks:asks + 1])
        assert (moved > 0.05) == seen, (place, moved)
        for schedule in (eu.whole([n]), eu.bulk_then_single([n], tail=n - 146),
                         eu.bulk_then_single([n], tail=n - 140),
                         eu.changing_portions([n], sizes=(47, 2, 96, 3, 2, 17))):
            got = eu.run_schedule(runner_for(model, page_size=16, tokens=256), [prompt], schedule)[0]
            if dtype == "float32":
                assert worst(got, want) < F32_BOUND, place
            else:
                assert worst(got[asks:asks + 1], want[asks:asks + 1]) < 0.03, place
                assert worst(got, want) < BF16_WORST, place


@pytest.mark.parametrize("dtype,dim", [("float32", 16), ("bfloat16", 64), ("bfloat16", 128),
                                       ("bfloat16", 32)])
def test_a_far_key_is_found(dtype, dim):
    cfg, tensors = edge_model("attention_2", dtype, dim)
    model, _ = build(cfg, tensors=tensors, dtype=dtype)
    n = 700
    for place in (0, 1, 15, 16, 63, 64, 333):           # first tokens, page and tile borders
        prompt = [t % 298 for t in nu.tokens(n, 298, place)]
        prompt[place] = 299
        prompt[-1] = 298
        other = list(prompt)
        other[place] = 5                                 # the same prompt without the key
        want = plain.forward(cfg, tensors, prompt)[0].float()
        assert worst(plain.forward(cfg, tensors, other)[0].float()[-1:], want[-1:]) > 0.05
        for schedule in (eu.whole([n]), eu.bulk_then_single([n], tail=3),
                         eu.changing_portions([n], sizes=(64, 2, 130, 17, 256))):
            got = eu.run_schedule(runner_for(model, page_size=16, tokens=1024), [prompt], schedule)[0]
            if dtype == "float32":
                assert worst(got, want) < F32_BOUND, place
            else:
                assert worst(got[-1:], want[-1:]) < 0.03, place


# --------------------------------------------------------------- the sink's share
@pytest.mark.parametrize("dtype,dim", [("float32", 16), ("bfloat16", 64), ("bfloat16", 24)])
def test_the_sink_counts_once_however_the_context_is_cut(dtype, dim):
    # scores so far below zero that the sink takes a third of every head's weight at 1,300
    # keys and nearly all of it at the first tokens: left out, or counted once per range of
    # a cut context, it would move every output by tens of percent
    cfg = nu.one_layer("attention_2", nu.attention_2(heads=4, kv_heads=1, dim=dim, vdim=dim,
                                                     scale=0.1, conv=2, rot_dims=8),
                       width=64, vocab=97)
    tensors = nu.make_tensors(cfg, seed=5)
    n = 1300
    prompt = nu.tokens(n, cfg["vocab"], 1)
    tensors["l0.mix.o"] *= 16.0
    # every token's first channel is the same; the last element of every query reads it with
    # one sign and the last element of the key with the other (the filter hands q and k on)
    tensors["embed"][:, 0] = 2.0
    tensors["l0.norm1"] = torch.ones_like(tensors["l0.norm1"])
    for name, rows, sign in (("q", range(dim - 1, 4 * dim, dim), -4.0), ("k", [dim - 1], 4.0)):
        for r in rows:
            tensors[f"l0.mix.{name}"][r, :] = 0.0
            tensors[f"l0.mix.{name}"][r, 0] = sign
        tensors[f"l0.mix.{name}.conv"][:, 0] = 0.0
        tensors[f"l0.mix.{name}.conv"][:, 1] = 1.0
    want = plain.forward(cfg, tensors, prompt)[0].float()

    # the same softmax without the sink, in the plain implementation
    original = plain.softmax_attention
    try:
        plain.softmax_attention = lambda *a, **kw: original(*a, **{**kw, "sink": False})
        assert worst(plain.forward(cfg, tensors, prompt)[0].float()[-40:], want[-40:]) > 0.05
    finally:
        plain.softmax_attention = original
    model, _ = build(cfg, tensors=tensors, dtype=dtype)
    bound = F32_BOUND if dtype == "float32" else 0.03
    # one request decoding at 1,300 keys: its context is cut into ranges that are merged
    for schedule in (eu.whole([n]), eu.bulk_then_single([n], tail=40),
                     eu.changing_portions([n], sizes=(600, 2, 500, 64, 100, 3))):
        got = eu.run_schedule(runner_for(model, page_size=16, tokens=2048), [prompt], schedule)[0]
        assert worst(got[-40:], want[-40:]) < bound
        assert worst(got[:8], want[:8]) < bound                    # the first tokens


# --------------------------------------------------- the convolution across the cuts
def test_the_convolution_carries_its_inputs_across_every_cut():
    cfg = nu.one_layer("attention_2", nu.attention_2(heads=2, kv_heads=1, dim=16, vdim=16, conv=6,
                                                     rot_dims=4))
    model, tensors = build(cfg, seed=14)
    n = 40
    prompt = nu.tokens(n, cfg["vocab"], 4)
    want = plain.forward(cfg, tensors, prompt)[0].float()
    # portions shorter than the filter, as long as it, and longer; single tokens between
    for sizes in ((1, 2, 3, 4, 5, 6, 7), (5, 1, 1, 6, 2), (2, 2, 2), (6, 6, 6), (39, 1)):
        got = eu.run_schedule(runner_for(model), [prompt], eu.changing_portions([n], sizes=sizes))[0]
        assert worst(got, want) < F32_BOUND, sizes
    # a slot that another request has left starts from zeros again
    runner = runner_for(model, slots=1)
    for p in (nu.tokens(n, cfg["vocab"], 5), prompt):
        got = eu.run_schedule(runner, [p], eu.bulk_then_single([n], tail=7))[0]
        assert worst(got, plain.forward(cfg, tensors, p)[0].float()) < F32_BOUND


# ----------------------------------------------------------------- far tokens count
def test_far_tokens_reach_the_end_through_the_state():
    cfg = nu.one_layer("lightning", nu.lightning(heads=2, dim=16, vdim=16,
                                                 decay=[0.99951171875, 1.0]))
    model, tensors = build(cfg, seed=9)
    n = 600
    a = nu.tokens(n, cfg["vocab"], 3)
    b = list(a)
    b[1] = (b[1] + 1) % cfg["vocab"]
    wa, wb = (plain.forward(cfg, tensors, p)[0].float() for p in (a, b))
    assert worst(wb[-8:], wa[-8:]) > 1e-3          # the second token still shows at the end
    for prompt, want in ((a, wa), (b, wb)):
        for schedule in (eu.whole([n]), eu.bulk_then_single([n], tail=64),
                         eu.changing_portions([n], sizes=(33, 2, 64, 17, 300))):
            got = eu.run_schedule(runner_for(model, tokens=1024), [prompt], schedule)[0]
            assert worst(got, want) < F32_BOUND
    # nothing is left of a request whose slot is taken again: b after a in a pool of one slot
    runner = runner_for(model, tokens=1024, slots=1)
    for prompt, want in ((a, wa), (b, wb), (a, wa)):
        got = eu.run_schedule(runner, [prompt], eu.bulk_then_single([n], tail=5))[0]
        assert worst(got, want) < F32_BOUND


# ------------------------------------------------------------------- long decoding
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype):
    cfg = nu.TINY_ALL
    model, tensors = build(cfg, seed=21, dtype=dtype)
    n = 330
    prompts = [nu.tokens(n, cfg["vocab"], 5)]
    want = plain_logits(cfg, tensors, prompts)[0]
    runner = runner_for(model, page_size=16, tokens=512)       # decode steps replay from graphs
    assert runner.graphs is not None
    got = eu.run_schedule(runner, prompts, eu.bulk_then_single([n], tail=300))[0]
    if dtype == "float32":
        assert worst(got, want) < F32_BOUND
    else:
        assert_bfloat16_close(got, want)
    # the same steps issued kernel by kernel
    again = eu.run_schedule(runner_for(model, page_size=16, tokens=512, graphs=False), prompts,
                            eu.bulk_then_single([n], tail=300))[0]
    if dtype == "float32":
        assert worst(again, got) < 1e-5
    else:
        assert_bfloat16_same(again, got)


# ------------------------------------------- unequal requests together and alone
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_batch_against_each_alone(dtype):
    cfg = nu.TINY_ALL
    model, tensors = build(cfg, seed=2, dtype=dtype)
    lengths = [64, 3, 41, 17]
    prompts = [nu.tokens(n, cfg["vocab"], 40 + i) for i, n in enumerate(lengths)]
    alone = eu.run_schedule(runner_for(model, tokens=256), prompts, eu.whole(lengths))
    together = [([(i, 0, n) for i, n in enumerate(lengths)], list(range(len(lengths))))]
    got = eu.run_schedule(runner_for(model, tokens=256), prompts, together)
    if dtype == "float32":
        assert worst(torch.cat(got), torch.cat(alone)) < 1e-5
    else:
        assert_bfloat16_same(torch.cat(got), torch.cat(alone))


# ------------------- sizes that the matrix-core kernels take, at widths of real layers
@pytest.mark.parametrize("dim,heads,kv", [(64, 8, 2), (128, 4, 1), (64, 16, 4)])
def test_matrix_core_paths(dim, heads, kv):
    cfg = nu.config([
        nu.layer("attention", nu.attention(heads=heads, kv_heads=kv, dim=dim, scale=dim ** -0.5,
                                           chunk=100, rot_dims=dim // 2, base=1e4),
                 nu.moe(ff=64, experts=6, top=2)),
        nu.layer("lightning", nu.lightning(heads=3, dim=64, vdim=32), nu.dense(256)),
        nu.layer("attention_2", nu.attention_2(heads=heads, kv_heads=kv, dim=dim, vdim=dim,
                                               scale=dim ** -0.5, conv=4, rot_dims=dim),
                 nu.moe(ff=32, experts=3, top=1)),
    ], width=256, vocab=211, loop=(0, 3, 2))
    model, tensors = build(cfg, seed=6, dtype="bfloat16")
    assert model.blocks[0].parts["mixer"].mfma and model.blocks[2].parts["mixer"].mfma
    lengths = [300, 70, 3]
    prompts = [nu.tokens(n, cfg["vocab"], 50 + i) for i, n in enumerate(lengths)]
    want = plain_logits(cfg, tensors, prompts)
    base = None
    for name, schedule in (("whole", eu.whole(lengths)),
                           ("bulk + tail", eu.bulk_then_single(lengths, tail=60)),
                           ("portions", eu.changing_portions(lengths, seed=3)),
                           ("mixed", eu.mixed(lengths, seed=1, max_live=3, decode_tail=30))):
        runner = runner_for(model, page_size=16, tokens=768, slots=3)
        got = eu.run_schedule(runner, prompts, schedule)
        assert_bfloat16_close(torch.cat(got), torch.cat(want), name)
        base = base or got
        assert_bfloat16_same(torch.cat(got), torch.cat(base), name)


# ------------------------------------------- generation through engine and scheduler
def test_greedy_generation():
    from zig_ai_amd.engine import Engine
    cfg = nu.TINY_ALL
    d, tensors = nu.folder(cfg, seed=8)
    engine = Engine(d, dtype="float32", page_size=4, num_pages=128, max_num_seqs=3,
                    max_num_batched_tokens=48, chunk_size=20, max_model_len=256)
    prompts = [nu.tokens(n, cfg["vocab"], 60 + i) for i, n in enumerate([33, 5, 70, 12, 1])]
    outs = engine.generate(prompts, max_new_tokens=20, temperature=0.0)
    assert all(len(o) == 20 for o in outs)
    for p, o in zip(prompts, outs):
        # every chosen token is the plain implementation's choice for the same history
        logits = plain.forward(cfg, tensors, p + o)[0]
        for j, tok in enumerate(o):
            row = logits[len(p) + j - 1]
            assert float(row.max() - row[tok]) <= 1e-3 * float(row.abs().max()), (j, tok)
    assert len(engine.runner.cache.requests) == 0
    engine.runner.cache.check()


def test_generation_bfloat16_runs_through_graphs():
    from zig_ai_amd.engine import Engine
    cfg = nu.TINY_OTHER
    d, tensors = nu.folder(cfg, seed=8)
    engine = Engine(d, dtype="bfloat16", page_size=16, num_pages=64, max_num_seqs=4,
                    max_model_len=256)
    assert engine.runner.graphs is not None        # every part can be recorded
    prompts = [nu.tokens(n, cfg["vocab"], 80 + i) for i, n in enumerate([40, 7, 19])]
    outs = engine.generate(prompts, max_new_tokens=24, temperature=0.0)
    for p, o in zip(prompts, outs):
        logits = plain.forward(cfg, tensors, p + o)[0]
        for j, tok in enumerate(o):
            row = logits[len(p) + j - 1]
            spread = float(row.max() - row.min())
            assert float(row.max() - row[tok]) <= 0.1 * spread, (j, tok)


def test_trace_replay_and_command_line(tmp_path):
    import json
    import os
    import subprocess
    import sys
    cfg = nu.TINY_LOOP_TWICE
    d, tensors = nu.folder(cfg, seed=12)
    prompt = nu.tokens(40, cfg["vocab"], 9)
    want = plain.forward(cfg, tensors, prompt)[0].float()
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": prompt[:25], "want": [3, 24]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": prompt[25:27], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": prompt[27:], "want": [12]}], "end": ["a"]}]
    out = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", d,
                          "--dtype", "float32", "--out", str(tmp_path), "--max-tokens", "64"],
                         input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
                         capture_output=True, timeout=600)
    assert out.returncode == 0, out.stderr[-2000:]
    assert [l for l in out.stdout.split("\n") if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    import numpy as np
    first = torch.from_numpy(np.fromfile(tmp_path / "0.f32", dtype="<f4").reshape(2, -1))
    last = torch.from_numpy(np.fromfile(tmp_path / "2.f32", dtype="<f4").reshape(1, -1))
    assert not (tmp_path / "1.f32").exists()
    assert worst(torch.cat([first, last]), want[[3, 24, 39]]) < F32_BOUND
    gen = subprocess.run([sys.executable, "-m", "zig_ai_amd", "--model", d, "--dtype", "float32",
                          "--prompt-ids", ",".join(map(str, prompt[:9])), "-n", "5",
                          "--temperature", "0", "--json"], cwd=root, text=True, capture_output=True,
                         timeout=600)
    assert gen.returncode == 0, gen.stderr[-2000:]
    outputs = json.loads(gen.stdout.strip().split("\n")[-1])["outputs"]
    assert len(outputs) == 1 and len(outputs[0]) == 5
    logits = plain.forward(cfg, tensors, prompt[:9] + outputs[0])[0]
    for j, tok in enumerate(outputs[0]):
        row = logits[9 + j - 1]
        assert float(row.max() - row[tok]) <= 1e-3 * float(row.abs().max()), (j, tok)


# ------------------------------------------------------------------ kernels alone
def _slots(n_slots, floats, device):
    # rows spaced wider than their length, as the cache manager's slot rows are
    mem = torch.zeros((n_slots, floats + 12), dtype=torch.float32, device=device)
    return mem, mem[:, :floats]


def _step_arrays(lengths, slots, device):
    start = [0]
    for n in lengths:
        start.append(start[-1] + n)
    mk = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    seq = [i for i, n in enumerate(lengths) for _ in range(n)]
    return mk(seq), mk(start), mk(slots)


@pytest.mark.parametrize("C,L,dtype", [(40, 3, torch.float32), (300, 1, torch.float32),
                                       (64, 8, torch.bfloat16), (17, 4, torch.bfloat16)])
def test_convolution_without_activation(C, L, dtype):
    """The convolution kernel with no activation, across two steps through the state slot."""
    from zig_ai_amd.kernels import ops
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(C + L)
    lengths = [9, 1, 30]
    T = sum(lengths)
    x = (torch.randn(T, C + 5, generator=g)).to(dtype)
    taps = torch.randn(C, L, generator=g)
    mem, state = _slots(4, 3 + C * max(L - 1, 1), dev)
    slots = [2, 0, 3]
    cut = [4, 0, 7]
    start = [0, 9, 10, 40]
    got = torch.zeros((T, C), dtype=torch.float64)
    for first in (True, False):
        lens = [c for c in cut if c] if first else [n - c for n, c in zip(lengths, cut)]
        used = [s for s, c in zip(slots, cut) if c] if first else slots
        rows = [r for i in range(3) for r in (range(start[i], start[i] + cut[i]) if first
                                              else range(start[i] + cut[i], start[i + 1]))]
        idx = torch.tensor(rows)
        seq, st, sl = _step_arrays(lens, used, dev)
        out = ops.causal_conv(x[idx].to(dev).contiguous(), 2, taps.to(dev), None, state, 3, seq, st,
                              sl, activation=None, out_dtype=dtype)
        assert out.dtype == dtype
        got[idx] = out.double().cpu()
    for i in range(3):
        u = x[start[i]:start[i + 1], 2:2 + C].double()
        want, _ = plain.causal_conv(u, taps.double())
        tol = 1e-5 if dtype == torch.float32 else 2e-2
        assert float((got[start[i]:start[i + 1]] - want).abs().max()) < tol * float(want.abs().max())


def test_lightning_prepare_and_norm_kernels():
    """silu on q, k and v ahead of the walk; one norm over all heads with a sigmoid gate."""
    from zig_ai_amd.kernels import ops
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(3)
    H, d, dv, T = 3, 24, 40, 11
    proj = torch.randn(T, 2 * H * d + 2 * H * dv, generator=g)
    pos = torch.arange(T, dtype=torch.int32)
    vec = ops.retention_prepare(proj.to(dev), 0, H * d, 2 * H * d, pos.to(dev), None, H, d, dv, 0,
                                1.0, "silu")
    want = plain.silu(proj[:, :2 * H * d + H * dv].double())
    assert float((vec.double().cpu() - want).abs().max()) < 1e-6
    o = torch.randn(T, H * dv, generator=g) * 3
    w = torch.randn(H * dv, generator=g)
    out = ops.gated_group_norm(o.to(dev), proj.to(dev), 2 * H * d + H * dv, w.to(dev), H * dv, 1e-5,
                               "sigmoid", gate_first=False)
    want = plain.rms_norm(o.double(), w.double(), 1e-5) * torch.sigmoid(proj[:, 2 * H * d + H * dv:].double())
    assert float((out.double().cpu() - want).abs().max()) < 1e-5 * float(want.abs().max())


def test_relu_squared_kernel():
    from zig_ai_amd.kernels import ops
    x = torch.randn(7, 33) * 2
    for dtype, tol in ((torch.float32, 1e-6), (torch.bfloat16, 1e-2)):
        got = ops.activate(x.to(dtype).cuda(), "relu2").double().cpu()
        want = torch.relu(x.to(dtype).double()) ** 2
        assert float((got - want).abs().max()) <= tol * float(want.abs().max())
