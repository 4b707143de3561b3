"""Nopozen's configuration, its translation into parts, and what pins the plain
implementation (``plain_nopozen.py``) besides the engine: library routines and invariants.
No GPU."""

import copy
import math

import pytest
import torch

import nopozen_util as nu
import plain_nopozen as plain
from zig_ai_amd.config import ConfigError, config_from_dict, known_architectures
from zig_ai_amd.config.nopozen import NopozenConfig
from zig_ai_amd.weights.loader import expected_tensors


def test_registered_and_round_trip():
    assert "Nopozen" in known_architectures()
    for cfg in (nu.TINY_ALL, nu.TINY_OTHER, nu.TINY_LOOP_ONCE, nu.TINY_LOOP_TWICE):
        c = config_from_dict(cfg)
        assert isinstance(c, NopozenConfig)
        assert c.to_dict() == cfg
        assert config_from_dict(c.to_dict()) == c


def test_every_tensor_is_named_with_its_shape():
    for cfg in (nu.TINY_ALL, nu.TINY_OTHER, nu.TINY_LOOP_TWICE):
        tensors = nu.make_tensors(cfg)
        spec = config_from_dict(cfg).to_spec()
        expected = {e.names[0]: tuple(e.rule.stored_shape or e.rule.shapes[0])
                    for e in expected_tensors(spec)}
        assert expected == {k: tuple(v.shape) for k, v in tensors.items()}


def test_run_order():
    spec = config_from_dict(nu.TINY_ALL).to_spec()          # 5 layers, 1..3 three times
    order = [(c.layer, c.before is not None) for c in spec.schedule]
    assert order == [(0, False)] + [(1, True), (2, False), (3, False)] * 3 + [(4, False)]
    assert plain.run_order(nu.TINY_ALL) == order
    # every time a layer runs it has a cache entry of its own
    assert len({c.cache for c in spec.resolved_schedule()}) == 11
    assert [p.kind for p in spec.stream_parts] == ["pass_mix"]
    once = config_from_dict(nu.TINY_LOOP_ONCE).to_spec()
    assert [(c.layer, c.before is not None) for c in once.schedule] == [(0, True), (1, False)]
    none = config_from_dict(nu.TINY_OTHER).to_spec()
    assert none.stream_parts == () and all(c.before is None for c in none.schedule)


def test_constants_reach_the_parts():
    spec = config_from_dict(nu.TINY_ALL).to_spec()
    a, l, a2 = (spec.layers[i].parts["mixer"] for i in range(3))
    assert a.kind == "gqa_attention" and a.params["chunk"] == 12 and a.params["gate"] == "head"
    assert a.params["bias"] is True and a.params["qk_norm"] and a.params["softmax_scale"] == 0.5
    assert a.params["position"].params["scaling"] == {"factor": 4.0, "low": 1.0, "high": 3.0,
                                                      "original": 40}
    assert l.kind == "retention" and l.params["activation"] == "silu" and l.params["key_scale"] == 1.0
    assert l.params["output_norm"] == "all" and l.params["gate"] == "sigmoid"
    assert l.params["position"] is None and len(l.params["decay"]) == 3
    assert a2.kind == "gqa_attention" and a2.params["conv"] == 3 and a2.params["sink_value"] == 0.0
    assert a2.params["gate"] == "element" and a2.params["value_dim"] == 16
    assert a2.params["position"].params["rotary_dim"] == 8 and not a2.params.get("chunk")
    assert spec.layers[0].arrangement == "parallel_residual"
    assert spec.layers[2].arrangement == "parallel_residual_no_ff"
    ff = spec.layers[1].parts["feed_forward"]
    assert ff.kind == "routed_experts" and ff.params["renormalize"] and ff.params["router_bias"]
    assert spec.layers[0].parts["feed_forward"].kind == "activated_mlp"
    assert spec.lm_head.params["tied"] is False


def test_cache_needs():
    from zig_ai_amd.parts import PagedNeed, PagedStateNeed, StateNeed, lookup
    spec = config_from_dict(nu.TINY_ALL).to_spec()
    needs = [lookup("mixer", spec.layers[i].parts["mixer"].kind).cache_need(
        spec.layers[i].parts["mixer"].params) for i in range(3)]
    assert needs[0] == PagedNeed.kv(2, 16)
    assert needs[1] == StateNeed((3 * 16 * 24,))
    assert isinstance(needs[2], PagedStateNeed)
    assert needs[2].paged == PagedNeed(((3, 24), (3, 16)))
    assert needs[2].state == StateNeed(((6 * 24 + 3 * 24 + 3 * 16) * 2,))


def test_a_cache_entry_with_pages_and_a_state():
    from zig_ai_amd.cache.manager import CacheManager
    from zig_ai_amd.parts import PagedNeed, PagedStateNeed, StateNeed
    needs = {0: PagedStateNeed(PagedNeed.kv(2, 8), StateNeed((10,))), 1: PagedNeed.kv(2, 8),
             2: StateNeed((3,))}
    cache = CacheManager(needs, page_size=4, num_pages=6, num_slots=2, allocate=False)
    assert len(cache.groups) == 1 and cache.groups[0].cache_ids == [0, 1]
    assert cache.bytes_per_slot == 48 + 16          # 10 floats rounded up to 16 bytes, then 3
    v = cache.view(0)
    assert v.kind == "paged" and v.group == 0
    assert cache.view(2).kind == "state"
    assert CacheManager.bytes_per_page_index(needs, 4, torch.bfloat16) == 2 * (2 * 2 * 8) * 4 * 2


@pytest.mark.parametrize("edit,text", [
    (lambda c: c["layers"][0].update(type="conv"), "type must be one of"),
    (lambda c: c["layers"][1]["mixer"].update(decay=[0.5]), "decay must list"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "do not divide"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "must be even"),
    (lambda c: c["layers"][2]["mixer"].pop("conv"), "conv"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "top 9 of 5"),
    (lambda c: c["loop"].update(stop=9), "loop spans"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_malformed_configurations(edit, text):
    cfg = copy.deepcopy(nu.TINY_ALL)
    edit(cfg)
    with pytest.raises(ConfigError, match=text):
        config_from_dict(cfg)


# ------------------------------------------------ what pins the plain implementation
def test_plain_small_pieces_against_the_library():
    x = torch.randn(5, 12, dtype=torch.float64)
    assert torch.allclose(plain.gelu_tanh(x), torch.nn.functional.gelu(x, approximate="tanh"))
    assert torch.allclose(plain.silu(x), torch.nn.functional.silu(x))
    w = torch.randn(12, dtype=torch.float64)
    want = torch.nn.functional.rms_norm(x, (12,), w, 1e-5)
    assert torch.allclose(plain.rms_norm(x, w, 1e-5), want)
    # the convolution against the library's, and two portions against one
    u, taps = torch.randn(9, 4, dtype=torch.float64), torch.randn(4, 3, dtype=torch.float64)
    want = torch.nn.functional.conv1d(torch.nn.functional.pad(u.T[None], (2, 0)), taps[:, None, :],
                                      groups=4)[0].T
    got, last = plain.causal_conv(u, taps)
    assert torch.allclose(got, want) and torch.equal(last, u[-2:])
    a, mid = plain.causal_conv(u[:4], taps)
    b, _ = plain.causal_conv(u[4:], taps, mid)
    assert torch.allclose(torch.cat([a, b]), want)


def test_plain_rotation():
    r = {"dims": 8, "base": 100.0}
    f = plain.rotary_frequencies(r)
    assert torch.allclose(f, torch.tensor([100.0 ** (-2 * i / 8) for i in range(4)], dtype=torch.float64))
    q, k = torch.randn(1, 1, 12, dtype=torch.float64), torch.randn(1, 1, 12, dtype=torch.float64)
    # a score depends on the distance only; elements beyond ``dims`` pass unchanged
    def score(p, s):
        return float((plain.rotate(q, torch.tensor([p]), r) * plain.rotate(k, torch.tensor([s]), r)).sum())
    assert abs(score(9, 4) - score(105, 100)) < 1e-9 and abs(score(9, 4) - score(9, 5)) > 1e-6
    assert torch.equal(plain.rotate(q, torch.tensor([7]), r)[..., 8:], q[..., 8:])
    # halves: element 0 pairs with element 4
    e = torch.zeros(1, 1, 12, dtype=torch.float64)
    e[0, 0, 0] = 1.0
    out = plain.rotate(e, torch.tensor([1]), r)[0, 0]
    assert abs(float(out[0]) - math.cos(1.0)) < 1e-12 and abs(float(out[4]) - math.sin(1.0)) < 1e-12
    # the three bands of the scaled frequencies
    s = {"dims": 8, "base": 100.0, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}}
    g = plain.rotary_frequencies(s)
    wave = 2 * math.pi / f
    assert wave[0] < 16 and g[0] == f[0]
    assert wave[3] > 64 and abs(float(g[3]) - float(f[3]) / 4) < 1e-15
    mid = [i for i in range(4) if 16 <= wave[i] <= 64]
    assert mid and all(f[i] / 4 < g[i] < f[i] for i in mid)


def test_plain_attention_masks_and_sink():
    q = torch.randn(6, 2, 4, dtype=torch.float64)
    k, v = torch.randn(6, 1, 4, dtype=torch.float64), torch.randn(6, 1, 3, dtype=torch.float64)
    pos = torch.arange(6)
    o = plain.softmax_attention(q, k, v, pos, pos, 0.5)
    assert torch.allclose(o[0, 0], v[0, 0])                     # the first token sees itself
    v2 = v.clone()
    v2[4] += 1.0
    assert torch.equal(plain.softmax_attention(q, k, v2, pos, pos, 0.5)[:4], o[:4])   # causal
    c = plain.softmax_attention(q, k, v, pos, pos, 0.5, chunk=3)
    assert torch.allclose(c[3, 0], v[3, 0]) and torch.allclose(c[:3], o[:3])
    assert not torch.allclose(c[5], o[5])
    s = plain.softmax_attention(q, k, v, pos, pos, 0.5, sink=True)
    w0 = 1.0 / (1.0 + math.exp(-float((q[0, 0] * k[0, 0]).sum()) * 0.5))
    assert torch.allclose(s[0, 0], w0 * v[0, 0])                # e^s / (1 + e^s)


def test_plain_lightning_state_and_experts():
    cfg = nu.one_layer("lightning", nu.lightning(heads=2, dim=4, vdim=3, decay=[0.5, 1.0]), nu.moe(8, 4, 2))
    W = {k: v.double() for k, v in nu.make_tensors(cfg, 1).items()}
    h = torch.randn(7, cfg["width"], dtype=torch.float64)
    m = cfg["layers"][0]["mixer"]
    cache = {}
    whole = plain.lightning_mixer(h, "l0.mix.", W, m, 1e-5, cache)
    # the state is the decayed sum of outer products
    k = plain.silu(h @ W["l0.mix.k"].T).view(7, 2, 4)
    v = plain.silu(h @ W["l0.mix.v"].T).view(7, 2, 3)
    S0 = sum(0.5 ** (6 - t) * torch.outer(k[t, 0], v[t, 0]) for t in range(7))
    assert torch.allclose(cache["S"][0], S0)
    parts = {}
    a = plain.lightning_mixer(h[:3], "l0.mix.", W, m, 1e-5, parts)
    b = plain.lightning_mixer(h[3:], "l0.mix.", W, m, 1e-5, parts)
    assert torch.allclose(torch.cat([a, b]), whole)
    # experts: the chosen two, weighted by the softmax over their two logits
    y = plain.moe_ff(h[:1], "l0.mlp.", W, cfg["layers"][0]["mlp"])
    z = h[0] @ W["l0.mlp.router"].T + W["l0.mlp.router.b"]
    top = z.topk(2)
    wts = torch.softmax(top.values, 0)
    want = sum(wts[j] * ((plain.silu(h[0] @ W[f"l0.mlp.e{int(e)}.gate"].T) * (h[0] @ W[f"l0.mlp.e{int(e)}.up"].T))
                         @ W[f"l0.mlp.e{int(e)}.down"].T) for j, e in enumerate(top.indices))
    assert torch.allclose(y[0], want)


def test_plain_walker_token_by_token():
    cfg = nu.TINY_ALL
    tensors = nu.make_tensors(cfg, 2)
    prompt = nu.tokens(30, cfg["vocab"], 1)
    whole, streams = plain.forward(cfg, tensors, prompt)
    w = plain.Walker(cfg, tensors)
    rows = [w.feed(prompt[:11])[0], w.feed(prompt[11:12])[0], w.feed(prompt[12:])[0]]
    assert torch.allclose(torch.cat(rows), whole, atol=1e-9)
    assert streams.shape == (11, 30, cfg["width"])


def test_random_model_folder(tmp_path):
    """The random model writer stores every tensor the design names, in the folder's format."""
    from zig_ai_amd.weights import write_random_model
    from zig_ai_amd.weights.safetensors_io import Checkpoint
    cfg = config_from_dict(nu.TINY_ALL)
    write_random_model(cfg, str(tmp_path), seed=3, dtype=torch.bfloat16)
    ckpt = Checkpoint(str(tmp_path))
    want = {k: tuple(v.shape) for k, v in nu.make_tensors(nu.TINY_ALL).items()}
    assert {name: tuple(ckpt.shape(name)) for name in want} == want
    from zig_ai_amd.config import load_config
    assert load_config(str(tmp_path)) == cfg
