"""Gemodra's configuration and description as parts (no GPU), and what pins the plain
implementation's mechanisms: identities that a consistent mistake would break."""

import copy
import math

import pytest
import torch

import gemodra_util as gu
import plain_gemodra as plain
from zig_ai_amd.config import ConfigError, config_from_dict, known_architectures
from zig_ai_amd.weights.loader import expected_tensors


def test_registered_and_round_trip():
    assert "Gemodra" in known_architectures()
    for cfg in (gu.TINY_ALL, gu.TINY_OTHER) + tuple(gu.random_config(s) for s in range(12)):
        typed = config_from_dict(cfg)
        assert config_from_dict(typed.to_dict()) == typed
        assert typed.to_dict() == cfg
        assert typed.hidden_size == cfg["width"] and typed.vocab_size == cfg["vocab"]


@pytest.mark.parametrize("cfg", [gu.TINY_ALL, gu.TINY_OTHER, gu.random_config(3), gu.random_config(8)])
def test_every_tensor_is_named_with_its_shape(cfg):
    tensors = gu.make_tensors(cfg)
    spec = config_from_dict(cfg).to_spec()
    expected = {e.names[0]: tuple(e.rule.shapes[0]) for e in expected_tensors(spec)}
    assert set(expected) == set(tensors)
    for name, shape in expected.items():
        assert tuple(tensors[name].shape) == shape, name


def test_run_order_and_token_input():
    spec = config_from_dict(gu.TINY_ALL).to_spec()
    assert [c.layer for c in spec.schedule] == [0, 1, 2, 3]
    assert [dict(c.after.args) for c in spec.schedule] == [{"layer": i} for i in range(4)]
    assert all(c.before is None for c in spec.schedule)
    assert len(spec.stream_parts) == 1 and spec.stream_parts[0].kind == "token_side"
    assert spec.stream_parts[0].params["dim"] == 8 and spec.stream_parts[0].params["scale"] == 0.5
    # a layer without a feed-forward may carry its second norm
    assert spec.ignored_tensors == ("l2.norm2",)
    other = config_from_dict(gu.TINY_OTHER).to_spec()
    assert other.stream_parts == () and all(c.after is None for c in other.schedule)
    # the two forms have caches of their own sizes: one plane of latent + rotated part
    from zig_ai_amd.parts import lookup
    needs = [lookup("mixer", l.parts["mixer"].kind).cache_need(l.parts["mixer"].params)
             for l in spec.layers]
    assert [n.planes for n in needs] == [((1, 40),), ((1, 40),), ((1, 40),), ((1, 16),)]


def test_constants_reach_the_parts():
    spec = config_from_dict(gu.TINY_ALL).to_spec()
    a = spec.layers[0].parts["mixer"].params
    assert a["gate"] == "element" and a["sink"] and a["rotated_dim"] == 8
    assert a["position"].params == {"head_dim": 8, "rotary_dim": 8, "theta": 300.0,
                                    "pairing": "adjacent"}
    assert a["softmax_scale"] == gu.TINY_ALL["layers"][0]["mixer"]["scale"]
    b = spec.layers[1].parts["mixer"].params
    assert b["gate"] == "head" and b["rotated_dim"] == 0 and b["position"] is None
    part = config_from_dict(gu.TINY_OTHER).to_spec().layers[1].parts["mixer"].params
    assert part["rotated_dim"] == 24 and part["position"].params["rotary_dim"] == 8
    ff = spec.layers[3].parts["feed_forward"]
    assert ff.kind == "routed_experts"
    assert (ff.params["experts"], ff.params["identity_experts"], ff.params["top"]) == (6, 2, 4)
    assert (ff.params["groups"], ff.params["groups_kept"]) == (4, 2)
    assert ff.params["route_scale"] == 2.5 and ff.params["shared_size"] == 24
    assert ff.params["scores"] == "softmax" and not ff.params["renormalize"]
    assert "shared.token_gate.weight" in ff.tensors and "experts.5.down.weight" in ff.tensors
    lone = spec.layers[1].parts["feed_forward"]
    assert lone.params["shared_size"] == 0 and "shared.gate.weight" not in lone.tensors
    assert spec.layers[2].arrangement == "scaled_residual_no_ff"
    assert spec.layers[0].arrangement == "scaled_residual"
    assert spec.layers[0].params == {"residual_scale": 0.5}
    assert spec.embedding.params["norm"] and spec.embedding.tensors["norm.weight"] == ("embed.norm",)
    assert not spec.lm_head.params["tied"] and spec.lm_head.params["softcap"] == 12.0
    assert spec.final_norm.kind == "rms_norm"


@pytest.mark.parametrize("breakage", [
    lambda c: c["layers"][0].update(type="attention"),
    lambda c: c["layers"][0]["mixer"].pop("kv_rank"),
    lambda c: c["layers"][0]["mixer"].pop("rot"),
    lambda c: c["layers"][0]["mixer"]["rot"].update(dims=10),
    lambda c: c["layers"][1]["mixer"].update(rot_dim=8),
    lambda c: c["layers"][0]["mlp"]["router"].update(top=9),
    lambda c: c["layers"][0]["mlp"]["router"].update(groups={"count": 4, "keep": 2}),
    lambda c: c["layers"][0]["mlp"]["router"].update(groups={"count": 3, "keep": 4}),
    lambda c: c["layers"][3]["mlp"]["router"].update(groups={"count": 4, "keep": 1}),
    lambda c: c["layers"][0]["mlp"].update(kind="dense"),
    lambda c: c.update(token_side={}),
    lambda c: c.pop("norm"),
    lambda c: c.update(layers=[]),
])
def test_malformed_configurations(breakage):
    cfg = copy.deepcopy(gu.TINY_ALL)
    breakage(cfg)
    with pytest.raises(ConfigError):
        config_from_dict(cfg)


def test_random_model_folder(tmp_path):
    from zig_ai_amd.weights.random_init import write_random_model
    from zig_ai_amd.weights.safetensors_io import Checkpoint
    write_random_model(gu.TINY_ALL, str(tmp_path), seed=3)
    ckpt = Checkpoint(str(tmp_path))
    assert set(ckpt.names()) == set(gu.make_tensors(gu.TINY_ALL))
    assert tuple(ckpt.shape("side.embed")) == (gu.TINY_ALL["vocab"], 4 * 8)


# ----------------------------------------------- what pins the plain implementation
def test_rotation_in_adjacent_pairs_depends_on_distance_only():
    g = torch.Generator().manual_seed(1)
    q = torch.randn(1, 12, generator=g, dtype=torch.float64)
    k = torch.randn(1, 12, generator=g, dtype=torch.float64)
    def dot(pq, pk):
        return float((plain.rotate_pairs(q, torch.tensor([pq]), 8, 100.0)
                      * plain.rotate_pairs(k, torch.tensor([pk]), 8, 100.0)).sum())
    assert abs(dot(17, 5) - dot(112, 100)) < 1e-9
    assert abs(dot(17, 5) - dot(18, 5)) > 1e-3
    r = plain.rotate_pairs(q, torch.tensor([3]), 8, 100.0)
    assert torch.equal(r[:, 8:], q[:, 8:])                      # the rest passes unchanged
    # the first pair turns by the position itself (frequency 1): (u, v) -> (u cos - v sin, ...)
    u, v = float(q[0, 0]), float(q[0, 1])
    assert abs(float(r[0, 0]) - (u * math.cos(3) - v * math.sin(3))) < 1e-12
    assert abs(float(r[0, 1]) - (v * math.cos(3) + u * math.sin(3))) < 1e-12
    # position 0 changes nothing
    assert torch.allclose(plain.rotate_pairs(q, torch.tensor([0]), 8, 100.0), q)


def test_sink_softmax():
    s = torch.tensor([[0.3, -1.0, 2.0]], dtype=torch.float64)
    far_below = plain.sink_softmax(s, torch.tensor(-80.0, dtype=torch.float64))
    assert torch.allclose(far_below, torch.softmax(s, dim=-1))
    far_above = plain.sink_softmax(s, torch.tensor(80.0, dtype=torch.float64))
    assert float(far_above.sum()) < 1e-30
    w = plain.sink_softmax(s, torch.tensor(0.7, dtype=torch.float64))
    total = math.exp(0.3) + math.exp(-1.0) + math.exp(2.0) + math.exp(0.7)
    assert abs(float(w[0, 2]) - math.exp(2.0) / total) < 1e-12
    assert abs(float(w.sum()) - (1.0 - math.exp(0.7) / total)) < 1e-12


def test_latent_attention_is_an_attention_over_expanded_keys():
    # one head, no rotation: against the library's attention on the expanded keys and values
    # with the sink as one more key whose value is zero
    cfg = gu.one_layer("latent_attention_2", gu.plain_latent(heads=1, dim=8, vdim=8, kv_rank=16,
                                                             q_rank=8, scale=0.4), side=0)
    t = gu.make_tensors(cfg, seed=2)
    h = torch.randn(9, cfg["width"], dtype=torch.float64, generator=torch.Generator().manual_seed(5))
    m, eps, p = cfg["layers"][0]["mixer"], 1e-5, "l0.mix."
    got = plain.latent_attention(h, t, p, m, eps, rotated=False)
    W = lambda n: t[p + n].double()
    cq = plain.rms_norm(h @ W("dq").T, W("dq.norm"), eps)
    q = cq @ W("uq").T
    c = plain.rms_norm(h @ W("dkv").T, W("dkv.norm"), eps)
    k, v = c @ W("uk").T, c @ W("uv").T
    out = torch.zeros(9, 8, dtype=torch.float64)
    for i in range(9):
        logits = torch.cat([(k[:i + 1] @ q[i]) * 0.4, W("sink")])
        w = torch.softmax(logits, dim=0)[:-1]
        out[i] = w @ v[:i + 1]
    want = (out * torch.sigmoid(h @ W("g").T)) @ W("o").T
    assert torch.allclose(got, want, atol=1e-10)


def test_the_router_obeys_groups_corrections_and_identity():
    W = 8
    t = {"r.router": torch.eye(6, W), "r.correction": torch.zeros(6)}
    h = torch.tensor([[3.0, 2.9, 0.0, 0.0, 2.0, 1.0, 0, 0]], dtype=torch.float64)
    router = {"experts": 6, "identity": 0, "top": 2, "scale": 2.0}
    chosen, w = plain.route(h, t, "r.", router)
    s = torch.softmax(h[0, :6], dim=0)
    assert chosen.tolist() == [[0, 1]]
    assert torch.allclose(w[0], 2.0 * s[[0, 1]])                # times scale, not renormalised
    # three groups of two of which one is kept: both must come from the best group ...
    chosen, _ = plain.route(h, t, "r.", dict(router, groups={"count": 3, "keep": 1}))
    assert chosen.tolist() == [[0, 1]]
    # ... which a correction can change, while the weights stay the uncorrected scores
    t["r.correction"] = torch.tensor([0.0, 0.0, 0.0, 0.0, 0.9, 0.0])
    chosen, w = plain.route(h, t, "r.", dict(router, groups={"count": 3, "keep": 1}))
    assert chosen.tolist() == [[4, 5]]
    assert torch.allclose(w[0], 2.0 * s[[4, 5]])
    # a closed group's experts count as minus infinity, also against negative choice scores
    t["r.correction"] = torch.tensor([-5.0, -5.0, -9.0, -9.0, -5.0, -9.0])
    chosen, _ = plain.route(h, t, "r.", dict(router, groups={"count": 3, "keep": 1}))
    assert sorted(chosen[0].tolist()) == [0, 1]
    # an identity expert hands the input on, times its weight
    cfg = {"router": {"experts": 0, "identity": 6, "top": 1, "scale": 3.0}}
    t["r.correction"] = torch.zeros(6)
    y = plain.routed_experts(h, t, "r.", cfg)
    assert torch.allclose(y, 3.0 * s[0] * h)


def test_token_input_and_capped_logits():
    cfg = gu.one_layer("latent_attention_2", gu.plain_latent(), side=8)
    t = gu.make_tensors(cfg, seed=1)
    x = torch.randn(3, cfg["width"], dtype=torch.float64, generator=torch.Generator().manual_seed(2))
    y = plain.token_side(x, [4, 9, 4], t, 0, 8, 1e-5)
    assert abs(float((y[0] / t["l0.side.norm"].double()).pow(2).mean()) - 1.0) < 1e-3
    z = torch.tensor([0.5, -2.0], dtype=torch.float64)
    want = torch.nn.functional.gelu(z, approximate="tanh")
    assert torch.allclose(plain.gelu_tanh(z), want, atol=1e-12)
    # the cap bounds the logits and leaves small ones nearly alone
    toks = gu.tokens(5, cfg["vocab"], 1)
    capped = plain.forward(cfg, t, toks)
    free = plain.forward(dict(cfg, logit_softcap=0.0), t, toks)
    assert float(capped.abs().max()) < cfg["logit_softcap"]
    assert torch.allclose(capped, cfg["logit_softcap"] * torch.tanh(free / cfg["logit_softcap"]))
