"""Small Gemodra configurations and weights for tests, made here: none of them is a model
anybody ships.  The weights are drawn so that faults show: attention scores spread over
several units, sinks that take a visible share of a head's weight, router scores that are
far from flat with corrections large enough to change the choice, groups that shut out
experts that would otherwise win, a token input as large as the other branches."""

import json
import os
import tempfile

import torch

FOLDERS = {}


def latent(heads=3, dim=16, vdim=24, kv_rank=32, q_rank=24, rot_dim=8, base=300.0, scale=None,
           rot_dims=None):
    out = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
           "scale": scale if scale is not None else 2.0 * (dim + rot_dim) ** -0.5}
    if rot_dim:
        out["rot_dim"] = rot_dim
        out["rot"] = {"dims": rot_dim if rot_dims is None else rot_dims, "base": base}
    return out


def plain_latent(heads=2, dim=24, vdim=16, kv_rank=40, q_rank=16, scale=None):
    return latent(heads, dim, vdim, kv_rank, q_rank, rot_dim=0, scale=scale)


def moe(ff=24, experts=5, identity=1, top=2, groups=None, scale=1.5, shared=16):
    router = {"experts": experts, "identity": identity, "top": top, "scale": scale}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    out = {"kind": "moe", "router": router}
    if experts:
        out["expert"] = {"ff": ff}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def layer(kind, mixer, mlp=None):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def config(layers, width=48, vocab=131, eps=1e-5, mult=0.5, softcap=12.0, side=8):
    out = {"architecture": "Gemodra", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "residual_mult": mult, "layers": layers}
    if softcap:
        out["logit_softcap"] = softcap
    if side:
        out["token_side"] = {"dim": side}
    return out


# both mixers in turn, feed-forwards with and without groups, identity experts, a shared
# expert and a layer without feed-forward; sizes differ wherever two could be equal
TINY_ALL = config([
    layer("latent_attention", latent(), moe(groups=(3, 2))),
    layer("latent_attention_2", plain_latent(), moe(ff=16, experts=3, identity=0, top=1, shared=0)),
    layer("latent_attention", latent(heads=5, dim=8, vdim=8, kv_rank=24, q_rank=40, rot_dim=16,
                                     base=10000.0), None),
    layer("latent_attention_2", plain_latent(heads=1, dim=32, vdim=40, kv_rank=16, q_rank=8),
          moe(ff=8, experts=6, identity=2, top=4, groups=(4, 2), scale=2.5, shared=24)),
])

# another order and other sizes: the form without positions first, one head, all router
# outputs chosen, identity experts only beside one expert, no cap on the logits, no token
# input, a weight of one on the branches, a rotation of a part of the rotated elements
TINY_OTHER = config([
    layer("latent_attention_2", plain_latent(heads=4, dim=8, vdim=8, kv_rank=8, q_rank=32),
          moe(ff=40, experts=1, identity=2, top=3, scale=1.0, shared=8)),
    layer("latent_attention", latent(heads=1, dim=24, vdim=16, kv_rank=48, q_rank=16, rot_dim=24,
                                     base=50.0, rot_dims=8), moe(ff=32, experts=4, identity=0,
                                                                 top=2, groups=(2, 1), shared=0)),
    layer("latent_attention", latent(heads=2, dim=16, vdim=32, kv_rank=16, q_rank=16, rot_dim=2),
          None),
], width=40, vocab=67, eps=1e-6, mult=1.0, softcap=0.0, side=0)


def one_layer(kind, mixer, mlp=None, **kw):
    return config([layer(kind, mixer, mlp)], **kw)


def make_tensors(cfg, seed=0):
    """name -> float32 tensor (values representable in bfloat16) for ``cfg``."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def normal(*shape, std=1.0, mean=0.0):
        t = torch.randn(*shape, generator=g) * std + mean
        return t.to(torch.bfloat16).to(torch.float32)

    out = {"embed": normal(V, W), "embed.norm": normal(W, std=0.3, mean=1.0),
           "final.norm": normal(W, std=0.3, mean=1.0), "head": normal(V, W, std=2.0 * W ** -0.5)}
    side = cfg.get("token_side")
    if side:
        out["side.embed"] = normal(V, len(cfg["layers"]) * side["dim"])
    for i, lay in enumerate(cfg["layers"]):
        p, m = f"l{i}.", lay["mixer"]
        out[p + "norm1"] = normal(W, std=0.3, mean=1.0)
        H, d, dv, R, Rq = m["heads"], m["dim"], m["vdim"], m["kv_rank"], m["q_rank"]
        dr = m.get("rot_dim", 0)
        out[p + "mix.dq"] = normal(Rq, W, std=W ** -0.5)
        out[p + "mix.dq.norm"] = normal(Rq, std=0.3, mean=1.0)
        out[p + "mix.uq"] = normal(H * (d + dr), Rq, std=2.0 * Rq ** -0.5)
        out[p + "mix.dkv"] = normal(R + dr, W, std=W ** -0.5)
        out[p + "mix.dkv.norm"] = normal(R, std=0.3, mean=1.0)
        out[p + "mix.uk"] = normal(H * d, R, std=2.0 * R ** -0.5)
        out[p + "mix.uv"] = normal(H * dv, R, std=R ** -0.5)
        out[p + "mix.sink"] = normal(H, std=1.5, mean=1.0)
        gate_rows = H * dv if lay["type"] == "latent_attention" else H
        out[p + "mix.g"] = normal(gate_rows, W, std=2.0 * W ** -0.5)
        out[p + "mix.o"] = normal(W, H * dv, std=2.0 * (H * dv) ** -0.5)
        if side:
            out[p + "side.gate"] = normal(side["dim"], W, std=2.0 * W ** -0.5)
            out[p + "side.proj"] = normal(W, side["dim"], std=side["dim"] ** -0.5)
            out[p + "side.norm"] = normal(W, std=0.3, mean=1.0)
        mlp = lay["mlp"]
        if mlp is None:
            continue
        out[p + "norm2"] = normal(W, std=0.3, mean=1.0)
        r = mlp["router"]
        E, n = r["experts"], r["experts"] + r.get("identity", 0)
        out[p + "mlp.router"] = normal(n, W, std=3.0 * W ** -0.5)
        out[p + "mlp.correction"] = normal(n, std=0.3)
        for e in range(E):
            F = mlp["expert"]["ff"]
            out[f"{p}mlp.e{e}.gate"] = normal(F, W, std=2.0 * W ** -0.5)
            out[f"{p}mlp.e{e}.up"] = normal(F, W, std=2.0 * W ** -0.5)
            out[f"{p}mlp.e{e}.down"] = normal(W, F, std=2.0 * F ** -0.5)
        if mlp.get("shared"):
            S = mlp["shared"]["ff"]
            out[p + "mlp.shared.gate"] = normal(S, W, std=2.0 * W ** -0.5)
            out[p + "mlp.shared.up"] = normal(S, W, std=2.0 * W ** -0.5)
            out[p + "mlp.shared.down"] = normal(W, S, std=2.0 * S ** -0.5)
            out[p + "mlp.shared.sg"] = normal(1, W, std=2.0 * W ** -0.5)
    return out


def folder(cfg, seed=0, tensors=None):
    """A model folder (config.json, model.safetensors in bfloat16) in a temporary place;
    returns (folder, tensors)."""
    from safetensors.torch import save_file
    key = (json.dumps(cfg, sort_keys=True), seed) if tensors is None else None
    if key is not None and key in FOLDERS:
        return FOLDERS[key]
    if tensors is None:
        tensors = make_tensors(cfg, seed)
    d = tempfile.mkdtemp(prefix="gemodra_model_")
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in tensors.items()},
              os.path.join(d, "model.safetensors"))
    if key is not None:
        FOLDERS[key] = (d, tensors)
    return d, tensors


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(3000 + seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def row_error(got, want):
    """Per row: the root mean square of the difference (means taken off) relative to the
    root mean square of the wanted logits over all rows."""
    got, want = got.double(), want.double()
    assert got.shape == want.shape, (got.shape, want.shape)
    assert torch.isfinite(got).all(), "non-finite logits"
    d = got - want
    d = d - d.mean(dim=1, keepdim=True)
    scale = (want - want.mean(dim=1, keepdim=True)).pow(2).mean().sqrt()
    return d.pow(2).mean(dim=1).sqrt() / scale


def random_config(seed):
    """A configuration drawn at random: layer order, every size and every constant."""
    import random
    rng = random.Random(seed)

    def pick(*values):
        return rng.choice(values)

    def rand_mixer():
        if pick(True, False):
            rot = pick(2, 8, 16, 24)
            return "latent_attention", latent(
                heads=pick(1, 2, 3, 6), dim=pick(8, 16, 24, 40), vdim=pick(8, 16, 24, 48),
                kv_rank=pick(8, 24, 32, 72), q_rank=pick(8, 16, 56), rot_dim=rot,
                base=pick(10.0, 1000.0, 5e5), scale=pick(0.1, 0.3, 0.6),
                rot_dims=pick(rot, rot, max(2, rot // 4 * 2)))
        return "latent_attention_2", plain_latent(
            heads=pick(1, 2, 4, 7), dim=pick(8, 16, 32, 48), vdim=pick(8, 16, 40),
            kv_rank=pick(8, 16, 40, 64), q_rank=pick(8, 24, 32), scale=pick(0.1, 0.3, 0.6))

    def rand_mlp():
        if pick(True, True, True, False) is False:
            return None
        groups = pick(None, None, 1, 2, 3)
        per = pick(1, 2, 3)
        n = (groups or pick(1, 2, 4)) * per
        identity = rng.randrange(0, n)                 # at least one expert has weights
        keep = rng.randrange(1, groups + 1) if groups else 0
        most = keep * per if groups else n
        return moe(ff=pick(8, 16, 40), experts=n - identity, identity=identity,
                   top=rng.randrange(1, min(most, 4) + 1),
                   groups=(groups, keep) if groups else None, scale=pick(0.5, 1.0, 2.5),
                   shared=pick(0, 8, 24))

    n = pick(1, 2, 3, 4, 5)
    layers = [layer(*rand_mixer(), rand_mlp()) for _ in range(n)]
    return config(layers, width=pick(16, 24, 40, 64, 104), vocab=pick(11, 50, 203),
                  eps=pick(1e-6, 1e-5, 1e-3), mult=pick(0.25, 0.5, 1.0), softcap=pick(0.0, 5.0, 30.0),
                  side=pick(0, 8, 16))
