"""Small Nopozen configurations and weights for tests, made here: none of them is a model
anybody ships.  The weights are drawn so that faults show: attention scores spread over
several units (so a key more or less, or a sink left out, moves the result), decays from
fast to very slow, router biases that matter, norms away from one."""

import json
import os
import tempfile

import torch

FOLDERS = {}


def lightning(heads=3, dim=16, vdim=24, decay=None):
    return {"heads": heads, "dim": dim, "vdim": vdim,
            "decay": list(decay) if decay is not None
            else [1.0 - 2.0 ** -(2 + 3 * h) for h in range(heads)]}


def rot(dims, base=300.0, scaling=None):
    out = {"dims": dims, "base": base}
    if scaling:
        out["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return out


def attention(heads=4, kv_heads=2, dim=16, vdim=None, scale=0.5, chunk=12, rot_dims=None,
              base=300.0, scaling=(4.0, 1.0, 3.0, 40)):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim or dim, "scale": scale}
    if rot_dims != 0:
        out["rot"] = rot(rot_dims or dim, base, scaling)
    if chunk:
        out["mask"] = {"size": chunk}
    return out


def attention_2(heads=6, kv_heads=3, dim=24, vdim=16, scale=0.4, conv=3, rot_dims=8, base=5000.0):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
            "conv": conv, "rot": rot(rot_dims, base)}


def dense(ff=72):
    return {"kind": "dense", "ff": ff}


def moe(ff=24, experts=5, top=2):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def layer(kind, mixer, mlp=None):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def config(layers, width=48, vocab=131, eps=1e-5, loop=None):
    out = {"architecture": "Nopozen", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "layers": layers}
    if loop is not None:
        out["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return out


# all three mixers, both kinds of feed-forward (and none), a loop over the middle that starts
# behind the first layer and runs three times; sizes differ wherever two could be equal
TINY_ALL = config([
    layer("attention", attention(), dense()),
    layer("lightning", lightning(), moe()),
    layer("attention_2", attention_2(), None),
    layer("attention", attention(heads=6, kv_heads=1, dim=8, vdim=24, scale=0.8, chunk=7,
                                 rot_dims=4, base=50.0, scaling=None), moe(ff=16, experts=3, top=1)),
    layer("lightning", lightning(heads=2, dim=24, vdim=8), dense(40)),
], loop=(1, 4, 3))

# another order and other sizes: no loop at all, one head, top = experts, a filter of one
# tap and one of five, a chunk of one token, whole rotation, no frequency scaling
TINY_OTHER = config([
    layer("attention_2", attention_2(heads=1, kv_heads=1, dim=32, vdim=32, scale=0.2, conv=1,
                                     rot_dims=32, base=10000.0), dense(56)),
    layer("lightning", lightning(heads=1, dim=32, vdim=32, decay=[0.96875]), None),
    layer("attention", attention(heads=3, kv_heads=3, dim=16, scale=0.45, chunk=1, scaling=None),
          moe(ff=32, experts=2, top=2)),
    layer("attention_2", attention_2(heads=4, kv_heads=2, dim=8, vdim=40, scale=0.7, conv=5,
                                     rot_dims=2, base=20.0), moe(ff=8, experts=1, top=1)),
    layer("attention", attention(heads=2, kv_heads=1, dim=40, vdim=8, scale=0.3, chunk=1000,
                                 rot_dims=20), None),
], width=40, vocab=67, eps=1e-6)

# a loop that is the whole model and runs once, and one that runs twice from layer 0
TINY_LOOP_ONCE = config([layer("lightning", lightning(), dense(24)),
                         layer("attention_2", attention_2(), None)], loop=(0, 2, 1))
TINY_LOOP_TWICE = config([layer("attention_2", attention_2(), moe()),
                          layer("attention", attention(), dense(24))], loop=(0, 1, 2))


def one_layer(kind, mixer, mlp=None, **kw):
    return config([layer(kind, mixer, mlp)], **kw)


def make_tensors(cfg, seed=0):
    """name -> float32 tensor (values representable in bfloat16) for ``cfg``."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def normal(*shape, std=1.0, mean=0.0):
        t = torch.randn(*shape, generator=g) * std + mean
        return t.to(torch.bfloat16).to(torch.float32)

    out = {"embed": normal(V, W), "final.norm": normal(W, std=0.3, mean=1.0),
           "head": normal(V, W, std=W ** -0.5)}
    if cfg.get("loop"):
        mix = normal(W, 2 * W, std=(2 * W) ** -0.5) \
            + torch.cat([torch.eye(W), torch.zeros(W, W)], dim=1) * 0.5
        out["loop.in"] = mix.to(torch.bfloat16).to(torch.float32)
    for i, lay in enumerate(cfg["layers"]):
        p, m = f"l{i}.", lay["mixer"]
        out[p + "norm1"] = normal(W, std=0.3, mean=1.0)
        if lay["type"] == "lightning":
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            out[p + "mix.q"] = normal(H * d, W, std=2.0 * W ** -0.5)
            out[p + "mix.k"] = normal(H * d, W, std=2.0 * W ** -0.5)
            out[p + "mix.v"] = normal(H * dv, W, std=W ** -0.5)
            out[p + "mix.g"] = normal(H * dv, W, std=2.0 * W ** -0.5)
            out[p + "mix.norm"] = normal(H * dv, std=0.3, mean=1.0)
            out[p + "mix.o"] = normal(W, H * dv, std=(H * dv) ** -0.5)
        else:
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out[p + "mix.q"] = normal(H * d, W, std=2.0 * W ** -0.5)
            out[p + "mix.k"] = normal(G * d, W, std=2.0 * W ** -0.5)
            out[p + "mix.v"] = normal(G * dv, W, std=W ** -0.5)
            out[p + "mix.o"] = normal(W, H * dv, std=(H * dv) ** -0.5)
            if lay["type"] == "attention":
                out[p + "mix.g"] = normal(H, W, std=2.0 * W ** -0.5)
                for n, rows in (("q", H * d), ("k", G * d), ("v", G * dv), ("o", W)):
                    out[p + f"mix.{n}.b"] = normal(rows, std=0.5)
                out[p + "mix.q.norm"] = normal(d, std=0.3, mean=1.5)
                out[p + "mix.k.norm"] = normal(d, std=0.3, mean=1.5)
            else:
                out[p + "mix.g"] = normal(H * dv, W, std=2.0 * W ** -0.5)
                for n, rows in (("q", H * d), ("k", G * d), ("v", G * dv)):
                    out[p + f"mix.{n}.conv"] = normal(rows, m["conv"], std=0.6, mean=0.3)
        mlp = lay["mlp"]
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            F = mlp["ff"]
            out[p + "mlp.up"] = normal(F, W, std=2.0 * W ** -0.5)
            out[p + "mlp.down"] = normal(W, F, std=F ** -0.5)
        else:
            F, E = mlp["expert"]["ff"], mlp["router"]["experts"]
            for e in range(E):
                out[f"{p}mlp.e{e}.gate"] = normal(F, W, std=2.0 * W ** -0.5)
                out[f"{p}mlp.e{e}.up"] = normal(F, W, std=2.0 * W ** -0.5)
                out[f"{p}mlp.e{e}.down"] = normal(W, F, std=2.0 * F ** -0.5)
            out[p + "mlp.router"] = normal(E, W, std=3.0 * W ** -0.5)
            out[p + "mlp.router.b"] = normal(E, std=1.5)
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
    d = tempfile.mkdtemp(prefix="nopozen_model_")
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in tensors.items()},
              os.path.join(d, "model.safetensors"))
    if key is not None:
        FOLDERS[key] = (d, tensors)
    return d, tensors


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(2000 + seed)
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

    def rand_lightning():
        heads = pick(1, 2, 3, 5)
        return lightning(heads=heads, dim=pick(8, 16, 24, 40, 72), vdim=pick(8, 16, 24, 40),
                         decay=[pick(0.5, 0.9, 0.96875, 0.99951171875, 1.0) for _ in range(heads)])

    def rand_attention():
        kv, dim = pick(1, 2, 3), pick(16, 32, 48, 64)
        return attention(heads=kv * pick(1, 2, 4), kv_heads=kv, dim=dim, vdim=pick(8, 16, dim),
                         scale=pick(0.1, 0.35, 0.7), chunk=pick(1, 3, 16, 50, 64, 300),
                         rot_dims=pick(2, dim // 2, dim), base=pick(10.0, 1000.0, 5e5),
                         scaling=pick(None, (8.0, 1.0, 4.0, 64), (2.0, 0.5, 8.0, 16)))

    def rand_attention_2():
        kv, dim = pick(1, 2, 3), pick(8, 16, 24, 64)
        return attention_2(heads=kv * pick(1, 2, 3), kv_heads=kv, dim=dim, vdim=pick(8, 24, dim),
                           scale=pick(0.1, 0.35, 0.7), conv=pick(1, 2, 3, 4, 6),
                           rot_dims=pick(2, dim // 2, dim), base=pick(10.0, 1000.0, 5e5))

    def rand_mlp():
        kind = pick("none", "dense", "moe", "moe")
        if kind == "none":
            return None
        if kind == "dense":
            return dense(pick(8, 24, 100))
        experts = pick(1, 2, 4, 9)
        return moe(ff=pick(8, 16, 40), experts=experts, top=pick(*range(1, min(experts, 4) + 1)))

    n = pick(1, 2, 3, 4)
    layers = []
    for _ in range(n):
        kind = pick("lightning", "attention", "attention_2")
        mixer = {"lightning": rand_lightning, "attention": rand_attention,
                 "attention_2": rand_attention_2}[kind]()
        layers.append(layer(kind, mixer, rand_mlp()))
    loop = None
    if pick(True, False):
        start = rng.randrange(n)
        loop = (start, rng.randrange(start + 1, n + 1), pick(1, 2, 3))
    return config(layers, width=pick(24, 40, 64, 96), vocab=pick(50, 131, 300),
                  eps=pick(1e-6, 1e-5), loop=loop)
