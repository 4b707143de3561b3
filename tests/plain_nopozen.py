"""Nopozen in plain, slow PyTorch on the CPU: one function per mechanism, written from the
design's equations and sharing no code with the engine.  Everything runs in the dtype of
the tensors it is given (the tests hand it float64).

A model is ``(config, tensors)``: the config.json dictionary and a dictionary from tensor
names to tensors.  ``forward`` runs whole sequences; ``Walker`` runs a sequence token by
token from explicit caches and states, which is what pins the meaning of "carried".
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


# ------------------------------------------------------------------ small pieces
def rms_norm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def rotary_frequencies(rot: dict, dtype=torch.float64) -> torch.Tensor:
    """``f_i = base^(-2i/dims)``, and with ``scaling`` the three-band rule: short waves are
    kept, long waves divided by ``factor``, the band between blended."""
    dims = int(rot["dims"])
    f = torch.tensor([float(rot["base"]) ** (-2.0 * i / dims) for i in range(dims // 2)],
                     dtype=torch.float64)
    sc = rot.get("scaling")
    if sc:
        factor, low, high, orig = (float(sc[k]) for k in ("factor", "low", "high", "original"))
        out = []
        for fi in f.tolist():
            wave = 2.0 * math.pi / fi
            if wave < orig / high:
                out.append(fi)
            elif wave > orig / low:
                out.append(fi / factor)
            else:
                s = (orig / wave - low) / (high - low)
                out.append((1.0 - s) * fi / factor + s * fi)
        f = torch.tensor(out, dtype=torch.float64)
    return f.to(dtype)


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """``x [T, heads, dim]``; element ``i`` pairs with ``i + dims/2`` among the first ``dims``."""
    dims = int(rot["dims"])
    half = dims // 2
    f = rotary_frequencies(rot, x.dtype)
    a = positions.to(x.dtype)[:, None] * f[None, :]            # [T, half]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def causal_conv(u: torch.Tensor, w: torch.Tensor, before: Optional[torch.Tensor] = None):
    """``u [T, C]``, ``w [C, taps]``: ``y_t = sum_j w[:, j] u_(t - taps + 1 + j)``; ``before``
    holds the ``taps - 1`` inputs ahead of ``u`` (zeros at a sequence's start).  Returns
    ``(y, the last taps - 1 inputs)``."""
    taps = w.shape[1]
    if before is None:
        before = u.new_zeros((taps - 1, u.shape[1]))
    full = torch.cat([before, u], dim=0)
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + w[:, j][None, :] * full[j:j + u.shape[0]]
    return y, full[full.shape[0] - (taps - 1):]


# ------------------------------------------------------------------------ mixers
def softmax_attention(q, k, v, q_pos, k_pos, scale: float, chunk: int = 0, sink: bool = False):
    """``q [T, H, d]``, ``k [S, G, d]``, ``v [S, G, dv]``; query at ``q_pos`` sees keys with
    ``k_pos <= q_pos`` (and in the same chunk of ``chunk`` positions); ``sink``: one is added
    to the denominator."""
    T, H, d = q.shape
    G = k.shape[1]
    out = q.new_zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale                         # [T, S]
        ok = k_pos[None, :] <= q_pos[:, None]
        if chunk:
            ok = ok & ((k_pos[None, :] // chunk) == (q_pos[:, None] // chunk))
        s = s.masked_fill(~ok, float("-inf"))
        m = s.max(dim=1, keepdim=True).values
        if sink:
            m = torch.clamp(m, min=0.0)
        e = torch.exp(s - m)
        den = e.sum(dim=1, keepdim=True)
        if sink:
            den = den + torch.exp(-m)
        out[:, h] = (e / den) @ v[:, g]
    return out


def attention_mixer(h, p: str, W: Dict[str, torch.Tensor], m: dict, eps: float, positions,
                    cache: dict):
    """The mixer ``attention``: biased projections, per-head norm of q and k, rotation with
    scaled frequencies, chunked mask, a gate a head."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, d)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(T, G, d)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).view(T, G, dv)
    q = rms_norm(q, W[p + "q.norm"], eps)
    k = rms_norm(k, W[p + "k.norm"], eps)
    if m.get("rot"):
        q, k = rotate(q, positions, m["rot"]), rotate(k, positions, m["rot"])
    cache["k"] = k if "k" not in cache else torch.cat([cache["k"], k])
    cache["v"] = v if "v" not in cache else torch.cat([cache["v"], v])
    k_pos = torch.arange(cache["k"].shape[0])
    o = softmax_attention(q, cache["k"], cache["v"], positions, k_pos, float(m["scale"]),
                          chunk=int(m["mask"]["size"]) if m.get("mask") else 0)
    gate = torch.sigmoid(h @ W[p + "g"].T)                       # [T, H]
    o = o * gate[:, :, None]
    return o.reshape(T, H * dv) @ W[p + "o"].T + W[p + "o.b"]


def attention_2_mixer(h, p: str, W, m: dict, eps: float, positions, cache: dict):
    """The mixer ``attention_2``: no biases, a short convolution over time on q, k and v,
    partial rotation, every earlier key, a softmax with one more in the denominator, a gate
    an element."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    outs = []
    for name in ("q", "k", "v"):
        y, cache["conv." + name] = causal_conv(h @ W[p + name].T, W[p + name + ".conv"],
                                               cache.get("conv." + name))
        outs.append(y)
    q, k, v = outs[0].view(T, H, d), outs[1].view(T, G, d), outs[2].view(T, G, dv)
    q, k = rotate(q, positions, m["rot"]), rotate(k, positions, m["rot"])
    cache["k"] = k if "k" not in cache else torch.cat([cache["k"], k])
    cache["v"] = v if "v" not in cache else torch.cat([cache["v"], v])
    k_pos = torch.arange(cache["k"].shape[0])
    o = softmax_attention(q, cache["k"], cache["v"], positions, k_pos, float(m["scale"]), sink=True)
    o = o.reshape(T, H * dv) * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def lightning_mixer(h, p: str, W, m: dict, eps: float, cache: dict):
    """The mixer ``lightning``: ``S <- decay_h S + k v^T``, ``o = S^T q`` per head, then one
    norm over all heads, a gate an element, the output projection."""
    T = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(h @ W[p + "q"].T).view(T, H, d)
    k = silu(h @ W[p + "k"].T).view(T, H, d)
    v = silu(h @ W[p + "v"].T).view(T, H, dv)
    S = cache.get("S")
    if S is None:
        S = h.new_zeros((H, d, dv))
    decay = torch.tensor([float(x) for x in m["decay"]], dtype=h.dtype)
    o = h.new_zeros((T, H, dv))
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    cache["S"] = S
    y = rms_norm(o.reshape(T, H * dv), W[p + "norm"], eps) * torch.sigmoid(h @ W[p + "g"].T)
    return y @ W[p + "o"].T


# ----------------------------------------------------------------- feed-forwards
def dense_ff(h, p: str, W):
    return torch.relu(h @ W[p + "up"].T) ** 2 @ W[p + "down"].T


def moe_ff(h, p: str, W, mlp: dict):
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    z = h @ W[p + "router"].T + W[p + "router.b"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: (-float(z[t, e]), e))[:top]
        w = torch.softmax(z[t, order], dim=0)
        for wj, e in zip(w, order):
            pe = f"{p}e{e}."
            a = silu(h[t] @ W[pe + "gate"].T) * (h[t] @ W[pe + "up"].T)
            out[t] = out[t] + wj * (a @ W[pe + "down"].T)
    return out


# ------------------------------------------------------------------- whole model
def run_order(config: dict) -> List[tuple]:
    """``[(layer, first of a pass)]``: every layer once, the loop's span ``times`` times."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, False) for i in range(start)]
    for _ in range(times):
        order += [(i, i == start) for i in range(start, stop)]
    return order + [(i, False) for i in range(stop, n)]


class Walker:
    """A sequence's caches and states, one per entry of the run order; ``feed`` runs the next
    tokens (any number) and returns their logits and the stream after every layer run."""

    def __init__(self, config: dict, tensors: Dict[str, torch.Tensor], dtype=torch.float64):
        self.config = config
        self.W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}
        self.order = run_order(config)
        self.caches = [dict() for _ in self.order]
        self.fed = 0
        self.dtype = dtype

    def feed(self, tokens):
        c, W = self.config, self.W
        eps = float(c["norm"]["eps"])
        ids = torch.as_tensor(tokens, dtype=torch.long)
        positions = torch.arange(self.fed, self.fed + len(ids))
        self.fed += len(ids)
        x = W["embed"][ids]
        x0 = x
        streams = []
        for (i, first), cache in zip(self.order, self.caches):
            layer = c["layers"][i]
            if first:
                x = torch.cat([x, x0], dim=1) @ W["loop.in"].T
            h = rms_norm(x, W[f"l{i}.norm1"], eps)
            p = f"l{i}.mix."
            if layer["type"] == "attention":
                y = attention_mixer(h, p, W, layer["mixer"], eps, positions, cache)
            elif layer["type"] == "attention_2":
                y = attention_2_mixer(h, p, W, layer["mixer"], eps, positions, cache)
            elif layer["type"] == "lightning":
                y = lightning_mixer(h, p, W, layer["mixer"], eps, cache)
            else:
                raise ValueError(layer["type"])
            mlp = layer.get("mlp")
            if mlp:
                y = y + (dense_ff(h, f"l{i}.mlp.", W) if mlp["kind"] == "dense"
                         else moe_ff(h, f"l{i}.mlp.", W, mlp))
            x = x + y
            streams.append(x)
        logits = rms_norm(x, W["final.norm"], eps) @ W["head"].T
        return logits, torch.stack(streams)


def forward(config: dict, tensors: Dict[str, torch.Tensor], tokens, dtype=torch.float64):
    """Logits ``[T, vocab]`` and streams ``[layer runs, T, width]`` of one whole sequence."""
    return Walker(config, tensors, dtype).feed(tokens)
