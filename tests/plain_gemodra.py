"""A plain, slow Gemodra: whole sequences, no cache, no batching, one function per
mechanism, on the CPU in float64.  It shares no code with the engine: it takes the
config.json dictionary and a mapping from tensor names to tensors.  The attention forms
every head's keys and values from the latent vectors (the engine never does: it folds the
two expansions into the query and the output).

Notation: ``h`` is a mixer's input ``[T, width]``; weights are ``[out, in]`` and applied
as ``h @ W.T``; positions count from 0.
"""

from __future__ import annotations

import math
from typing import List, Mapping, Optional

import torch

DT = torch.float64


def _w(tensors: Mapping[str, torch.Tensor], name: str) -> torch.Tensor:
    return tensors[name].to(DT)


# ------------------------------------------------------------------ small pieces
def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * w


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * torch.sigmoid(x)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """Rotary positions on the first ``dims`` elements of the last axis, element 2i paired
    with 2i + 1, angle = position * base^(-2i / dims).  ``x``: [T, ..., width]."""
    out = x.clone()
    i = torch.arange(dims // 2, dtype=DT)
    freq = torch.pow(torch.tensor(base, dtype=DT), -2.0 * i / dims)
    ang = positions.to(DT)[:, None] * freq[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def sink_softmax(s: torch.Tensor, sink: torch.Tensor) -> torch.Tensor:
    """Weights over the last axis of ``s`` (masked entries are -inf) whose denominator
    holds exp(sink) once more; they add up to less than one."""
    top = torch.maximum(s.max(dim=-1, keepdim=True).values, sink)
    e = torch.exp(s - top)
    return e / (e.sum(dim=-1, keepdim=True) + torch.exp(sink - top))


# ------------------------------------------------------------- latent attention
def latent_attention(h: torch.Tensor, tensors, p: str, m: Mapping, eps: float,
                     rotated: bool, positions: Optional[torch.Tensor] = None,
                     reach: int = 0) -> torch.Tensor:
    """Queries through a normed latent; keys and values of every head expanded from one
    normed latent a token; with ``rotated`` a rotated key part shared by all heads beside
    each head's unrotated one, and a gate an element; without, a gate a head.  ``reach``
    is 0; tests that ask whether a mask that is one token off would show set it to -1 (a
    query does not see itself) or 1 (it sees its successor)."""
    T = h.shape[0]
    H, d, dv, r = int(m["heads"]), int(m["dim"]), int(m["vdim"]), int(m["kv_rank"])
    dr = int(m["rot_dim"]) if rotated else 0
    pos = torch.arange(T) if positions is None else positions
    cq = rms_norm(h @ _w(tensors, p + "dq").T, _w(tensors, p + "dq.norm"), eps)
    q = (cq @ _w(tensors, p + "uq").T).view(T, H, d + dr)
    down = h @ _w(tensors, p + "dkv").T
    c = rms_norm(down[:, :r], _w(tensors, p + "dkv.norm"), eps)
    k = (c @ _w(tensors, p + "uk").T).view(T, H, d)
    v = (c @ _w(tensors, p + "uv").T).view(T, H, dv)
    q_plain, q_rot = q[..., :d], q[..., d:]
    if rotated:
        rot = m["rot"]
        q_rot = rotate_pairs(q_rot, pos, int(rot["dims"]), float(rot["base"]))
        k_rot = rotate_pairs(down[:, r:r + dr], pos, int(rot["dims"]), float(rot["base"]))
    sink = _w(tensors, p + "sink")
    causal = pos[None, :] <= pos[:, None] + reach
    out = torch.zeros((T, H, dv), dtype=DT)
    for hh in range(H):
        s = q_plain[:, hh] @ k[:, hh].T
        if rotated:
            s = s + q_rot[:, hh] @ k_rot.T
        s = (s * float(m["scale"])).masked_fill(~causal, -math.inf)
        out[:, hh] = sink_softmax(s, sink[hh]) @ v[:, hh]
    gate = torch.sigmoid(h @ _w(tensors, p + "g").T)
    if rotated:
        out = out.reshape(T, H * dv) * gate          # one number an element
    else:
        out = (out * gate[:, :, None]).reshape(T, H * dv)   # one number a head
    return out @ _w(tensors, p + "o").T


# ----------------------------------------------------------------- feed-forward
def gated_ff(h: torch.Tensor, tensors, p: str) -> torch.Tensor:
    a = silu(h @ _w(tensors, p + "gate").T) * (h @ _w(tensors, p + "up").T)
    return a @ _w(tensors, p + "down").T


def route(h: torch.Tensor, tensors, p: str, router: Mapping):
    """(chosen [T, top], weights [T, top]): softmax over all router outputs, the choice by
    score plus correction among the experts of the best groups, the weight the score itself
    times ``scale``."""
    z = h @ _w(tensors, p + "router").T
    s = torch.softmax(z, dim=-1)
    choice = s + _w(tensors, p + "correction")
    n = choice.shape[-1]
    groups = router.get("groups")
    if groups:
        count, keep = int(groups["count"]), int(groups["keep"])
        per = n // count
        best = choice.view(-1, count, per).max(dim=-1).values
        kept = best.topk(keep, dim=-1).indices
        allowed = torch.zeros_like(best, dtype=torch.bool).scatter_(1, kept, True)
        allowed = allowed[:, :, None].expand(-1, count, per).reshape(-1, n)
        choice = choice.masked_fill(~allowed, -math.inf)
    chosen = choice.topk(int(router["top"]), dim=-1).indices
    return chosen, s.gather(1, chosen) * float(router.get("scale", 1.0))


def routed_experts(h: torch.Tensor, tensors, p: str, mlp: Mapping) -> torch.Tensor:
    router = mlp["router"]
    n_identity = int(router.get("identity", 0))
    n_real = int(router["experts"])
    chosen, weights = route(h, tensors, p, router)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(chosen[t].tolist(), weights[t]):
            if e >= n_real:
                assert e < n_real + n_identity
                out[t] += w * h[t]
            else:
                out[t] += w * gated_ff(h[t:t + 1], tensors, f"{p}e{e}.")[0]
    if mlp.get("shared"):
        sg = torch.sigmoid(h @ _w(tensors, p + "shared.sg").T)          # [T, 1]
        out = out + sg * gated_ff(h, tensors, p + "shared.")
    return out


# ------------------------------------------------------------- per-layer input
def token_side(x: torch.Tensor, token_ids: List[int], tensors, i: int, dim: int, eps: float):
    """What layer ``i`` adds to the stream from the tokens themselves (before the block's
    weight): a slice of a second embedding, gated by the stream, projected and normed."""
    e = _w(tensors, "side.embed")[torch.tensor(token_ids)][:, i * dim:(i + 1) * dim]
    g = gelu_tanh(x @ _w(tensors, f"l{i}.side.gate").T) * e
    y = g @ _w(tensors, f"l{i}.side.proj").T
    return rms_norm(y, _w(tensors, f"l{i}.side.norm"), eps)


# ------------------------------------------------------------------- the model
def forward(config: Mapping, tensors: Mapping[str, torch.Tensor], token_ids: List[int],
            streams: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Logits [T, vocab] in float64.  ``streams`` receives the residual stream after
    every layer."""
    eps = float(config["norm"]["eps"])
    m = float(config.get("residual_mult", 1.0))
    side = config.get("token_side")
    x = rms_norm(_w(tensors, "embed")[torch.tensor(token_ids)], _w(tensors, "embed.norm"), eps)
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        h = rms_norm(x, _w(tensors, p + "norm1"), eps)
        if layer["type"] == "latent_attention":
            x = x + m * latent_attention(h, tensors, p + "mix.", layer["mixer"], eps, True)
        elif layer["type"] == "latent_attention_2":
            x = x + m * latent_attention(h, tensors, p + "mix.", layer["mixer"], eps, False)
        else:
            raise ValueError(layer["type"])
        mlp = layer.get("mlp")
        if mlp is not None:
            h = rms_norm(x, _w(tensors, p + "norm2"), eps)
            x = x + m * routed_experts(h, tensors, p + "mlp.", mlp)
        if side:
            x = x + m * token_side(x, token_ids, tensors, i, int(side["dim"]), eps)
        if streams is not None:
            streams.append(x.clone())
    x = rms_norm(x, _w(tensors, "final.norm"), eps)
    logits = x @ _w(tensors, "head").T
    cap = float(config.get("logit_softcap") or 0.0)
    return cap * torch.tanh(logits / cap) if cap else logits
