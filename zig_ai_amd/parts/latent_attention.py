"""Attention over one small latent vector a token, as a part (mixer ``latent_attention``).

Per token, with ``h`` the mixer's input:

  c_q = rmsnorm(Wdq h) * q_norm                     the query latent, ``q_rank`` wide
  q_i = Wuq c_q                                     per head [head_dim unrotated | rotated_dim rotated]
  [c' | k_r] = Wdkv h;  c = rmsnorm(c') * kv_norm   the latent, ``kv_rank`` wide; ``k_r`` (not
                                                    normed) is one rotated key part for all heads
  k_i = Wuk_i c,  v_i = Wuv_i c                     every head's keys and values
  s_ij = (q_i,n . k_j,i + rot(q_i,r) . rot(k_r,j)) * softmax_scale,  j <= i
  o_i = sum_j softmax(s_i, with exp(sink_i) in the denominator)_j v_j,i
  y   = Wo (o * sigmoid(Wg h))                      ``gate="element"``: a number an element of
                                                    o; ``"head"``: a number a head; None: none

Only ``[c | rot(k_r)]`` is cached, one plane of ``kv_rank + rotated_dim`` elements a token, and
keys and values are never formed: ``Wuk_i^T q_i,n`` is taken instead (the score against ``c``
is the same number) and ``Wuv_i`` is applied to ``sum_j p_j c_j``, so the attention kernel sees
one key/value head whose value is a prefix of its key (``csrc/latent.hip``).  bfloat16 rows of
16-byte pieces run on the matrix cores (work items of 64 rows; a step that only decodes takes the
kernel whose four waves share 16 rows, its contexts cut into ranges), everything else the
general kernel.

All sizes and constants come from ``params``: ``hidden_size, num_heads, head_dim,
rotated_dim`` (0: no positions), ``value_dim, kv_rank, q_rank, softmax_scale`` (None:
``(head_dim + rotated_dim)^-1/2``), ``norm_eps, sink`` (true: a tensor ``sink [num_heads]``),
``gate`` and ``position`` (a nested rotary spec whose ``head_dim`` is ``rotated_dim``; its
``rotary_dim`` may be smaller: the other elements of the rotated part pass unchanged).
"""

from __future__ import annotations

import math
from typing import Any, Dict, Mapping, Optional

import torch

from ..kernels import ops
from .attention import plan_split
from .base import Mixer, PagedNeed, Runtime, TensorRule, lookup, register_mixer
from .feed_forward import fuse_rows, pad_rows


LATENT_SPLIT_TARGET = 1024    # workgroups to reach by cutting contexts into ranges
LATENT_SPLIT_KEYS = 128       # keys of a range at least
LATENT_SPLIT_BYTES = 32 << 20  # the most that the ranges' partial results may take


def plan_latent_split(groups: int, max_keys: int):
    """(keys per range, number of ranges) for one launch of the matrix-core kernel: a function
    of the batch shape and of the longest context only.  A workgroup holds one or four waves
    and takes 32 keys a tile, so short ranges pay: as many as reach ``LATENT_SPLIT_TARGET``
    workgroups, of at least ``LATENT_SPLIT_KEYS`` keys each."""
    if groups >= LATENT_SPLIT_TARGET or max_keys <= 2 * LATENT_SPLIT_KEYS:
        return 0, 1
    nsplit = min(LATENT_SPLIT_TARGET // groups, max_keys // LATENT_SPLIT_KEYS, 64)
    if nsplit <= 1:
        return 0, 1
    keys = ((max_keys + nsplit - 1) // nsplit + 63) // 64 * 64
    nsplit = (max_keys + keys - 1) // keys
    return (keys, nsplit) if nsplit > 1 else (0, 1)


class LatentAttention(Mixer):
    kind = "latent_attention"
    graph_safe = True
    kernel_sources = ("gemm", "gemm_rows64", "latent", "norm", "activation")

    @staticmethod
    def _sizes(params):
        return tuple(int(params[k]) for k in ("hidden_size", "num_heads", "head_dim", "value_dim",
                                              "kv_rank", "q_rank")) \
            + (int(params.get("rotated_dim") or 0),)

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        H, nh, d, dv, R, Rq, dr = cls._sizes(params)
        rules = {"q_down.weight": TensorRule(((Rq, H),)),
                 "q_norm.weight": TensorRule(((Rq,),), role="norm"),
                 "q_up.weight": TensorRule(((nh * (d + dr), Rq),)),
                 "kv_down.weight": TensorRule(((R + dr, H),)),
                 "kv_norm.weight": TensorRule(((R,),), role="norm"),
                 "k_up.weight": TensorRule(((nh * d, R),)),
                 "v_up.weight": TensorRule(((nh * dv, R),)),
                 "out_proj.weight": TensorRule(((H, nh * dv),))}
        if params.get("sink"):
            rules["sink"] = TensorRule(((nh,),), role="bias")
        if params.get("gate") == "head":
            rules["gate_proj.weight"] = TensorRule(((nh, H),))
        elif params.get("gate") == "element":
            rules["gate_proj.weight"] = TensorRule(((nh * dv, H),))
        return rules

    @classmethod
    def cache_need(cls, params: Mapping[str, Any]):
        _, _, _, _, R, _, dr = cls._sizes(params)
        return PagedNeed(((1, R + dr),))

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        H, nh, d, dv, R, Rq, dr = self._sizes(params)
        self.num_heads, self.head_dim, self.value_dim = nh, d, dv
        self.kv_rank, self.q_rank, self.rotated_dim = R, Rq, dr
        self.width = R + dr                    # cached elements a token
        if params.get("gate") not in (None, "head", "element"):
            raise ValueError(f"gate must be None, 'head' or 'element', got {params.get('gate')!r}")
        self.gate = params.get("gate")
        if self.width > ops.LATENT_MAX_WIDTH or R > ops.LATENT_MAX_RANK:
            raise ValueError(f"a latent of {R} with {dr} rotated elements: the kernels take rows up "
                             f"to {ops.LATENT_MAX_WIDTH} and latents up to {ops.LATENT_MAX_RANK}")
        scale = params.get("softmax_scale")
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(d + dr)
        self.eps = float(params.get("norm_eps", 0.0))
        self.sink = tensors["sink"] if params.get("sink") else None
        pos = params.get("position")
        self.position = None
        self.rot_dims, self.adjacent, self.inv_freq = 0, False, None
        if dr:
            if pos is None:
                raise ValueError("a rotated part needs a position encoding")
            self.position = lookup("position", pos.kind)(pos.params, {}, runtime)
            if not getattr(self.position, "fused_rotation", False) or self.position.head_dim != dr:
                raise ValueError("the rotated part takes a rotary encoding of its own width")
            self.rot_dims = self.position.rotary_dim
            self.adjacent = self.position.pairing == "adjacent"
            self.inv_freq = self.position.inv_freq
        elif pos is not None:
            raise ValueError("a position encoding needs a rotated part")
        # the opening product: query latent | latent and rotated key part | gate, each
        # starting on a 16-byte boundary
        pieces = [pad_rows(tensors["q_down.weight"]), pad_rows(tensors["kv_down.weight"])]
        self.c_col = pieces[0].shape[0]
        self.gate_col = self.c_col + pieces[1].shape[0]
        if self.gate is not None:
            pieces.append(pad_rows(tensors["gate_proj.weight"]))
        self.w_open = ops.projection_weight(fuse_rows(*pieces))
        self.q_norm = tensors["q_norm.weight"]
        self.kv_norm = tensors["kv_norm.weight"]
        self.w_q_up = ops.projection_weight(tensors["q_up.weight"])
        self.w_out = ops.projection_weight(tensors["out_proj.weight"])
        # per head: Wuk^T as [R, d] (folds into the query), Wuv as [dv, R] (expands the result)
        k_up = tensors["k_up.weight"].view(nh, d, R).transpose(1, 2).contiguous()
        v_up = tensors["v_up.weight"].view(nh, dv, R).contiguous()
        # (the matrix-core form reads 16-byte pieces of its rows)
        if k_up.dtype == torch.bfloat16 and (d % 8 or (d + dr) % 8):
            k_up = k_up.float()
        if v_up.dtype == torch.bfloat16 and R % 8:
            v_up = v_up.float()
        self.k_fold, self.v_expand = k_up, v_up
        # bfloat16 rows of 16-byte pieces run on the matrix cores, in work items of 64 rows
        self.mfma = ops.latent_mfma_fits(runtime.dtype, self.width, R)
        most = ops.LATENT_MFMA_ROWS if self.mfma else ops.LATENT_MAX_ROWS
        self.rows_per_item = max(1, most // min(nh, most))
        self.item_granularities = [self.rows_per_item]
        for w, what in ((self.w_open, "w_open"), (self.w_q_up, "w_q_up"), (self.w_out, "w_out")):
            ops.check_projection_weight(w, "latent attention " + what)

    def forward(self, x, step, cache):
        nh, d, dv, R, dr = self.num_heads, self.head_dim, self.value_dim, self.kv_rank, self.rotated_dim
        T = x.shape[0]
        tune = self.runtime.tune
        plane = cache.planes[0]
        down = ops.linear(x, self.w_open, tune=tune)
        cq = ops.latent_prepare(down, 0, self.q_rank, self.c_col, R, dr, self.q_norm, self.kv_norm,
                                self.eps, step.positions, step.slot_mapping[cache.group],
                                self.inv_freq, self.rot_dims, self.adjacent,
                                plane if cache.writes else None)
        q = ops.linear(cq, self.w_q_up, tune=tune).view(T, nh, d + dr)
        # the folded query [Wuk^T q_n | rot(q_r)]
        qf = torch.empty((T, nh, self.width), dtype=q.dtype, device=q.device)
        ops.head_linear(q, 0, self.k_fold, out=qf, out_col=0)
        if dr:
            ops.rotate_part_(q, d, qf, R, dr, step.positions, self.inv_freq, self.rot_dims,
                             self.adjacent)
        item_seq, item_row0, item_count, n_items = step.attention_items(self.rows_per_item)
        waves = 0
        if self.mfma:
            # a step that only decodes: a wave a workgroup, heads in chunks of 16
            waves = 1 if step.n_tokens == step.n_seqs else 4
            keys, nsplit = plan_latent_split(n_items * (-(-nh // (16 * waves))), step.max_keys)
            # (the ranges' partial results are 32-bit rows of the latent's width: no cut where
            # they would be larger than the step is worth)
            if T * nh * nsplit * R * 4 > LATENT_SPLIT_BYTES:
                keys, nsplit = 0, 1
        else:
            keys, nsplit = plan_split(n_items, 1, step.max_keys)
        o = ops.latent_attention(qf, plane, R, step.block_tables[cache.group], step.positions,
                                 item_seq, item_row0, item_count, n_items, self.scale, self.sink,
                                 keys, nsplit, waves)
        # every head's result expanded by its Wuv, times the gate
        a = ops.head_linear(o, 0, self.v_expand, gate=down if self.gate else None,
                            gate_col=self.gate_col, gate_mode=self.gate)
        if getattr(step, "taps", None) is not None:
            step.taps["q"] = qf.clone()
            step.taps["o"] = a.clone()
        return ops.linear(a.view(T, nh * dv), self.w_out, tune=tune)


register_mixer(LatentAttention.kind, LatentAttention)
