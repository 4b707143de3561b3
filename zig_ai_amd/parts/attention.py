"""Grouped-query attention over a paged cache, as a part.

Per token (/root/reference/src/transformer/hybrid_attn.zig:286-640):
  q, k, v = x Wq^T, x Wk^T, x Wv^T           (one fused projection, optional bias)
  q, k    = per-head RMSNorm(q), RMSNorm(k)  if ``qk_norm``   (371-382)
  q, k    = position encoding(q, k)          (rotary: fused into the same kernel)
  k, v   -> the request's pages
  o       = softmax(q k^T * scale, causal [, window]) v       (553-608)
  y       = o Wo^T

All sizes come from ``params``: ``hidden_size, num_heads, num_kv_heads,
head_dim, qk_norm, norm_eps, window`` (0 = all keys), ``softmax_scale`` (None =
1/sqrt(head_dim)), ``bias`` (true: on all four projections; ``"qkv"``: on the three
opening ones only) and ``position`` (a nested position-encoding spec or None).

Two more, for designs that need them: ``value_dim`` (values, and with them the
attention's output per head, of another width than queries and keys) and ``gate``
(``"head"``: every head's output is multiplied by ``sigmoid(x Wg^T)_h`` before the output
projection; the gate's rows ride along in the opening projection).  With either, the
cache is a plane of keys and a plane of values per page.

And what a design may do to the scores (``ops.ScoreShape``; every attention kernel takes
it): ``softcap`` (``s <- softcap * tanh(s / softcap)`` after the scale), ``sink`` (true: a
tensor ``sink [num_heads]`` whose exponential joins each head's softmax denominator once,
with no key and no value) and ``query_temperature`` (``(coef, every)``: the query at
position ``p`` is multiplied by ``1 + coef * ln(floor((p + 1) / every) + 1)``).
``values="keys"``: there is no value projection, a token's value is its key as projected
(the key rows of the opening projection are there a second time, so whatever stores
q | k | v rows finds the same numbers in the value columns).

Further: ``gate="element"`` (a sigmoid gate for every element of every head's output,
``gate_proj`` of ``num_heads * value_dim`` rows), ``chunk`` (positions are counted in chunks of
that many from the sequence's start and a query sees the earlier keys of its own chunk only;
0: none), ``sink_value`` (a number: every head's softmax denominator also holds its
exponential, a sink with a fixed score and no tensor) and ``conv`` (the number of taps of a
depth-wise causal convolution over time that q, k and v pass right behind their
projection, before norm and rotation; tensors ``q_conv.weight``, ``k_conv.weight``,
``v_conv.weight`` of ``[channels, taps]``, no bias, no activation; the last ``taps - 1``
projected rows of a request are kept in its state slot, so the mixer needs pages and a
state).  These go through the path that takes the cache as two planes: the matrix-core
kernels where the sizes fit (the gate then is a small kernel behind them), the general
attention kernel otherwise.

Head widths that are no multiple of 8 (what the kernels read at a time) are filled up with
zeros when the part is built: zero rows of the q, k and v projections (and of their biases and
filters), zero columns of the output projection; a score and a weighted sum do not change.
The per-head norm then divides by the padded width: with ``eps * d / d_pad`` for eps and the
norm's weight times ``sqrt(d / d_pad)`` the result is the same, ``x / sqrt(sum x^2 / d + eps) =
sqrt(d / d_pad) x / sqrt(sum x^2 / d_pad + eps d / d_pad)``.  More query heads a key head than a
work item of the kernels holds (``ops.ATTENTION_MAX_ROWS``) are served by key heads that are
there several times: the rows of the k and v projections are repeated until a group fits.
"""

from __future__ import annotations

import math
from typing import Any, Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import (Mixer, PagedNeed, PagedStateNeed, Runtime, StateNeed, TensorRule, lookup,
                   register_mixer)
from .feed_forward import fuse_rows, pad_rows

# Cutting long contexts pays only when the launch would otherwise leave most of the
# machine idle (decoding few requests, or a portion of a prompt far into a long
# request).  Measured on one MI355X with 8 key/value heads, contexts from 2,048 to
# 131,072 keys and 1 to 64 requests: from 512 workgroups on nothing is gained; below,
# as many ranges as still stay within SPLIT_TARGET workgroups (one decode workgroup of
# eight waves a compute unit) are best or within a few percent of it, all of the same length.
BUSY_WORKGROUPS = 512
SPLIT_TARGET = 256
SPLIT_KEYS_MIN = 512
SPLIT_MAX = 64


def plan_split(n_items: int, num_kv_heads: int, max_keys: int, target: int = SPLIT_TARGET):
    """(keys per range, number of ranges) for one launch; a function of the batch
    shape and of the longest context only.  ``target``: workgroups to reach (the
    kernel for prompt portions runs two workgroups per compute unit and wants 512)."""
    groups = n_items * num_kv_heads
    # (a range of 512 keys is one tile for each of the decode kernel's eight waves; short
    # contexts are cut finer: decoding one request at 512 keys, 4 ranges 0.692 ms a step,
    # none 0.707; at 8,192 keys ranges of 512 0.745, of 256 0.774)
    keys_min = SPLIT_KEYS_MIN if max_keys > 4 * SPLIT_KEYS_MIN else SPLIT_KEYS_MIN // 2
    if groups >= BUSY_WORKGROUPS or max_keys <= 2 * keys_min:
        return 0, 1
    # as many ranges as keep the launch within `target` workgroups (one more range would send
    # part of them into a second round: 12 requests at 2,048 keys, 2 ranges 0.862 ms a step, 3
    # ranges 0.878; 20 requests uncut 1.18, in 2 ranges 1.27)
    wanted = target // groups
    nsplit = min(wanted, max_keys // keys_min, SPLIT_MAX)
    if nsplit <= 1:
        return 0, 1
    keys = ((max_keys + nsplit - 1) // nsplit + 63) // 64 * 64   # a multiple of the key tile
    nsplit = (max_keys + keys - 1) // keys
    return (keys, nsplit) if nsplit > 1 else (0, 1)


def _round_up8(n: int) -> int:
    return -(-int(n) // 8) * 8


def _kv_repeat(num_heads: int, num_kv_heads: int) -> int:
    """How many times every key head is kept so that its group of query heads fits a work
    item: the smallest divisor ``r`` of the group with ``group / r <= ATTENTION_MAX_ROWS``."""
    group = num_heads // max(1, num_kv_heads)
    for r in range(1, group + 1):
        if group % r == 0 and group // r <= ops.ATTENTION_MAX_ROWS:
            return r
    return 1


def _repeat_heads(w: torch.Tensor, heads: int, times: int) -> torch.Tensor:
    """``w [heads * width, ...]`` with every head's rows ``times`` times in a row."""
    if times == 1:
        return w
    rest = tuple(w.shape[1:])
    return w.reshape((heads, -1) + rest).repeat_interleave(times, dim=0) \
        .reshape((-1,) + rest).contiguous()


def _pad_heads(w: torch.Tensor, heads: int, width: int, padded: int) -> torch.Tensor:
    """``w [heads * width, ...]`` -> ``[heads * padded, ...]``: zero rows behind every head's."""
    if padded == width:
        return w
    rest = tuple(w.shape[1:])
    w = w.reshape((heads, width) + rest)
    return torch.cat([w, w.new_zeros((heads, padded - width) + rest)], dim=1) \
        .reshape((heads * padded,) + rest).contiguous()


class GroupedQueryAttention(Mixer):
    kind = "gqa_attention"
    graph_safe = True
    takes_stream = True
    kernel_sources = ("gemm", "gemm_rows64", "rope_kv", "attention", "norm", "activation")

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        H, nh, nkv, d = (int(params[k]) for k in
                         ("hidden_size", "num_heads", "num_kv_heads", "head_dim"))
        dv = int(params.get("value_dim") or d)
        rules = {"q_proj.weight": TensorRule(((nh * d, H),)),
                 "k_proj.weight": TensorRule(((nkv * d, H),)),
                 "v_proj.weight": TensorRule(((nkv * dv, H),)),
                 "out_proj.weight": TensorRule(((H, nh * dv),))}
        if params.get("values") == "keys":
            del rules["v_proj.weight"]
        if params.get("sink"):
            rules["sink"] = TensorRule(((nh,),), role="bias")
        if params.get("gate") == "head":
            rules["gate_proj.weight"] = TensorRule(((nh, H),))
        elif params.get("gate") == "element":
            rules["gate_proj.weight"] = TensorRule(((nh * dv, H),))
        taps = int(params.get("conv") or 0)
        if taps:
            rules["q_conv.weight"] = TensorRule(((nh * d, taps),), role="filter")
            rules["k_conv.weight"] = TensorRule(((nkv * d, taps),), role="filter")
            rules["v_conv.weight"] = TensorRule(((nkv * dv, taps),), role="filter")
        if params.get("qk_norm"):
            rules["q_norm.weight"] = TensorRule(((d,),), role="norm")
            rules["k_norm.weight"] = TensorRule(((d,),), role="norm")
        if params.get("bias"):
            rules["q_proj.bias"] = TensorRule(((nh * d,),), role="bias")
            rules["k_proj.bias"] = TensorRule(((nkv * d,),), role="bias")
            rules["v_proj.bias"] = TensorRule(((nkv * dv,),), role="bias")
            if params["bias"] != "qkv":
                rules["out_proj.bias"] = TensorRule(((H,),), role="bias")
        return rules

    @classmethod
    def cache_need(cls, params: Mapping[str, Any]):
        nkv, d = int(params["num_kv_heads"]), int(params["head_dim"])
        nkv *= _kv_repeat(int(params["num_heads"]), nkv)    # (as they lie in the cache)
        dv = _round_up8(params.get("value_dim") or d)       # (filled up)
        d = _round_up8(d)
        if dv == d:
            paged = PagedNeed.kv(nkv, d, int(params.get("window") or 0))
        else:
            paged = PagedNeed(((nkv, d), (nkv, dv)), int(params.get("window") or 0))
        taps = int(params.get("conv") or 0)
        if not taps:
            return paged
        # the convolution's last inputs, [channel][taps - 1] 32-bit floats a request
        channels = (int(params["num_heads"]) + nkv) * d + nkv * dv
        return PagedStateNeed(paged, StateNeed((max(1, channels * (taps - 1)),)))

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        self.num_heads = int(params["num_heads"])
        self.num_kv_heads = int(params["num_kv_heads"])
        if self.num_heads % self.num_kv_heads:
            raise ValueError(f"{self.num_heads} heads do not divide into {self.num_kv_heads} groups")
        self.group = self.num_heads // self.num_kv_heads
        # the widths as the model has them, and as the kernels see them
        self.model_head_dim = int(params["head_dim"])
        self.model_value_dim = int(params.get("value_dim") or self.model_head_dim)
        self.head_dim, self.value_dim = _round_up8(self.model_head_dim), _round_up8(self.model_value_dim)
        norm_eps = float(params.get("norm_eps", 0.0))
        if (self.head_dim, self.value_dim) != (self.model_head_dim, self.model_value_dim):
            tensors, norm_eps = self._filled_up(params, tensors, norm_eps)
        repeat = _kv_repeat(self.num_heads, self.num_kv_heads)
        if repeat > 1:
            tensors = dict(tensors)
            for name in ("k_proj.weight", "k_proj.bias", "k_conv.weight", "v_proj.weight",
                         "v_proj.bias", "v_conv.weight"):
                if name in tensors:
                    tensors[name] = _repeat_heads(tensors[name], self.num_kv_heads, repeat)
            self.num_kv_heads *= repeat
            self.group //= repeat
        if params.get("gate") not in (None, "head", "element"):
            raise ValueError(f"attention gate must be None, 'head' or 'element', got "
                             f"{params.get('gate')!r}")
        self.gated = params.get("gate") in ("head", "element")
        self.gate_element = params.get("gate") == "element"
        self.chunk = int(params.get("chunk") or 0)
        self.taps = int(params.get("conv") or 0)
        if self.chunk < 0 or self.taps < 0 or self.taps > ops.CONV_MAX_TAPS:
            raise ValueError(f"chunk {self.chunk} and conv {self.taps}: neither negative, at most "
                             f"{ops.CONV_MAX_TAPS} taps")
        # values of their own width, a gate, chunks or a convolution: the kernels that take
        # the cache as two planes
        self.wide = self.gated or self.value_dim != self.head_dim or bool(self.chunk) \
            or bool(self.taps) or params.get("sink_value") is not None
        if self.value_dim % 8 or self.value_dim > 256:
            raise ValueError(f"value_dim {self.value_dim} must be a multiple of 8, at most 256")
        if self.group > ops.ATTENTION_MAX_ROWS:
            raise ValueError(f"{self.group} query heads per key/value head exceed the attention "
                             f"kernel's limit of {ops.ATTENTION_MAX_ROWS}")
        # (the general kernels read eight elements at a time)
        multiple = 8
        if self.head_dim % multiple or self.head_dim > 256:
            raise ValueError(f"head_dim {self.head_dim} must be a multiple of {multiple}, at most 256")
        # tokens per work item of the two attention kernels
        self.rows_per_item = max(1, ops.ATTENTION_MAX_ROWS // self.group)
        self.mfma_rows_per_item = max(1, ops.ATTENTION_MFMA_ROWS // self.group)
        self.mfma_decode_rows_per_item = max(1, ops.ATTENTION_MFMA_DECODE_ROWS // self.group)
        self.window = int(params.get("window") or 0)
        scale = params.get("softmax_scale")
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.model_head_dim)
        # whether the matrix-core kernels take these sizes (the page size is checked per step)
        self.mfma = ops.attention_mfma_supported(runtime.dtype, self.num_heads,
                                                 self.num_kv_heads, self.head_dim,
                                                 scale=self.scale)
        self.item_granularities = [self.rows_per_item] + (
            [self.mfma_rows_per_item, self.mfma_decode_rows_per_item] if self.mfma else [])
        self.eps = norm_eps
        if params.get("values") not in (None, "own", "keys"):
            raise ValueError(f"attention values must be 'own' or 'keys', got {params.get('values')!r}")
        self.shared_values = params.get("values") == "keys"
        if self.shared_values and (self.value_dim != self.head_dim or params.get("bias")):
            raise ValueError("values that are the keys have the keys' width and no bias")
        temperature = params.get("query_temperature")
        sink = tensors["sink"] if params.get("sink") else None
        if params.get("sink_value") is not None:
            if sink is not None:
                raise ValueError("a sink is a tensor or a fixed number, not both")
            sink = torch.full((self.num_heads,), float(params["sink_value"]), dtype=torch.float32,
                              device=runtime.device)
        self.shape = ops.ScoreShape(params.get("softcap") or 0.0, sink,
                                    tuple(temperature) if temperature else None, self.chunk)
        opening = [tensors["q_proj.weight"], tensors["k_proj.weight"],
                   tensors["k_proj.weight" if self.shared_values else "v_proj.weight"]]
        self.gate_col = (self.num_heads + self.num_kv_heads) * self.head_dim \
            + self.num_kv_heads * self.value_dim
        if self.gated:
            opening.append(tensors["gate_proj.weight"])
        self.w_qkv = fuse_rows(*opening)
        self.w_out = tensors["out_proj.weight"]
        if self.wide:
            self.w_qkv = ops.projection_weight(pad_rows(self.w_qkv))
            self.w_out = ops.projection_weight(self.w_out)
        elif self.shared_values or self.shape:
            self.w_qkv = ops.projection_weight(self.w_qkv)
            self.w_out = ops.projection_weight(self.w_out)
        self.b_qkv = self.b_out = None
        if params.get("bias"):
            b = torch.cat([tensors["q_proj.bias"], tensors["k_proj.bias"], tensors["v_proj.bias"]])
            self.b_qkv = torch.cat([b, b.new_zeros((self.w_qkv.shape[0] - b.numel(),))]).contiguous()
            self.b_out = tensors.get("out_proj.bias")
        self.conv_w = None
        if self.taps:
            self.conv_w = torch.cat([tensors["q_conv.weight"], tensors["k_conv.weight"],
                                     tensors["v_conv.weight"]], dim=0).contiguous()
        self.q_norm = tensors.get("q_norm.weight") if params.get("qk_norm") else None
        self.k_norm = tensors.get("k_norm.weight") if params.get("qk_norm") else None
        pos = params.get("position")
        self.position = None
        if pos is not None:
            self.position = lookup("position", pos.kind)(pos.params, {}, runtime)
        self.fused_rotation = bool(getattr(self.position, "fused_rotation", False))
        # recorded into a graph only if the position encoding, too, never looks at a
        # step's numbers on the host
        self.graph_safe = self.position is None or bool(getattr(self.position, "graph_safe", False))
        # a decode step's norm, rotation and cache write can run inside its attention kernel
        if self.wide and self.position is not None and not self.fused_rotation:
            raise ValueError("an attention with value_dim or gate takes a rotary position "
                             "encoding or none")
        self.mfma = self.mfma and self.value_dim == self.head_dim
        if not self.mfma:
            self.item_granularities = [self.rows_per_item]
        self.rotation_in_attention = (
            not self.wide and self.fused_rotation and runtime.dtype == torch.bfloat16
            and self.position.rotary_dim == self.head_dim and self.position.pairing != "adjacent")
        ops.check_projection_weight(self.w_qkv, "attention w_qkv")
        ops.check_projection_weight(self.w_out, "attention w_out")

    def _filled_up(self, params, tensors, eps: float):
        """The part's tensors with every head filled up with zeros to the kernels' widths, and
        the eps that goes with the padded per-head norm."""
        nh, nkv = self.num_heads, self.num_kv_heads
        d0, dv0, d, dv = self.model_head_dim, self.model_value_dim, self.head_dim, self.value_dim
        t = dict(tensors)
        for name, heads, w0, w1 in (("q", nh, d0, d), ("k", nkv, d0, d), ("v", nkv, dv0, dv)):
            for suffix in ("_proj.weight", "_proj.bias", "_conv.weight"):
                if name + suffix in t:
                    t[name + suffix] = _pad_heads(t[name + suffix], heads, w0, w1)
        if params.get("gate") == "element":
            t["gate_proj.weight"] = _pad_heads(t["gate_proj.weight"], nh, dv0, dv)
        t["out_proj.weight"] = _pad_heads(t["out_proj.weight"].t().contiguous(), nh, dv0, dv) \
            .t().contiguous()
        if params.get("qk_norm"):
            for name in ("q_norm.weight", "k_norm.weight"):
                w = t[name].float() * math.sqrt(d0 / d)
                t[name] = torch.cat([w, w.new_zeros((d - d0,))]).contiguous()
            eps = eps * d0 / d
        return t, eps

    def forward(self, x, step, cache, stream: Optional[torch.Tensor] = None):
        nh, nkv, d = self.num_heads, self.num_kv_heads, self.head_dim
        T = x.shape[0]
        if self.wide:
            return self._forward_wide(x, step, cache, stream)
        qkv = ops.linear(x, self.w_qkv, self.b_qkv, tune=self.runtime.tune)
        slots = step.slot_mapping[cache.group]
        if self.rotation_in_attention and step.n_tokens == step.n_seqs and cache.writes \
                and ops.decode_rope_fusable(qkv, nh, nkv, d, d, False, cache.kv.shape[3], self.scale):
            # single tokens only: the attention kernel prepares queries, key and value itself
            keys, nsplit = plan_split(step.n_seqs, nkv, step.max_keys)
            # few rows in few ranges: the output projection merges the ranges on its way in
            unmerged = stream is not None and self.b_out is None and ops.merged_rows_pay(T, nsplit)
            o = ops.rope_attention_decode(qkv, step.positions, slots, self.q_norm, self.k_norm,
                                          self.position.inv_freq, cache.kv,
                                          step.block_tables[cache.group], nh, self.eps, self.scale,
                                          self.window, keys, nsplit, combine=not unmerged)
            if getattr(step, "taps", None) is not None:
                # (diagnostics want the queries too: from the kernel the attention replaced)
                q = ops.qk_norm_rope_kv_write(qkv, step.positions, None, self.q_norm, self.k_norm,
                                              self.position.inv_freq, None, nh, nkv, d, d, False,
                                              self.eps, write_kv=False)
                merged = o.materialise() if isinstance(o, ops.MergedRows) else o
                self._leave_taps(step, cache, q, merged.view(T, nh, d))
            if not isinstance(o, ops.MergedRows):
                o = o.view(T, nh * d)
            return ops.linear(o, self.w_out, self.b_out, partial_ok=True, accumulate=stream,
                              tune=self.runtime.tune)
        if self.position is None or self.fused_rotation:
            rot = self.position.rotary_dim if self.position is not None else 0
            q = ops.qk_norm_rope_kv_write(
                qkv, step.positions, slots, self.q_norm, self.k_norm,
                self.position.inv_freq if rot else None, cache.kv, nh, nkv, d, rot,
                bool(rot) and self.position.pairing == "adjacent", self.eps,
                write_kv=cache.writes)
        else:
            # Any other encoding: norm with the norm kernel, encode through the part's own
            # ``apply``, then let the fused kernel store what it is given.  q and k are
            # taken out of the projection's rows and put back by a copy kernel.
            qh = ops.copy_columns(qkv, 0, nh * d)
            kh = ops.copy_columns(qkv, nh * d, nkv * d)
            if self.q_norm is not None:
                qh = ops.add_rmsnorm(None, qh.view(T * nh, d), self.q_norm, self.eps, qkv.dtype)
                kh = ops.add_rmsnorm(None, kh.view(T * nkv, d), self.k_norm, self.eps, qkv.dtype)
            qh, kh = self.position.apply(qh.view(T, nh, d), kh.view(T, nkv, d), step.positions)
            if tuple(qh.shape) != (T, nh, d) or tuple(kh.shape) != (T, nkv, d):
                raise ValueError(f"position encoding {self.position.kind!r} returned "
                                 f"{tuple(qh.shape)} and {tuple(kh.shape)}")
            packed = torch.empty_like(qkv)
            ops.copy_columns(qh.reshape(T, nh * d).contiguous(), 0, nh * d, packed, 0)
            ops.copy_columns(kh.reshape(T, nkv * d).contiguous(), 0, nkv * d, packed, nh * d)
            ops.copy_columns(qkv, (nh + nkv) * d, nkv * d, packed, (nh + nkv) * d)
            q = ops.qk_norm_rope_kv_write(packed, step.positions, slots, None, None,
                                          None, cache.kv, nh, nkv, d, 0, False, self.eps,
                                          write_kv=cache.writes)
        mfma = self.mfma and cache.kv.shape[3] % 4 == 0
        if mfma and step.n_tokens > step.n_seqs:
            # prompt portions in the step: both products on the matrix cores
            items = step.attention_items(self.mfma_rows_per_item)
            # a portion far into a long request yields few work items: cut its context
            keys, nsplit = plan_split(items[3], nkv, step.max_keys, target=BUSY_WORKGROUPS)
            # tiles of 128 keys spread a tile's fixed work over twice the scores (measured
            # faster from 512 tokens to 32,768); head size 128 keeps tiles of 64 (LDS)
            o = ops.paged_attention_mfma(q, cache.kv, step.block_tables[cache.group],
                                         step.positions, *items, self.scale, self.window,
                                         keys, nsplit, tile_keys=128 if d == 64 else 64,
                                         shape=self.shape)
        elif mfma:
            # single tokens only: the matrix-core kernel whose waves split the keys
            # (every request brings one token: row i is request i, no work-item arrays)
            item_seq = item_row0 = item_count = None
            n_items = step.n_seqs
            keys, nsplit = plan_split(n_items, nkv, step.max_keys)
            o = ops.paged_attention_decode_mfma(q, cache.kv, step.block_tables[cache.group],
                                                step.positions, item_seq, item_row0, item_count,
                                                n_items, self.scale, self.window, keys, nsplit,
                                                shape=self.shape)
        else:
            item_seq, item_row0, item_count, n_items = step.attention_items(self.rows_per_item)
            keys, nsplit = plan_split(n_items, nkv, step.max_keys)
            o = ops.paged_attention(q, cache.kv, step.block_tables[cache.group], step.positions,
                                    item_seq, item_row0, item_count, n_items, self.scale,
                                    self.window, keys, nsplit, shape=self.shape)
        if getattr(step, "taps", None) is not None:
            self._leave_taps(step, cache, q, o)
        return ops.linear(o.view(T, nh * d), self.w_out, self.b_out, partial_ok=True,
                          accumulate=stream, tune=self.runtime.tune)

    def _forward_wide(self, x, step, cache, stream: Optional[torch.Tensor] = None):
        """Values of their own width and/or a gate per head: the opening projection is
        q | k | v | gate, the cache a plane of keys and a plane of values."""
        nh, nkv, d, dv = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        T = x.shape[0]
        qkv = ops.linear(x, self.w_qkv, self.b_qkv, tune=self.runtime.tune)
        key_plane, value_plane = cache.planes
        rot = self.position.rotary_dim if self.position is not None else 0
        gate = qkv if self.gated else None
        if self.taps:
            # q | k | v through the convolution over time (the gate's columns stay as they
            # are); the request's state slot carries the last inputs from step to step
            qkv = ops.causal_conv(qkv, 0, self.conv_w, None, cache.state, 0, step.token_seq,
                                  step.seq_start, step.slot_id, activation=None,
                                  out_dtype=qkv.dtype)
        q = ops.qk_norm_rope_kv_write_wide(
            qkv, step.positions, step.slot_mapping[cache.group], self.q_norm, self.k_norm,
            self.position.inv_freq if rot else None, key_plane, value_plane, nh, nkv, d, dv, rot,
            bool(rot) and self.position.pairing == "adjacent", self.eps, write_kv=cache.writes)
        table = step.block_tables[cache.group]
        # (ranges are cut at absolute key positions: behind a window nearly all of them
        # would be empty, so a windowed layer's contexts are never cut)
        def split(n_items, **kw):
            # (nor are a chunked layer's, for the same reason)
            return (0, 1) if self.window or self.chunk \
                else plan_split(n_items, nkv, step.max_keys, **kw)
        if self.mfma and cache.kv is not None and cache.kv.shape[3] % 4 == 0:
            if step.n_tokens > step.n_seqs:
                items = step.attention_items(self.mfma_rows_per_item)
                keys, nsplit = split(items[3], target=BUSY_WORKGROUPS)
                o = ops.paged_attention_mfma(q, cache.kv, table, step.positions, *items,
                                             self.scale, self.window, keys, nsplit,
                                             tile_keys=128 if d == 64 else 64, shape=self.shape)
            else:
                keys, nsplit = split(step.n_seqs)
                o = ops.paged_attention_decode_mfma(q, cache.kv, table, step.positions, None,
                                                    None, None, step.n_seqs, self.scale,
                                                    self.window, keys, nsplit, shape=self.shape)
            if gate is not None:
                ops.head_gate_(o, gate, self.gate_col, element=self.gate_element)
        else:
            item_seq, item_row0, item_count, n_items = step.attention_items(self.rows_per_item)
            keys, nsplit = split(n_items)
            o = ops.paged_attention_gated(q, key_plane, value_plane, table, step.positions,
                                          item_seq, item_row0, item_count, n_items, self.scale,
                                          self.window, keys, nsplit, gate, self.gate_col,
                                          shape=self.shape, gate_element=self.gate_element)
        if getattr(step, "taps", None) is not None:
            step.taps["q"] = q.clone()
            step.taps["o"] = o.clone()
        return ops.linear(o.view(T, nh * dv), self.w_out, self.b_out, accumulate=stream,
                          tune=self.runtime.tune)

    def _leave_taps(self, step, cache, q: torch.Tensor, o: torch.Tensor) -> None:
        """Diagnostics: the queries, the keys and values of the step's tokens as they lie in
        the cache now (read back through the tokens' places), and the attention's output."""
        step.taps["q"] = q.clone()
        step.taps["o"] = o.clone()
        if not cache.writes:
            return
        page_size = cache.kv.shape[3]
        place = step.slot_mapping[cache.group].long()
        page, offset = place // page_size, place % page_size
        step.taps["k"] = cache.kv[page, 0, :, offset, :]
        values = cache.kv[:, 1].reshape(cache.kv.shape[0], self.num_kv_heads, self.head_dim, page_size)
        step.taps["v"] = values[page, :, :, offset]


register_mixer(GroupedQueryAttention.kind, GroupedQueryAttention)
