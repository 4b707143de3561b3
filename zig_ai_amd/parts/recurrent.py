"""Mixers that carry a matrix state per request instead of keys and values.

``ssd`` (state-space duality, the Mamba-2 mixer).  With ``inner = heads * head_dim``,
``N = state_size`` and ``G = groups``, one projection yields
``[z: inner | x: inner | B: G*N | C: G*N | dt: heads]``; x, B and C pass a causal
depth-wise convolution (with bias) and silu; per head ``h`` (group ``h // (heads/G)``)

    dt = softplus(dt + dt_bias);   S <- exp(-exp(A_log) dt) S + dt B x^T;   y = S^T C + D x

then ``y * silu(z)``, an RMS norm over ``norm_groups`` equal parts times ``norm``, and the
output projection.

``gated_delta`` (the gated delta rule with one decay per key channel).  Projections
q, k (``num_kv_heads x head_dim``) and v (``num_heads x value_dim``) each pass a causal
depth-wise convolution (no bias) and silu; q and k become unit vectors (q also times
``head_dim^-1/2``); ``beta = sigmoid(W_b h)`` per head; the decay is
``g = exp(-exp(A_log) softplus(W_a2 W_a1 h + dt_bias))`` per head and key channel; per head

    S <- diag(g) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q

then ``o`` over its root mean square per head, times ``norm`` (one weight per value
channel, shared by the heads), times ``sigmoid(W_g2 W_g1 h)``, and the output projection.

Both keep, per request, the state matrix in 32-bit and the convolution's last
``kernel_size - 1`` inputs, in one state slot: ``[conv inputs | S]``.

``retention`` (linear attention with one fixed decay a head, no softmax and no
denominator).  Projections q, k (``num_heads x head_dim``), v and a gate g (``num_heads x
value_dim``), no biases, no convolution; the position encoding (``position``, a nested
rotary spec or None) turns the leading elements of every q and k, the keys are then
multiplied by ``head_dim^-1/2``; per head ``h``

    S <- decay[h] S + k v^T;   o = S^T q

then each head's ``o`` over its root mean square (``norm_eps``, no weight), times
``silu(g)``, and the output projection.  ``decay`` is a tuple of constants, one a head.
The state slot holds ``S`` in 32-bit; what enters the walk (rotated q and k, v) is 32-bit.
Four parameters turn it into other linear attentions of the same walk: ``activation``
(``"silu"``: q, k and v pass silu right behind their projection; None), ``key_scale`` (what the
keys are multiplied by; ``head_dim^-1/2`` unless given), ``output_norm`` (``"head"``: every
head's read-out over its own root mean square, no weight; ``"all"``: the heads' read-outs
side by side are normed together, times a weight ``norm.weight`` of ``num_heads * value_dim``)
and ``gate`` (``"silu"`` or ``"sigmoid"`` of the gate's projection, applied behind the norm).
Lightning attention is ``activation="silu"``, ``key_scale=1``, ``output_norm="all"``,
``gate="sigmoid"`` and no position encoding.
A step in which some request brings more than ``ops.RETENTION_CHUNK`` tokens walks its
portions as chunks side by side (``ops.fixed_decay_recurrence_chunked``): with a constant
decay the state is linear in what the tokens bring.
"""

from __future__ import annotations

from typing import Any, Dict, Mapping

import torch

from ..kernels import ops
from .base import Mixer, Runtime, StateNeed, TensorRule, lookup, register_mixer
from .feed_forward import fuse_rows, pad_columns, pad_rows


class StateSpaceDuality(Mixer):
    kind = "ssd"
    graph_safe = True
    takes_normed_rows = True      # ``x`` is only ever handed to ``ops.linear``
    kernel_sources = ("gemm", "recurrent")

    @staticmethod
    def _sizes(params):
        W, H, P, N, G, L = (int(params[k]) for k in
                            ("hidden_size", "num_heads", "head_dim", "state_size", "groups",
                             "kernel_size"))
        return W, H, P, N, G, L

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        W, H, P, N, G, L = cls._sizes(params)
        inner, C = H * P, H * P + 2 * G * N
        return {"in_proj.weight": TensorRule(((2 * inner + 2 * G * N + H, W),)),
                "conv.weight": TensorRule(((C, L),), role="filter"),
                "conv.bias": TensorRule(((C,),), role="bias"),
                "dt_bias": TensorRule(((H,),), role="bias"),
                "A_log": TensorRule(((H,),), role="bias"),
                "D": TensorRule(((H,),), role="bias"),
                "norm.weight": TensorRule(((inner,),), role="norm"),
                "out_proj.weight": TensorRule(((W, inner),))}

    @classmethod
    def cache_need(cls, params: Mapping[str, Any]):
        W, H, P, N, G, L = cls._sizes(params)
        return StateNeed(((H * P + 2 * G * N) * (L - 1) + H * N * P,))

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        W, H, P, N, G, L = self._sizes(params)
        if H % G:
            raise ValueError(f"{H} heads do not divide into {G} groups")
        self.norm_groups = int(params.get("norm_groups", 1))
        if (H * P) % self.norm_groups:
            raise ValueError(f"{H * P} channels do not divide into {self.norm_groups} norm groups")
        if L > ops.CONV_MAX_TAPS:
            raise ValueError(f"conv kernel_size {L} exceeds the kernel's limit of {ops.CONV_MAX_TAPS}")
        ops.recurrence_plan(N, P)
        self.heads, self.head_dim, self.state_size, self.groups, self.taps = H, P, N, G, L
        self.inner = H * P
        self.eps = float(params["norm_eps"])
        self.w_in = ops.projection_weight(pad_rows(tensors["in_proj.weight"]))
        self.w_out = ops.projection_weight(tensors["out_proj.weight"])
        self.conv_w = tensors["conv.weight"]
        self.conv_b = tensors["conv.bias"]
        self.dt_bias, self.A_log, self.D = tensors["dt_bias"], tensors["A_log"], tensors["D"]
        self.norm_w = tensors["norm.weight"]
        self.conv_state = (self.inner + 2 * G * N) * (L - 1)      # floats before S in a slot
        ops.check_projection_weight(self.w_in, "ssd in_proj")
        ops.check_projection_weight(self.w_out, "ssd out_proj")

    def forward(self, x, step, cache):
        inner, G, N = self.inner, self.groups, self.state_size
        z = ops.linear(x, self.w_in, tune=self.runtime.tune)
        conv = ops.causal_conv_silu(z, inner, self.conv_w, self.conv_b, cache.state, 0,
                                    step.token_seq, step.seq_start, step.slot_id)
        y = ops.matrix_recurrence("ssd", conv, inner + G * N, inner, 0, z, 2 * inner + 2 * G * N,
                                  None, self.dt_bias, self.A_log, self.D, cache.state,
                                  self.conv_state, step.seq_start, step.slot_id, self.heads, G, N,
                                  self.head_dim)
        h = ops.gated_group_norm(y, z, 0, self.norm_w, inner // self.norm_groups, self.eps,
                                 "silu", gate_first=True)
        return ops.linear(h, self.w_out, tune=self.runtime.tune)


class GatedDeltaRule(Mixer):
    kind = "gated_delta"
    graph_safe = True
    takes_normed_rows = True      # ``x`` is only ever handed to ``ops.linear``
    kernel_sources = ("gemm", "recurrent", "activation")

    @staticmethod
    def _sizes(params):
        return tuple(int(params[k]) for k in
                     ("hidden_size", "num_heads", "num_kv_heads", "head_dim", "value_dim",
                      "kernel_size", "decay_rank", "gate_rank"))

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        W, H, G, d, dv, L, ra, rg = cls._sizes(params)
        return {"q_proj.weight": TensorRule(((G * d, W),)),
                "k_proj.weight": TensorRule(((G * d, W),)),
                "v_proj.weight": TensorRule(((H * dv, W),)),
                "q_conv.weight": TensorRule(((G * d, L),), role="filter"),
                "k_conv.weight": TensorRule(((G * d, L),), role="filter"),
                "v_conv.weight": TensorRule(((H * dv, L),), role="filter"),
                "beta_proj.weight": TensorRule(((H, W),)),
                "A_log": TensorRule(((H,),), role="bias"),
                "dt_bias": TensorRule(((H * d,),), role="bias"),
                "decay_down.weight": TensorRule(((ra, W),)),
                "decay_up.weight": TensorRule(((H * d, ra),)),
                "gate_down.weight": TensorRule(((rg, W),)),
                "gate_up.weight": TensorRule(((H * dv, rg),)),
                "norm.weight": TensorRule(((dv,),), role="norm"),
                "out_proj.weight": TensorRule(((W, H * dv),))}

    @classmethod
    def cache_need(cls, params: Mapping[str, Any]):
        W, H, G, d, dv, L, ra, rg = cls._sizes(params)
        return StateNeed(((2 * G * d + H * dv) * (L - 1) + H * d * dv,))

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        W, H, G, d, dv, L, ra, rg = self._sizes(params)
        if H % G:
            raise ValueError(f"{H} heads do not divide into {G} query/key heads")
        if L > ops.CONV_MAX_TAPS:
            raise ValueError(f"conv kernel_size {L} exceeds the kernel's limit of {ops.CONV_MAX_TAPS}")
        ops.recurrence_plan(d, dv)
        self.heads, self.kv_heads, self.head_dim, self.value_dim, self.taps = H, G, d, dv, L
        self.eps = float(params["norm_eps"])
        # one opening product: q | k | v | beta | decay_down | gate_down; each low-rank
        # block is filled up with zero rows to a multiple of 8, the input width that the
        # second product wants
        down_a, down_g = pad_rows(tensors["decay_down.weight"]), pad_rows(tensors["gate_down.weight"])
        self.w_in = pad_rows(fuse_rows(tensors["q_proj.weight"], tensors["k_proj.weight"],
                                       tensors["v_proj.weight"], tensors["beta_proj.weight"],
                                       down_a, down_g))
        self.beta_col = 2 * G * d + H * dv
        self.low_col = self.beta_col + H
        self.low_width = down_a.shape[0] + down_g.shape[0]
        # the second product: [decay_up 0; 0 gate_up] on the low-rank columns
        up_a, up_g = pad_columns(tensors["decay_up.weight"]), pad_columns(tensors["gate_up.weight"])
        top = torch.cat([up_a, up_a.new_zeros((up_a.shape[0], up_g.shape[1]))], dim=1)
        bottom = torch.cat([up_g.new_zeros((up_g.shape[0], up_a.shape[1])), up_g], dim=1)
        self.w_up = pad_rows(torch.cat([top, bottom], dim=0))
        self.w_in = ops.projection_weight(self.w_in)
        self.conv_w = torch.cat([tensors["q_conv.weight"], tensors["k_conv.weight"],
                                 tensors["v_conv.weight"]], dim=0).contiguous()
        self.A_log, self.dt_bias = tensors["A_log"], tensors["dt_bias"]
        self.norm_w = tensors["norm.weight"]
        self.w_out = ops.projection_weight(tensors["out_proj.weight"])
        self.conv_state = (2 * G * d + H * dv) * (L - 1)
        for w, what in ((self.w_in, "in"), (self.w_up, "low-rank up"), (self.w_out, "out")):
            ops.check_projection_weight(w, f"gated_delta {what} projection")

    def forward(self, x, step, cache):
        H, G, d, dv = self.heads, self.kv_heads, self.head_dim, self.value_dim
        z = ops.linear(x, self.w_in, tune=self.runtime.tune)
        conv = ops.causal_conv_silu(z, 0, self.conv_w, None, cache.state, 0, step.token_seq,
                                    step.seq_start, step.slot_id)
        low = ops.copy_columns(z, self.low_col, self.low_width)
        up = ops.linear(low, self.w_up, tune=self.runtime.tune)      # decay: H*d | gate: H*dv
        o = ops.matrix_recurrence("delta", conv, 0, G * d, 2 * G * d, z, self.beta_col, up,
                                  self.dt_bias, self.A_log, None, cache.state, self.conv_state,
                                  step.seq_start, step.slot_id, H, G, d, dv)
        h = ops.gated_group_norm(o, up, H * d, self.norm_w, dv, self.eps, "sigmoid",
                                 gate_first=False)
        return ops.linear(h, self.w_out, tune=self.runtime.tune)


class Retention(Mixer):
    kind = "retention"
    graph_safe = True
    takes_normed_rows = True      # ``x`` is only ever handed to ``ops.linear``
    accepts_stream = True         # ``forward`` takes ``stream`` and may add its result there
    kernel_sources = ("gemm", "recurrent")

    @staticmethod
    def _sizes(params):
        return tuple(int(params[k]) for k in ("hidden_size", "num_heads", "head_dim", "value_dim"))

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        W, H, d, dv = cls._sizes(params)
        rules = {"q_proj.weight": TensorRule(((H * d, W),)),
                 "k_proj.weight": TensorRule(((H * d, W),)),
                 "v_proj.weight": TensorRule(((H * dv, W),)),
                 "gate_proj.weight": TensorRule(((H * dv, W),)),
                 "out_proj.weight": TensorRule(((W, H * dv),))}
        if params.get("output_norm", "head") == "all":
            rules["norm.weight"] = TensorRule(((H * dv,),), role="norm")
        return rules

    @classmethod
    def cache_need(cls, params: Mapping[str, Any]):
        W, H, d, dv = cls._sizes(params)
        return StateNeed((H * d * dv,))

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        W, H, d, dv = self._sizes(params)
        decay = [float(x) for x in params["decay"]]
        if len(decay) != H:
            raise ValueError(f"{len(decay)} decays for {H} heads")
        ops.recurrence_plan(d, dv)
        self.heads, self.head_dim, self.value_dim = H, d, dv
        self.eps = float(params["norm_eps"])
        self.decay = torch.tensor(decay, dtype=torch.float32, device=runtime.device)
        scale = params.get("key_scale")
        self.k_scale = float(d) ** -0.5 if scale is None else float(scale)
        self.activation = params.get("activation")
        self.output_norm = str(params.get("output_norm", "head"))
        self.gate = str(params.get("gate", "silu"))
        if self.activation not in (None, "silu") or self.output_norm not in ("head", "all") \
                or self.gate not in ("silu", "sigmoid"):
            raise ValueError(f"retention: activation {self.activation!r}, output_norm "
                             f"{self.output_norm!r}, gate {self.gate!r}")
        pos = params.get("position")
        self.position = lookup("position", pos.kind)(pos.params, {}, runtime) if pos is not None \
            else None
        if self.position is not None and not (getattr(self.position, "fused_rotation", False)
                                               and self.position.pairing == "half"):
            raise ValueError("retention takes a rotary position encoding in halves, or none")
        self.rotary_dim = self.position.rotary_dim if self.position is not None else 0
        # one opening product: q | k | v | g
        self.w_in = ops.projection_weight(pad_rows(fuse_rows(
            tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"],
            tensors["gate_proj.weight"])))
        self.w_out = ops.projection_weight(tensors["out_proj.weight"])
        self.gate_col = 2 * H * d + H * dv
        if self.output_norm == "all":
            self.norm_w, self.norm_group = tensors["norm.weight"], H * dv
        else:
            self.norm_w = torch.ones((1,), dtype=torch.float32, device=runtime.device)
            self.norm_group = dv
        # long portions are walked in chunks side by side (the step's work items of that size)
        self.chunked = d <= ops.RETENTION_CHUNK_MAX_DK
        self.item_granularities = [ops.RETENTION_CHUNK] if self.chunked else []
        ops.check_projection_weight(self.w_in, "retention opening projection")
        ops.check_projection_weight(self.w_out, "retention out_proj")

    def forward(self, x, step, cache, stream=None):
        H, d, dv = self.heads, self.head_dim, self.value_dim
        z = ops.linear(x, self.w_in, tune=self.runtime.tune)
        vectors = ops.retention_prepare(
            z, 0, H * d, 2 * H * d, step.positions,
            self.position.inv_freq if self.rotary_dim else None, H, d, dv, self.rotary_dim,
            self.k_scale, self.activation)
        items = step.attention_items(ops.RETENTION_CHUNK) if self.chunked else None
        if items is not None and items[3] > step.n_seqs:
            # some request brings more than a chunk: chunks side by side (a function of the
            # step's shape alone)
            o = ops.fixed_decay_recurrence_chunked(vectors, 0, H * d, 2 * H * d, self.decay,
                                                   cache.state, 0, step.slot_id, items, H, d, dv)
        else:
            o = ops.matrix_recurrence("fixed", vectors, 0, H * d, 2 * H * d, None, 0, self.decay,
                                      None, None, None, cache.state, 0, step.seq_start,
                                      step.slot_id, H, H, d, dv)
        if getattr(step, "taps", None) is not None:
            step.taps["vectors"] = vectors.clone()
            step.taps["o"] = o.clone()
        h = ops.gated_group_norm(o, z, self.gate_col, self.norm_w, self.norm_group, self.eps,
                                 self.gate, gate_first=False)
        return ops.linear(h, self.w_out, accumulate=stream, tune=self.runtime.tune)


register_mixer(StateSpaceDuality.kind, StateSpaceDuality)
register_mixer(Retention.kind, Retention)
register_mixer(GatedDeltaRule.kind, GatedDeltaRule)
