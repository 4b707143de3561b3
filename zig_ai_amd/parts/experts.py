"""A feed-forward of many small experts of which every token uses a few.

``table_experts``: no router.  A table ``[vocab, top]`` of integers names, for each
token id, the ``top`` experts its tokens use (the entries of a row differ); each counts
``1 / top``:

    y[t] = (1 / top) * sum_j  down[e_j] act(up[e_j] x[t]),   e_j = table[token_id[t], j]

``act`` is ``relu2`` (the square of relu); experts have no gate and no biases.  Sizes and
the activation come from ``params``: ``hidden_size``, ``intermediate_size`` (of one expert),
``experts``, ``top``, ``vocab_size``, ``activation``.

The step's tokens are listed per expert on the device (``ops.expert_lists``), two grouped
products run every expert's rows against its own weights in one launch each, and the
second leaves a token's ``top`` results as a stack of 32-bit partial sums that the next
norm adds up: nothing is looked at on the host, so steps can be recorded.
"""

from __future__ import annotations

from typing import Any, Dict, Mapping

import torch

from ..kernels import ops
from .base import FeedForward, Runtime, TensorRule, register_feed_forward


class TableExperts(FeedForward):
    kind = "table_experts"
    graph_safe = True
    kernel_sources = ("experts",)

    @staticmethod
    def _sizes(params):
        return tuple(int(params[k]) for k in ("hidden_size", "intermediate_size", "experts", "top",
                                              "vocab_size"))

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        H, I, E, top, V = cls._sizes(params)
        rules = {"table": TensorRule(((V, top),), role="choice", bound=E)}
        for e in range(E):
            rules[f"experts.{e}.up.weight"] = TensorRule(((I, H),))
            rules[f"experts.{e}.down.weight"] = TensorRule(((H, I),))
        return rules

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        H, I, E, top, V = self._sizes(params)
        if not 0 < top <= E or E > ops.EXPERTS_MAX:
            raise ValueError(f"{top} of {E} experts: top must be within 1..experts, experts at "
                             f"most {ops.EXPERTS_MAX}")
        self.experts, self.top = E, top
        self.activation = str(params.get("activation", "relu2"))
        if self.activation not in ops.EXPERT_ACTIVATIONS:
            raise ValueError(f"expert activation must be relu2, got {self.activation!r}")
        self.table = tensors["table"]
        if self.table.dtype != torch.int32:
            raise ValueError(f"the experts' table must hold integers, got {self.table.dtype}")
        self.up = self._stack([tensors[f"experts.{e}.up.weight"] for e in range(E)])
        self.down = self._stack([tensors[f"experts.{e}.down.weight"] for e in range(E)])

    @staticmethod
    def _stack(mats) -> torch.Tensor:
        w = torch.stack(list(mats), dim=0)
        # (rows of a bfloat16 weight start on 16-byte boundaries, or it is kept in 32-bit)
        if w.dtype == torch.bfloat16 and w.shape[2] % 8:
            w = w.float()
        return w.contiguous()

    def forward(self, x, step):
        T = x.shape[0]
        lists, counts = ops.expert_lists(step.token_ids, self.table, T, self.experts)
        a = ops.grouped_linear(x, self.up, lists, counts, T, per_token=True,
                               activation=self.activation, out_dtype=x.dtype)
        # a stack [top, T, width] of 32-bit partial results, already times 1 / top
        return ops.grouped_linear(a, self.down, lists, counts, T, per_token=False, stacked=True,
                                  out_scale=1.0 / self.top)


register_feed_forward(TableExperts.kind, TableExperts)


class RoutedExperts(FeedForward):
    """Small gated experts of which a router picks ``top`` for every token:

        z = Wr x (+ ``router.bias`` with ``router_bias``: part of the logits, unlike the
        correction);  s = softmax(z) over all router outputs  (``scores="sigmoid"``: sigmoid(z))
        the choice goes by s + correction (``correction``: a tensor, used for the choice
        only), among the outputs of the ``groups_kept`` best of ``groups`` equal groups of
        neighbouring outputs (a group counts by its largest choice score; ``groups = 0``: no
        limit); weight = s * route_scale (``renormalize``: divided by the chosen scores' sum)
        y = sum_chosen weight_e * expert_e(x) + gate * shared(x)

    ``expert_e(x) = Wdown_e (act(Wgate_e x) * (Wup_e x))`` for the ``experts`` outputs that have
    weights; the ``identity_experts`` outputs behind them hand ``x`` on.  ``shared_size > 0``:
    one more expert of that width runs for every token, times ``sigmoid(Wsg x)`` (one number
    a token) when ``shared_gate``.  The router's product and everything after it up to the
    weights is 32-bit; the weighted sum is taken in 32-bit in a fixed order.

    Nothing is looked at on the host: the router's choice becomes per-expert lists on the
    device and two grouped products run every expert's rows in one launch each."""

    kind = "routed_experts"
    graph_safe = True
    kernel_sources = ("experts", "gemm", "gemm_rows64", "activation")

    @staticmethod
    def _sizes(params):
        return (int(params["hidden_size"]), int(params.get("intermediate_size") or 0),
                int(params["experts"]), int(params.get("identity_experts") or 0),
                int(params["top"]), int(params.get("shared_size") or 0))

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        H, I, E, ident, top, S = cls._sizes(params)
        rules = {"router.weight": TensorRule(((E + ident, H),))}
        if params.get("correction"):
            rules["correction"] = TensorRule(((E + ident,),), role="bias")
        if params.get("router_bias"):
            rules["router.bias"] = TensorRule(((E + ident,),), role="bias")
        for e in range(E):
            rules[f"experts.{e}.gate.weight"] = TensorRule(((I, H),))
            rules[f"experts.{e}.up.weight"] = TensorRule(((I, H),))
            rules[f"experts.{e}.down.weight"] = TensorRule(((H, I),))
        if S:
            rules["shared.gate.weight"] = TensorRule(((S, H),))
            rules["shared.up.weight"] = TensorRule(((S, H),))
            rules["shared.down.weight"] = TensorRule(((H, S),))
            if params.get("shared_gate"):
                rules["shared.token_gate.weight"] = TensorRule(((1, H),))
        return rules

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        H, I, E, ident, top, S = self._sizes(params)
        n = E + ident
        if not 0 < top <= n or n > ops.EXPERTS_MAX:
            raise ValueError(f"{top} of {n} router outputs: top must be within 1..outputs, outputs "
                             f"at most {ops.EXPERTS_MAX}")
        self.experts, self.identity, self.top, self.outputs = E, ident, top, n
        self.groups = int(params.get("groups") or 0)
        self.keep = int(params.get("groups_kept") or 0)
        if self.groups and (n % self.groups or not 0 < self.keep <= self.groups
                            or self.keep * (n // self.groups) < top):
            raise ValueError(f"{n} router outputs in {self.groups} groups of which {self.keep} are "
                             f"kept cannot yield {top}")
        self.route_scale = float(params.get("route_scale", 1.0))
        self.scores = str(params.get("scores", "softmax"))
        self.renormalize = bool(params.get("renormalize", False))
        self.activation = str(params.get("activation", "silu"))
        if self.activation not in ops.GATE_ACTIVATIONS:
            raise ValueError(f"expert activation must be one of {sorted(ops.GATE_ACTIVATIONS)}, "
                             f"got {self.activation!r}")
        self.correction = tensors["correction"] if params.get("correction") else None
        # the router's rows and, behind them, the shared expert's gate: one 32-bit product
        rows = [tensors["router.weight"]]
        self.shared_gated = bool(S and params.get("shared_gate"))
        if self.shared_gated:
            rows.append(tensors["shared.token_gate.weight"])
        self.w_router = ops.projection_weight(torch.cat(rows, dim=0).contiguous())
        self.b_router = None
        if params.get("router_bias"):
            b = tensors["router.bias"]
            self.b_router = torch.cat([b, b.new_zeros((self.w_router.shape[0] - b.numel(),))]).contiguous()
        self.gate_up = self.down = None
        if E:
            self.gate_up = TableExperts._stack(
                [torch.cat([tensors[f"experts.{e}.gate.weight"], tensors[f"experts.{e}.up.weight"]],
                           dim=0) for e in range(E)])
            self.down = TableExperts._stack([tensors[f"experts.{e}.down.weight"] for e in range(E)])
        self.shared_gate_up = self.shared_down = None
        if S:
            self.shared_gate_up = ops.projection_weight(
                torch.cat([tensors["shared.gate.weight"], tensors["shared.up.weight"]], dim=0).contiguous())
            self.shared_down = ops.projection_weight(tensors["shared.down.weight"])

    def forward(self, x, step):
        T = x.shape[0]
        tune = self.runtime.tune
        logits = ops.linear(x, self.w_router, self.b_router, out_dtype=torch.float32, tune=tune)
        chosen, weight = ops.route_topk(logits, self.outputs, self.top, self.correction,
                                        self.groups, self.keep, self.route_scale, self.scores,
                                        self.renormalize)
        out = None
        if self.experts:
            # an output beyond the experts that have weights is in nobody's list
            lists, counts = ops.expert_lists(None, chosen, T, self.experts)
            a = ops.grouped_linear(x, self.gate_up, lists, counts, T, per_token=True,
                                   out_dtype=x.dtype)
            a = ops.gated_unit(a, self.activation)
            out = ops.grouped_linear(a, self.down, lists, counts, T, per_token=False,
                                     out_dtype=torch.float32)
        shared = None
        if self.shared_gate_up is not None:
            if x.dtype == torch.bfloat16 and self.shared_gate_up.dtype == torch.bfloat16 \
                    and T <= 16 and x.shape[1] <= 8192:
                # a decode batch: the gate is applied to the projection's accumulators
                s = ops.linear_swiglu(x, self.shared_gate_up, self.activation)
            else:
                s = ops.gated_unit(ops.linear(x, self.shared_gate_up, tune=tune), self.activation)
            shared = ops.linear(s, self.shared_down, out_dtype=torch.float32, tune=tune)
        return ops.experts_combine(out, chosen, weight, x, self.experts, shared,
                                   logits if self.shared_gated else None, self.outputs)


register_feed_forward(RoutedExperts.kind, RoutedExperts)
