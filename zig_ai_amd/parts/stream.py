"""Parts that add to the residual stream between two run-order entries (family
``stream``).  A run-order entry names one with ``LayerCall.before`` and the keywords its
``forward`` takes; the model hands it the stream, what is still pending for it, and the
embedding's output as it was before the first layer (``origin``).

``pass_offset``: for models that run a span of layers several times with the same weights.
Before pass ``row`` of the span the stream takes the row ``row`` of a table ``[passes,
width]`` and, with ``add_origin``, the embedding's output once more:

    x <- x (+ pending) (+ origin) + table[row]

``pass_mix``: for the same kind of model, where each pass of the span starts from a
projection of the stream and the embedding's output side by side:

    x <- W [x (+ pending); origin]          W: [width, 2 width], the stream's half first
"""

from __future__ import annotations

from typing import Any, Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import Part, Runtime, TensorRule, register_stream_step


class PassOffset(Part):
    kind = "pass_offset"
    graph_safe = True
    kernel_sources = ("norm",)

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        return {"table": TensorRule(((int(params["passes"]), int(params["width"])),), role="bias")}

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        self.passes = int(params["passes"])
        self.table = tensors["table"]          # 32-bit [passes, width]

    def forward(self, residual: torch.Tensor, pending: Optional[torch.Tensor],
                origin: Optional[torch.Tensor], step, row: int = 0, add_origin: bool = False):
        if not 0 <= int(row) < self.passes:
            raise ValueError(f"pass {row} of {self.passes}")
        if add_origin and origin is None:
            raise ValueError("the embedding's output was not kept for this model")
        ops.stream_add_(residual, pending, origin if add_origin else None, self.table[int(row)])
        return residual, None


register_stream_step(PassOffset.kind, PassOffset)


class PassMix(Part):
    kind = "pass_mix"
    graph_safe = True
    kernel_sources = ("norm", "gemm", "gemm_rows64", "activation")

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        width = int(params["width"])
        return {"weight": TensorRule(((width, 2 * width),))}

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        self.width = int(params["width"])
        self.weight = ops.projection_weight(tensors["weight"])
        ops.check_projection_weight(self.weight, "pass_mix weight")

    def forward(self, residual: torch.Tensor, pending: Optional[torch.Tensor],
                origin: Optional[torch.Tensor], step):
        if origin is None:
            raise ValueError("the embedding's output was not kept for this model")
        if pending is not None:
            ops.stream_add_(residual, pending)
        T, W = residual.shape
        both = torch.empty((T, 2 * W), dtype=self.runtime.dtype, device=residual.device)
        ops.copy_columns(residual, 0, W, both, 0)
        ops.copy_columns(origin, 0, W, both, W)
        # (a new stream: the product's 32-bit sums)
        return ops.linear(both, self.weight, out_dtype=torch.float32, tune=self.runtime.tune), None


register_stream_step(PassMix.kind, PassMix)


class TokenSide(Part):
    """What a layer takes from the tokens themselves, past its mixer and feed-forward
    (``token_side``).  A second embedding table ``[vocab, layers * dim]`` holds ``dim`` numbers
    for every layer and token id; for layer ``i``

        e = table[token, i * dim : (i + 1) * dim]
        g = act(Wgate_i x) * e                 x: the stream itself, not normed
        y = Wproj_i g
        x <- x (+ pending) + scale * y / sqrt(mean(y^2) + eps) * norm_i

    ``layers``, ``dim``, ``width``, ``vocab_size``, ``eps``, ``scale`` and ``activation`` are
    parameters; a run-order entry names the layer with ``args = {"layer": i}``."""

    kind = "token_side"
    graph_safe = True
    needs_origin = False
    kernel_sources = ("norm", "gemm", "gemm_rows64", "activation")

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        L, dim, width = int(params["layers"]), int(params["dim"]), int(params["width"])
        rules = {"table": TensorRule(((int(params["vocab_size"]), L * dim),), role="table")}
        for i in range(L):
            rules[f"layers.{i}.gate.weight"] = TensorRule(((dim, width),))
            rules[f"layers.{i}.proj.weight"] = TensorRule(((width, dim),))
            rules[f"layers.{i}.norm.weight"] = TensorRule(((width,),), role="norm")
        return rules

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        self.layers, self.dim = int(params["layers"]), int(params["dim"])
        self.eps = float(params["eps"])
        self.scale = float(params.get("scale", 1.0))
        self.activation = str(params.get("activation", "gelu_tanh"))
        if self.activation not in ops.GATE_ACTIVATIONS:
            raise ValueError(f"activation must be one of {sorted(ops.GATE_ACTIVATIONS)}, got "
                             f"{self.activation!r}")
        self.table = tensors["table"]
        self.gate = [ops.projection_weight(tensors[f"layers.{i}.gate.weight"])
                     for i in range(self.layers)]
        self.proj = [ops.projection_weight(tensors[f"layers.{i}.proj.weight"])
                     for i in range(self.layers)]
        self.norm = [tensors[f"layers.{i}.norm.weight"] for i in range(self.layers)]

    def forward(self, residual: torch.Tensor, pending: Optional[torch.Tensor],
                origin: Optional[torch.Tensor], step, layer: int = 0):
        i = int(layer)
        if not 0 <= i < self.layers:
            raise ValueError(f"layer {layer} of {self.layers}")
        if pending is not None:
            ops.stream_add_(residual, pending)
        x = ops.cast(residual, self.runtime.dtype)
        g = ops.table_gate(ops.linear(x, self.gate[i], tune=self.runtime.tune), step.token_ids,
                           self.table, i * self.dim, self.activation)
        y = ops.linear(g, self.proj[i], out_dtype=torch.float32, tune=self.runtime.tune)
        ops.normed_add_(residual, y, self.norm[i], self.eps, self.scale)
        return residual, None


register_stream_step(TokenSide.kind, TokenSide)
