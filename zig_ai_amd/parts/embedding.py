"""Token embedding (row gather into the 32-bit residual stream) and the output
head (a projection to 32-bit logits, optionally sharing the embedding table).
/root/reference/src/transformer/embedding.zig:6-41 (which clamps ids; here an
id outside the table is an error raised before the launch) and
/root/reference/src/loader/gguf_model.zig:47-54 (tied fallback).

Two options for designs that need them: ``token_embedding`` with ``norm`` (the rows that
open the stream are RMS-normed, ``x / sqrt(mean(x^2) + norm_eps) * norm.weight``, in 32-bit)
and ``linear_head`` with ``softcap`` (``logits <- softcap * tanh(logits / softcap)``)."""

from __future__ import annotations

from typing import Any, Dict, Mapping

import torch

from ..kernels import ops
from .base import Part, Runtime, TensorRule, register_embedding, register_head


class TokenEmbedding(Part):
    kind = "token_embedding"
    graph_safe = True
    kernel_sources = ("norm",)

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        rules = {"weight": TensorRule(((int(params["vocab_size"]), int(params["hidden_size"])),),
                                      role="table")}
        if params.get("norm"):
            rules["norm.weight"] = TensorRule(((int(params["hidden_size"]),),), role="norm")
        return rules

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        self.weight = tensors["weight"]
        self.vocab_size = int(params["vocab_size"])
        # a norm on the rows that open the stream (None: none)
        self.norm_weight = tensors["norm.weight"] if params.get("norm") else None
        self.norm_eps = float(params.get("norm_eps", 0.0))

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        x = ops.embed_gather(token_ids, self.weight)
        if self.norm_weight is not None:
            x = ops.add_rmsnorm(x, None, self.norm_weight, self.norm_eps, torch.float32,
                                write_residual=False)
        return x


class LinearHead(Part):
    kind = "linear_head"
    graph_safe = True
    takes_stream = True       # ``forward`` accepts a norm that has not run yet
    kernel_sources = ("gemm", "activation")

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        if params.get("tied"):
            return {}
        return {"weight": TensorRule(((int(params["vocab_size"]), int(params["hidden_size"])),),
                                     role="table")}

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        self.tied = bool(params.get("tied"))
        self.weight = tensors.get("weight")   # the model hands a tied head the embedding table
        # a constant factor on the logits (1: none)
        self.logit_scale = float(params.get("logit_scale", 1.0))
        # a cap on the logits, ``cap * tanh(logits / cap)`` (0: none)
        self.softcap = float(params.get("softcap") or 0.0)
        if self.softcap < 0.0:
            raise ValueError(f"the logits' cap must not be negative, got {self.softcap}")

    def forward(self, x) -> torch.Tensor:
        if not self.tied and self.weight.dtype == torch.bfloat16 and self.weight.shape[1] % 8:
            self.weight = ops.projection_weight(self.weight)     # kept in 32-bit from now on
        ops.check_projection_weight(self.weight, "output head")
        logits = ops.linear(x, self.weight, out_dtype=torch.float32, tune=self.runtime.tune)
        if self.logit_scale != 1.0:
            ops.scale_(logits, self.logit_scale)
        if self.softcap:
            ops.softcap_(logits, self.softcap)
        return logits


register_embedding(TokenEmbedding.kind, TokenEmbedding)
register_head(LinearHead.kind, LinearHead)
