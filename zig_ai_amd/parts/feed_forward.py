"""Dense SwiGLU feed-forward: ``(silu(x Wg^T) * (x Wu^T)) Wd^T`` without biases
(/root/reference/src/transformer/ffn.zig:19-33).  Gate and up weights are fused
into one ``[2I, H]`` matrix at load so the input is read once.  The result may be
a stack of partial sums (see ``Norm.add_forward``)."""

from __future__ import annotations

from typing import Any, Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import FeedForward, Runtime, TensorRule, register_feed_forward


def fuse_rows(*mats: torch.Tensor) -> torch.Tensor:
    """Stack weight matrices along the output dimension; mixed precisions are
    widened to 32-bit rather than narrowed."""
    if len({m.dtype for m in mats}) > 1:
        mats = tuple(m.float() for m in mats)
    return torch.cat(mats, dim=0).contiguous()


def pad_rows(w: torch.Tensor, multiple: int = 8) -> torch.Tensor:
    """``w [N, K]`` with zero rows appended up to a multiple: a fused projection's output
    rows then start on 16-byte boundaries in either storage type."""
    extra = -w.shape[0] % multiple
    if not extra:
        return w
    return torch.cat([w, w.new_zeros((extra,) + tuple(w.shape[1:]))], dim=0).contiguous()


def pad_columns(w: torch.Tensor, multiple: int = 8) -> torch.Tensor:
    """``w [N, K]`` with zero columns appended up to a multiple (a product's input width
    has to be one; the inputs that meet the new columns must be zero as well)."""
    extra = -w.shape[1] % multiple
    if not extra:
        return w
    return torch.cat([w, w.new_zeros((w.shape[0], extra))], dim=1).contiguous()


class SwiGLU(FeedForward):
    kind = "swiglu"
    graph_safe = True
    takes_stream = True
    opens_with_swiglu = True
    kernel_sources = ("gemm", "gemm_rows64", "activation")

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        H, I = int(params["hidden_size"]), int(params["intermediate_size"])
        return {"gate.weight": TensorRule(((I, H),)), "up.weight": TensorRule(((I, H),)),
                "down.weight": TensorRule(((H, I),))}

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        self.gate_up = fuse_rows(tensors["gate.weight"], tensors["up.weight"])
        self.down = tensors["down.weight"]
        # the gate's activation: ``silu`` (SwiGLU) or ``gelu_tanh`` (the tanh form of gelu);
        # of the products that apply the gate to their own sums the one for decode batches
        # knows both, the one that also runs the norm of a larger step silu only
        self.activation = str(params.get("activation", "silu"))
        if self.activation not in ops.GATE_ACTIVATIONS:
            raise ValueError(f"feed-forward activation must be one of "
                             f"{sorted(ops.GATE_ACTIVATIONS)}, got {self.activation!r}")
        if self.activation != "silu":
            self.opens_with_swiglu = False
            self.gate_up = ops.projection_weight(self.gate_up)
            self.down = ops.projection_weight(self.down)
        ops.check_projection_weight(self.gate_up, "feed_forward gate_up")
        ops.check_projection_weight(self.down, "feed_forward down")

    def forward(self, x, step=None, stream: Optional[torch.Tensor] = None):
        if self.activation != "silu":
            if isinstance(x, ops.NormedRows):
                x = x.materialise()
            if x.dtype == torch.bfloat16 and self.gate_up.dtype == torch.bfloat16 \
                    and x.shape[0] <= 16 and x.shape[1] <= 8192:
                # a decode batch: the gate is applied to the projection's accumulators
                a = ops.linear_swiglu(x, self.gate_up, self.activation)
            else:
                a = ops.gated_unit(ops.linear(x, self.gate_up, tune=self.runtime.tune),
                                   self.activation)
            return ops.linear(a, self.down, partial_ok=True, accumulate=stream,
                              tune=self.runtime.tune)
        bf16 = x.dtype == torch.bfloat16 and self.gate_up.dtype == torch.bfloat16
        if bf16 and x.shape[0] <= 16 and x.shape[1] <= 8192:
            # a decode batch: the gate is applied to the projection's accumulators
            a = ops.linear_swiglu(x, self.gate_up)
        elif bf16 and isinstance(x, ops.NormedRows) and ops.rows64_swiglu_fusable(*x.shape):
            # a step beyond 16 rows whose norm has not run: norm, product and gate in one kernel
            a = ops.linear_swiglu(x, self.gate_up)
        else:
            if isinstance(x, ops.NormedRows):
                x = x.materialise()
            a = ops.swiglu(ops.linear(x, self.gate_up, tune=self.runtime.tune))
        return ops.linear(a, self.down, partial_ok=True, accumulate=stream, tune=self.runtime.tune)


class ClampedGLU(FeedForward):
    """A gated unit whose two inputs are bounded before they meet:

        g = min(x Wg^T, limit);  u = clamp(x Wu^T, -limit, limit)
        y = (g * sigmoid(alpha * g) * (u + up_offset)) Wd^T

    ``limit`` (none if 0), ``alpha`` and ``up_offset`` come from ``params``.  Gate and up
    weights are one matrix, as in ``SwiGLU``; the activation is a kernel of its own."""

    kind = "clamped_glu"
    graph_safe = True
    kernel_sources = ("gemm", "activation")

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        H, I = int(params["hidden_size"]), int(params["intermediate_size"])
        return {"gate.weight": TensorRule(((I, H),)), "up.weight": TensorRule(((I, H),)),
                "down.weight": TensorRule(((H, I),))}

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        self.limit = float(params.get("limit") or 0.0)
        self.alpha = float(params.get("alpha", 1.0))
        self.up_offset = float(params.get("up_offset", 0.0))
        self.gate_up = ops.projection_weight(fuse_rows(tensors["gate.weight"], tensors["up.weight"]))
        self.down = ops.projection_weight(tensors["down.weight"])

    def forward(self, x, step=None):
        a = ops.clamped_glu(ops.linear(x, self.gate_up, tune=self.runtime.tune), self.limit,
                            self.alpha, self.up_offset)
        return ops.linear(a, self.down, tune=self.runtime.tune)


class ActivatedMLP(FeedForward):
    """A feed-forward without a gate: ``Wd act(Wu x)``, no biases.  ``activation``: ``relu2``,
    the square of relu, taken in 32-bit by a kernel of its own."""

    kind = "activated_mlp"
    graph_safe = True
    accepts_stream = True     # ``forward`` takes ``stream`` and may add its result there
    kernel_sources = ("gemm", "gemm_rows64", "activation")

    @classmethod
    def tensor_rules(cls, params: Mapping[str, Any]) -> Dict[str, TensorRule]:
        H, I = int(params["hidden_size"]), int(params["intermediate_size"])
        return {"up.weight": TensorRule(((I, H),)), "down.weight": TensorRule(((H, I),))}

    def __init__(self, params, tensors, runtime: Runtime):
        super().__init__(params, tensors, runtime)
        self.activation = str(params.get("activation", "relu2"))
        if self.activation not in ops.UNARY_ACTIVATIONS:
            raise ValueError(f"feed-forward activation must be one of "
                             f"{sorted(ops.UNARY_ACTIVATIONS)}, got {self.activation!r}")
        self.up = ops.projection_weight(pad_rows(tensors["up.weight"]))
        self.down = ops.projection_weight(pad_columns(tensors["down.weight"]))
        ops.check_projection_weight(self.up, "feed_forward up")
        ops.check_projection_weight(self.down, "feed_forward down")

    def forward(self, x, step=None, stream: Optional[torch.Tensor] = None):
        a = ops.activate(ops.linear(x, self.up, tune=self.runtime.tune), self.activation)
        return ops.linear(a, self.down, out_dtype=torch.float32, accumulate=stream,
                          tune=self.runtime.tune)


register_feed_forward(SwiGLU.kind, SwiGLU)
register_feed_forward(ClampedGLU.kind, ClampedGLU)
register_feed_forward(ActivatedMLP.kind, ActivatedMLP)
