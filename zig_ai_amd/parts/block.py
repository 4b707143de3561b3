"""Arrangements: how a block's parts are wired.  An arrangement declares its parts
(``slots``: name -> family; the model builds each from the layer's ``PartSpec`` of that
name and hands them over as a dictionary) and runs them in ``forward``.

``pre_norm_residual`` is the reference's decoder block
(/root/reference/src/transformer/hybrid_layer.zig:366-492):

    h = x + mixer(norm1(x));   y = h + feed_forward(norm2(h))

The residual stream is kept in 32-bit.  A block receives the stream and a
``pending`` tensor that has not been added to it yet, and returns the same
pair: every add is then fused with the norm that follows it, including across
the boundary between two blocks.  Where a part says so (``takes_stream``) the norm
before it is handed over without having run (``Norm.deferred``) and the part may add
its result to the stream itself; nothing is pending after it then.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from .base import register_arrangement


class PreNormResidualBlock:
    kind = "pre_norm_residual"
    slots = {"mixer_norm": "norm", "mixer": "mixer", "feed_forward_norm": "norm",
             "feed_forward": "feed_forward"}

    def __init__(self, parts):
        self.parts = dict(parts)
        self.mixer_norm = parts["mixer_norm"]
        self.mixer = parts["mixer"]
        self.feed_forward_norm = parts["feed_forward_norm"]
        self.feed_forward = parts["feed_forward"]

    def forward(self, residual: torch.Tensor, pending: Optional[torch.Tensor], step,
                cache) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        m = apply_normed(self.mixer_norm, self.mixer, residual, pending, step, cache)
        f = apply_normed(self.feed_forward_norm, self.feed_forward, residual, m, step)
        return residual, f


def apply_normed(norm, part, residual: torch.Tensor, pending: Optional[torch.Tensor], *args):
    """``part(norm(residual + pending))``: what is still to be added to the stream
    afterwards, or ``None`` when the part has added it already."""
    if not getattr(part, "takes_stream", False):
        return part.forward(norm.add_forward(residual, pending), *args)
    x = None
    if pending is None:
        x = norm.deferred(residual, swiglu=True) if getattr(part, "opens_with_swiglu", False) \
            else norm.deferred(residual)
    if x is None:
        x = norm.add_forward(residual, pending)
    runtime = getattr(part, "runtime", None)
    adds = runtime is None or getattr(runtime, "stream_additions", True)
    return part.forward(x, *args, stream=residual if adds else None)


register_arrangement(PreNormResidualBlock.kind, PreNormResidualBlock)


class PreNormMixerBlock:
    """The pre-norm block of a layer that has no feed-forward: ``y = x + mixer(norm1(x))``."""

    kind = "pre_norm_residual_no_ff"
    slots = {"mixer_norm": "norm", "mixer": "mixer"}

    def __init__(self, parts):
        self.parts = dict(parts)
        self.mixer_norm = parts["mixer_norm"]
        self.mixer = parts["mixer"]

    def forward(self, residual: torch.Tensor, pending: Optional[torch.Tensor], step,
                cache) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        return residual, apply_normed(self.mixer_norm, self.mixer, residual, pending, step, cache)


register_arrangement(PreNormMixerBlock.kind, PreNormMixerBlock)


class ParallelResidualBlock:
    """One norm, and mixer and feed-forward side by side on its output:

        h = norm(x);   y = x + (mixer(h) + feed_forward(h))

    The norm runs as a kernel of its own, so both parts read a tensor that nothing adds to.
    A part that sets ``takes_stream`` or ``accepts_stream`` is handed the stream as the keyword
    ``stream`` and may add its result there itself (it then returns ``None``); what a part
    returns instead is added here (the mixer's) or left pending for the norm that follows,
    which adds it while it reads the stream (the feed-forward's)."""

    kind = "parallel_residual"
    slots = {"norm": "norm", "mixer": "mixer", "feed_forward": "feed_forward"}

    def __init__(self, parts):
        self.parts = dict(parts)
        self.norm = parts["norm"]
        self.mixer = parts["mixer"]
        self.feed_forward = parts.get("feed_forward")

    def forward(self, residual: torch.Tensor, pending: Optional[torch.Tensor], step,
                cache) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        from ..kernels import ops
        h = self.norm.add_forward(residual, pending)

        def adds(part):
            runtime = getattr(part, "runtime", None)
            return (getattr(part, "takes_stream", False) or getattr(part, "accepts_stream", False)) \
                and (runtime is None or getattr(runtime, "stream_additions", True))

        m = self.mixer.forward(h, step, cache, stream=residual) if adds(self.mixer) \
            else self.mixer.forward(h, step, cache)
        f = None
        if self.feed_forward is not None:
            f = self.feed_forward.forward(h, step, stream=residual) if adds(self.feed_forward) \
                else self.feed_forward.forward(h, step)
        if m is not None:
            ops.stream_add_(residual, m)
        return residual, f


class ParallelMixerBlock(ParallelResidualBlock):
    """The same for a layer that has no feed-forward: ``y = x + mixer(norm(x))``."""

    kind = "parallel_residual_no_ff"
    slots = {"norm": "norm", "mixer": "mixer"}


register_arrangement(ParallelResidualBlock.kind, ParallelResidualBlock)
register_arrangement(ParallelMixerBlock.kind, ParallelMixerBlock)


class ScaledResidualBlock:
    """A pre-norm block whose parts enter the stream with weights, and which may run two
    mixers side by side on the same normed input and may lack the feed-forward:

        h = x + m * (a * left(norm1(x)) + b * right(norm1(x)));   y = h + m * ff(norm2(h))

    ``m`` (``residual_scale``), ``a`` and ``b`` (``mixer_scales``) are the layer's
    ``params``.  The weighted sums are taken in 32-bit by one kernel that also runs the
    norm that follows inside the block; nothing is left pending."""

    mixers = ("mixer",)
    has_feed_forward = True

    def __init__(self, parts, residual_scale: float = 1.0, mixer_scales=None):
        self.parts = dict(parts)
        self.mixer_norm = parts["mixer_norm"]
        self.mixer_parts = [parts[name] for name in self.mixers]
        self.feed_forward_norm = parts.get("feed_forward_norm")
        self.feed_forward = parts.get("feed_forward")
        self.residual_scale = float(residual_scale)
        scales = list(mixer_scales) if mixer_scales is not None else [1.0] * len(self.mixers)
        if len(scales) != len(self.mixers) or not 1 <= len(scales) <= 2:
            raise ValueError(f"{len(self.mixers)} mixers need as many scales, got {scales!r}")
        self.mixer_scales = [float(s) * self.residual_scale for s in scales]

    def forward(self, residual: torch.Tensor, pending: Optional[torch.Tensor], step,
                cache) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        from ..kernels import ops
        h = None
        if pending is None and all(getattr(p, "takes_stream", False)
                                   or getattr(p, "takes_normed_rows", False)
                                   for p in self.mixer_parts):
            # a decode batch: the mixers' opening products run the norm themselves (the
            # stream is added to only after every mixer has returned)
            h = self.mixer_norm.deferred(residual)
        if h is None:
            h = self.mixer_norm.add_forward(residual, pending)
        if len(self.mixers) == 1:
            outs = [self.mixer_parts[0].forward(h, step, cache)]
        else:
            outs = [part.forward(h, step, cache[name])
                    for name, part in zip(self.mixers, self.mixer_parts)]
        second = (outs[1], self.mixer_scales[1]) if len(outs) == 2 else (None, 0.0)
        if not self.has_feed_forward:
            ops.scaled_add_rmsnorm(residual, outs[0], self.mixer_scales[0], *second)
            return residual, None
        norm = self.feed_forward_norm
        if hasattr(norm, "weight") and hasattr(norm, "eps"):
            h = ops.scaled_add_rmsnorm(residual, outs[0], self.mixer_scales[0], *second,
                                       weight=norm.weight, eps=norm.eps, out_dtype=outs[0].dtype)
        else:
            ops.scaled_add_rmsnorm(residual, outs[0], self.mixer_scales[0], *second)
            h = norm.forward(residual)
        y = self.feed_forward.forward(h, step)
        ops.scaled_add_rmsnorm(residual, y, self.residual_scale)
        return residual, None


def _scaled_variant(kind: str, mixers, feed_forward: bool):
    slots = {"mixer_norm": "norm"}
    slots.update({name: "mixer" for name in mixers})
    if feed_forward:
        slots.update({"feed_forward_norm": "norm", "feed_forward": "feed_forward"})
    cls = type("ScaledResidualBlock_" + kind, (ScaledResidualBlock,),
               {"kind": kind, "slots": slots, "mixers": tuple(mixers),
                "has_feed_forward": feed_forward})
    register_arrangement(kind, cls)
    return cls


_scaled_variant("scaled_residual", ("mixer",), True)
_scaled_variant("scaled_residual_no_ff", ("mixer",), False)
_scaled_variant("scaled_residual_parallel", ("left", "right"), True)
_scaled_variant("scaled_residual_parallel_no_ff", ("left", "right"), False)
