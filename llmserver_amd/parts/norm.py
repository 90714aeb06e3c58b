"""RMSNorm fused with the residual sum.

``y = s * rsqrt(mean(s^2) + eps) * w`` with ``s = resid + delta`` and everything in 32-bit inside
(utils/layers.py:131-138; fused form utils/fused_ops.py:23-26,
65-78).  ``s`` is rounded to the activation dtype once, when it is stored back as the new
residual stream (utils/fused_ops.py:73).
"""
from __future__ import annotations

from .base import VECTOR, Norm, ParamSpec


class RMSNorm(Norm):
    """``offset``: what is added to the stored weight before it multiplies (0: the weight as stored; 1: a weight that
    is stored around zero).  The sum is formed once, in 32-bit, when the tensor has been loaded, so every kernel sees a
    plain weight.  ``tensor``: the weight's name below the part's own ("" if the part's name is the tensor's).  ``scale``:
    a constant that multiplies the result (a model whose logits are a multiple of the head's product of the normed rows
    says so here); it joins the weight in 32-bit when the tensor has been loaded.  ``single``: the checkpoint holds one
    number that multiplies every coordinate; it is spread over the width when it has been loaded, so every kernel sees a
    plain weight."""

    def __init__(self, width: int, eps: float, offset: float = 0.0, tensor: str = "weight", scale: float = 1.0, single: bool = False):
        self.width = width
        self.single = bool(single)
        self.eps = float(eps)
        self.offset = float(offset)
        self.scale = float(scale)
        self.tensor = tensor
        self.weight = None  # float32 [width], the offset added and the scale multiplied in

    def param_specs(self):
        return {self.tensor: ParamSpec(() if self.single else (self.width,), VECTOR, "bias" if self.offset else "norm")}

    def assign(self, name, tensor):
        assert name == self.tensor
        if self.single:
            tensor = tensor.reshape(1).expand(self.width).contiguous()
        self.weight = tensor + self.offset if self.offset else tensor
        if self.scale != 1.0:
            self.weight = self.weight * self.scale

    def add_norm(self, resid, delta, ctx, rows=None):
        n = resid.shape[0] if rows is None else rows.shape[0]
        out = ctx.empty((n, self.width))
        if resid.dtype != out.dtype:
            # A stream that is kept in 32-bit beside 16-bit activations: nothing is added here, rows are normalised
            # in 32-bit and rounded once for the product that follows.
            if delta is not None:
                raise ValueError("a 32-bit residual stream takes its updates where they are made, not in the norm")
            ctx.ops.norm_rows(resid, rows, self.weight, self.eps, out)
            return out
        ctx.ops.add_rmsnorm(resid, delta, self.weight, self.eps, out, rows)
        return out

    def row_scale_form(self):
        return self.weight, self.eps


class StreamReadNorm(RMSNorm):
    """The norm of what a sublayer reads from several residual streams: ``rmsnorm(sum_s read[s] * x_s) * w`` for streams
    ``x [S, T, W]`` kept in 32-bit.  ``read`` belongs to whoever connects the sublayer to the streams (a block's
    :class:`~llmserver_amd.parts.block.HyperConnection`, which sets ``read_weights``); left alone, the streams are
    summed as they are, which is also how a model reads its streams in front of the head."""

    def __init__(self, width: int, eps: float, streams: int, tensor: str = "weight", scale: float = 1.0):
        super().__init__(width, eps, tensor=tensor, scale=scale)
        self.streams = int(streams)
        self.read_weights = None    # float32 [streams]

    def finalize(self):
        if self.read_weights is None:
            self.read_weights = self.weight.new_ones((self.streams,))

    def add_norm(self, resid, delta, ctx, rows=None):
        if delta is not None:
            raise ValueError("several residual streams take their updates where they are made, not in the norm")
        n = resid.shape[1] if rows is None else rows.shape[0]
        out = ctx.empty((n, self.width))
        ctx.ops.streams_read(resid, self.read_weights, self.weight, self.eps, out, rows)
        return out

    def row_scale_form(self):
        return None
