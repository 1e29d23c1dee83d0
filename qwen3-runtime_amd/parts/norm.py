"""Norms with the residual update fused in front of them.

``rmsnorm``: ``y = x * rsqrt(mean(x^2) + eps) * w`` over the last dimension, all in
float32, the weight multiplying after normalisation, no offset, no bias; with ``delta_scale``
the pending output joins the stream as ``x + delta_scale * delta``
(reference: qwen3_runtime/layers/ops.py:17-20). The fused form first adds the
pending sub-layer output into the residual stream
(reference: qwen3_runtime/layers/ops.py:28-37), here in float32.

``layernorm``: ``y = (x - mean) / sqrt(var + eps) * w + b`` with the variance the mean of the
squared deviations, float32.

Either norm also serves several residual streams ``[T, S, H]`` (hyper-connections): the update
that is pending is then a ``StreamUpdate`` (the streams mixed among themselves plus the
sub-layer's output times a weight per stream), and what is normalised is the sum of the
streams weighted by ``read``; a ``ScaledUpdate`` (the outputs of sub-layers that ran side by side,
each times a vector) joins one stream as ``x + sum_i s_i * y_i``; a norm built with ``streams=S`` and called without ``read`` takes
the plain sum (the model's last norm).
"""

from __future__ import annotations

import torch

from ..registry import register_part
from .base import Norm, NormedUpdate, ScaledUpdate
from .plan import TensorDecl


@register_part("norm", "rmsnorm")
class RMSNorm(Norm):
    has_bias = False

    def __init__(self, size: int, eps: float, streams: int = 1, delta_scale: float = 1.0, tensors=None):
        super().__init__(tensors)
        self.size = int(size)
        self.eps = float(eps)
        self.streams = int(streams)
        self.weight = self.bias = self.read_all = None
        # what multiplies a pending sub-layer output as it joins the stream (1: the plain sum)
        self.delta_scale = float(delta_scale)
        if self.delta_scale != 1.0 and (self.streams > 1 or self.has_bias):
            raise ValueError("a scaled residual sum goes with the RMS norm over one stream")

    def tensor_decls(self):
        decls = [TensorDecl(self._name("weight"), (self.size,), init="norm")]
        if self.has_bias:
            decls.append(TensorDecl(self._name("bias"), (self.size,), init="matrix"))
        return decls

    def load(self, fetch):
        self.weight = fetch.vector_f32(self._name("weight"))
        if self.has_bias:
            self.bias = fetch.vector_f32(self._name("bias"))
        if self.streams > 1:
            self.read_all = fetch.constant(torch.ones(self.streams, dtype=torch.float32))

    def forward(self, ctx, residual, delta=None, rows=None, read=None):
        """Apply ``delta`` to ``residual`` (in place), return its normalised rows.

        With ``rows`` (int32 indices) only those rows are normalised and
        returned, packed; ``residual`` is then left as it is.
        """
        if residual.dim() == 3:  # several streams
            return ctx.ops.mix_norm(residual, delta, self.read_all if read is None else read, self.weight,
                                    self.bias, self.eps, ctx.dtype, rows)
        if isinstance(delta, NormedUpdate):
            # a sub-layer output that is normed on its way into the stream
            if self.has_bias or self.delta_scale != 1.0:
                raise NotImplementedError("a normed update meets the plain RMS norm only")
            return ctx.ops.add_rmsnorm(residual, delta.y, self.weight, self.eps, ctx.dtype, rows,
                                       delta_norm=(delta.weight, delta.eps))
        if isinstance(delta, ScaledUpdate):
            # outputs of sub-layers that ran side by side, each times its vector
            if self.has_bias or self.delta_scale != 1.0:
                raise NotImplementedError("a sum of scaled updates meets the plain RMS norm only")
            return ctx.ops.scaled_add_rmsnorm(residual, delta.parts, self.weight, self.eps, ctx.dtype, rows)
        if self.has_bias:
            return ctx.ops.mix_norm(residual, delta, None, self.weight, self.bias, self.eps, ctx.dtype, rows)
        if self.delta_scale != 1.0:
            return ctx.ops.add_rmsnorm(residual, delta, self.weight, self.eps, ctx.dtype, rows, delta_scale=self.delta_scale)
        return ctx.ops.add_rmsnorm(residual, delta, self.weight, self.eps, ctx.dtype, rows)


@register_part("norm", "layernorm")
class LayerNorm(RMSNorm):
    has_bias = True
