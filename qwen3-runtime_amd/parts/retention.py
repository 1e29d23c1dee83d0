"""Retention: linear attention with a fixed decay per head, no softmax and no denominator.

From the mixer's input ``h``: ``q = W_q h`` and ``k = W_k h`` (``heads x dim``), ``v = W_v h``
(``heads x vdim``), no biases. The first ``rot_dims`` elements of every query and key head turn,
element ``i`` against ``i + rot_dims / 2``, by ``position * base^(-2i/rot_dims)``; keys are then
multiplied by ``dim^(-1/2)``. Per head, with its constant ``decay``::

    S <- decay S + k v^T;  o = S^T q

Each head's ``o`` is divided by its root mean square over ``vdim`` (no weight), the heads are
concatenated, multiplied by ``silu(W_g h)`` and projected out. ``S`` starts at zero, is float32 and
is the request's state, kept in its slot from step to step; rotation, scaling, recurrence and the
read-out's norm are float32.
"""

from __future__ import annotations

import torch

from ..registry import register_part
from .base import Mixer
from .plan import CacheSpec, TensorDecl


@register_part("mixer", "retention")
class Retention(Mixer):
    """``tensors``: ``q``, ``k``, ``v``, ``g``, ``o``."""

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, decay, norm_eps: float,
                 rot_dims: int, rot_base: float, tensors=None):
        super().__init__(tensors)
        self.hidden_size, self.heads = int(hidden_size), int(num_heads)
        self.dim, self.vdim = int(head_dim), int(value_dim)
        self.decay_cpu = torch.tensor([float(x) for x in decay], dtype=torch.float32)
        if self.decay_cpu.numel() != self.heads:
            raise ValueError(f"{self.decay_cpu.numel()} decays for {self.heads} heads")
        if not 1 <= self.dim <= 512:
            raise ValueError(f"the state's rows are held in registers: key size 1 to 512, not {head_dim}")
        self.eps = float(norm_eps)
        self.rot_dims, self.rot_base = int(rot_dims), float(rot_base)
        if self.rot_dims % 2 or not 0 <= self.rot_dims <= self.dim:
            raise ValueError(f"{rot_dims} rotated elements in heads of {head_dim}: even, and no more than the head")
        i = torch.arange(self.rot_dims // 2, dtype=torch.float64)
        self.freq_cpu = (self.rot_base ** (-2.0 * i / max(self.rot_dims, 1))).to(torch.float32)
        self.proj = self.o = self.decay = self.freq = self.ones = None

    def cache_spec(self):
        # the state transposed, [heads, vdim, dim]: a value channel's column of S is contiguous
        return CacheSpec("state", shape=(self.heads, self.vdim, self.dim), dtype="float32")

    def tensor_decls(self):
        h, n = self.hidden_size, self.heads
        return [TensorDecl(self._name("q"), (n * self.dim, h)), TensorDecl(self._name("k"), (n * self.dim, h)),
                TensorDecl(self._name("v"), (n * self.vdim, h)), TensorDecl(self._name("g"), (n * self.vdim, h)),
                TensorDecl(self._name("o"), (h, n * self.vdim))]

    def load(self, fetch):
        self.proj = fetch.fused([self._name(n) for n in ("q", "k", "v", "g")], dim=0)
        self.o = fetch.matrix(self._name("o"))
        self.decay = fetch.constant(self.decay_cpu)
        self.freq = fetch.constant(self.freq_cpu) if self.rot_dims else None
        self.ones = fetch.constant(torch.ones(self.vdim, dtype=torch.float32))  # the read-out's norm has no weight

    def step_cost(self, spans, rows, elem_bytes):
        cost = super().step_cost(spans, rows, elem_bytes)
        tokens = sum(q for q, _ in spans)
        # per token and head: decay and write, and one sum over the state's rows: 2 passes over D x Dv
        cost.flop += 2.0 * 2 * tokens * self.heads * self.dim * self.vdim
        return cost

    def forward(self, ctx, x, cache):
        ops = ctx.ops
        n = self.heads
        y = ops.linear(x, self.proj)
        qkv = ops.retention_prepare(y, n, self.dim, self.vdim, ctx.positions, self.freq, self.dim ** -0.5)
        o = ops.retention_rule(ctx, qkv, self.decay, cache.state, n, self.dim, self.vdim)
        gate_first = 2 * n * self.dim + n * self.vdim
        out = ops.delta_out(o, self.ones, y[:, gate_first: gate_first + n * self.vdim], self.eps, "silu", ctx.dtype)
        return ops.linear_for_residual(out, self.o)
