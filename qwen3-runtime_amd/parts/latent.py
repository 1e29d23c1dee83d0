"""Attention through a latent: queries and keys/values are each made from a low-rank vector.

From the mixer's input ``h``: ``c_q = rmsnorm(W_dq h)`` and ``q = W_uq c_q``, laid out head by head
as ``dim`` elements that do not turn followed by ``rot_dim`` that do; ``W_dkv h`` gives ``kv_rank``
elements that, RMS-normed, are the latent ``c``, and ``rot_dim`` more that, rotated, are one key part
shared by all heads. Per head the plain key is ``W_uk c`` and the value ``W_uv c``; the score is
``(q_plain . k_plain + q_rot . k_rot) * scale``, causal, ordinary softmax. The concatenated heads are
multiplied by ``sigmoid(W_g h)`` and projected out. The rotation turns the first ``rot_dims`` elements of
the rotated part, element ``i`` against ``i + rot_dims / 2``, by ``position * base^(-2i/rot_dims)``.

Only ``c`` and the rotated key part are cached, and the attention runs on them directly: since
``q_plain . (W_uk c) = (W_uk^T q_plain) . c``, every head's query becomes ``[W_uk^T q_plain | q_rot]``,
``kv_rank + rot_dim`` wide, all heads read the one cached row ``[c | k_rot]`` as their key and ``c`` as
their value, and ``W_uv`` is applied to the attention's output. To the attention kernels this is
grouped-query attention with one key/value head of size ``kv_rank + rot_dim`` whose value row is
the latent followed by ``rot_dim`` zeros, which lets keys and values share one head size.
"""

from __future__ import annotations

import torch

from ..registry import register_part
from .base import Mixer
from .plan import CacheSpec, TensorDecl


@register_part("mixer", "latent_attention")
class LatentAttention(Mixer):
    """``tensors``: ``dq``, ``dq_norm``, ``uq``, ``dkv``, ``dkv_norm``, ``uk``, ``uv``, ``g``, ``o``."""

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, value_dim: int, q_rank: int,
                 kv_rank: int, scale: float, norm_eps: float, rot_dims: int, rot_base: float, tensors=None):
        super().__init__(tensors)
        self.hidden_size, self.heads = int(hidden_size), int(num_heads)
        self.dim, self.rot_dim, self.vdim = int(head_dim), int(rot_dim), int(value_dim)
        self.q_rank, self.kv_rank = int(q_rank), int(kv_rank)
        self.scale, self.eps = float(scale), float(norm_eps)
        self.rot_dims, self.rot_base = int(rot_dims), float(rot_base)
        if self.rot_dims % 2 or not 0 <= self.rot_dims <= self.rot_dim:
            raise ValueError(f"{rot_dims} rotated elements in a part of {rot_dim}: even, and no more than the part")
        # frequencies in float64, rounded once; angles are float32 products of position and frequency
        i = torch.arange(self.rot_dims // 2, dtype=torch.float64)
        self.freq_cpu = (self.rot_base ** (-2.0 * i / max(self.rot_dims, 1))).to(torch.float32)
        self.down = self.uq = self.uk_t = self.uv = self.o = None
        self.dq_norm = self.dkv_norm = self.freq = None

    @property
    def latent_width(self) -> int:
        return self.kv_rank + self.rot_dim

    def cache_spec(self):
        # one key/value head: the row [c | k_rot] as key, [c | 0] as value
        return CacheSpec("paged_kv", heads=1, head_dim=self.latent_width)

    def tensor_decls(self):
        h, n = self.hidden_size, self.heads
        return [TensorDecl(self._name("dq"), (self.q_rank, h)),
                TensorDecl(self._name("dq_norm"), (self.q_rank,), init="norm"),
                TensorDecl(self._name("uq"), (n * (self.dim + self.rot_dim), self.q_rank)),
                TensorDecl(self._name("dkv"), (self.latent_width, h)),
                TensorDecl(self._name("dkv_norm"), (self.kv_rank,), init="norm"),
                TensorDecl(self._name("uk"), (n * self.dim, self.kv_rank)),
                TensorDecl(self._name("uv"), (n * self.vdim, self.kv_rank)),
                TensorDecl(self._name("g"), (n * self.vdim, h)),
                TensorDecl(self._name("o"), (h, n * self.vdim))]

    def load(self, fetch):
        n = self.heads
        # one product of the mixer's input: query latent | key/value latent and rotated key part | gate
        self.down = fetch.fused([self._name("dq"), self._name("dkv"), self._name("g")], dim=0)
        self.uq = fetch.matrix(self._name("uq"))
        # per head [kv_rank, dim]: the plain key's matrix transposed, which takes a query to the latent
        uk = fetch.matrix(self._name("uk")).view(n, self.dim, self.kv_rank)
        self.uk_t = fetch.constant(uk.transpose(1, 2).contiguous())
        self.uv = fetch.matrix(self._name("uv")).view(n, self.vdim, self.kv_rank)
        self.o = fetch.matrix(self._name("o"))
        self.dq_norm = fetch.vector_f32(self._name("dq_norm"))
        self.dkv_norm = fetch.vector_f32(self._name("dkv_norm"))
        self.freq = fetch.constant(self.freq_cpu) if self.rot_dims else None

    def step_cost(self, spans, rows, elem_bytes):
        cost = super().step_cost(spans, rows, elem_bytes)
        for q, kv in spans:  # scores over the latent row, values of the latent
            pairs = q * (kv - q) + q * (q + 1) // 2
            cost.flop += 2.0 * self.heads * (self.latent_width + self.kv_rank) * pairs
        return cost

    def forward(self, ctx, x, cache):
        ops = ctx.ops
        n, w = self.heads, self.latent_width
        y = ops.linear(x, self.down)
        cq = ops.rmsnorm_columns(y, 0, self.q_rank, self.dq_norm, self.eps)
        q = ops.linear(cq, self.uq)
        # norm of the latent, rotation of the shared key part, and the cache write, in one pass
        ops.latent_store(y, self.q_rank, self.kv_rank, self.rot_dim, self.dkv_norm, self.eps, ctx.positions, self.freq,
                         cache if cache.writes else None)
        # queries as the cached rows see them: [W_uk^T q_plain | rotated part] per head
        ql = ops.new_rows(ctx.num_tokens, n * w, q.dtype, x.device)
        ops.heads_linear(q, self.dim + self.rot_dim, 0, self.uk_t, ql, w, 0)
        ops.rotate_half(q, self.dim + self.rot_dim, self.dim, ql, w, self.kv_rank, n, self.rot_dim, ctx.positions, self.freq)
        attn = ops.paged_attention(ql, cache, ctx, n, 1, w, self.scale, None)
        out = ops.new_rows(ctx.num_tokens, n * self.vdim, q.dtype, x.device)
        ops.heads_linear(attn, w, 0, self.uv, out, self.vdim, 0)
        gate_first = self.q_rank + w
        ops.sigmoid_gate(out, y[:, gate_first: gate_first + n * self.vdim])
        return ops.linear_for_residual(out, self.o)
