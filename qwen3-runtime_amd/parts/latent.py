"""Attention through a latent: keys and values (and, in one form, queries) are made from a low-rank vector.

From the mixer's input ``h``: ``c_q = rmsnorm(W_dq h)`` and ``q = W_uq c_q`` (or, with ``q_rank=None``,
``q = W_q h`` at full rank), laid out head by head
as ``dim`` elements that do not turn followed by ``rot_dim`` that do; ``W_dkv h`` gives ``kv_rank``
elements that, RMS-normed, are the latent ``c``, and ``rot_dim`` more that, rotated, are one key part
shared by all heads. Per head the plain key is ``W_uk c`` and the value ``W_uv c``; the score is
``(q_plain . k_plain + q_rot . k_rot) * scale``, causal (with ``window``: a query sees itself and the
``window - 1`` tokens before it), ordinary softmax. The concatenated heads are
multiplied by ``sigmoid(W_g h)`` (``output_gate``) and projected out. The rotation turns the first
``rot_dims`` elements of the rotated part by ``position * f_i``, ``f_i = base^(-2i/rot_dims)``: element
``i`` against ``i + rot_dims / 2`` (``rotation="half"``) or element ``2i`` against ``2i + 1`` (``"pairs"``).
``rot_scaling`` = (factor, original, fast, slow) stretches the frequencies as YaRN does: with
``pair(t) = rot_dims ln(original / (2 pi t)) / (2 ln base)``, ``lo = max(floor(pair(fast)), 0)``,
``hi = min(ceil(pair(slow)), rot_dims - 1)`` and ``ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)``
the frequency is ``f_i / factor * ramp_i + f_i (1 - ramp_i)``, and cosines and sines are multiplied
by ``0.1 ln(factor) + 1``; ``scale`` is taken as given.

Only ``c`` and the rotated key part are cached, and the attention runs on them directly: since
``q_plain . (W_uk c) = (W_uk^T q_plain) . c``, every head's query becomes ``[W_uk^T q_plain | q_rot]``,
``kv_rank + rot_dim`` wide, all heads read the one cached row ``[c | k_rot]`` as their key and ``c`` as
their value, and ``W_uv`` is applied to the attention's output. To the attention kernels this is
grouped-query attention with one key/value head of size ``kv_rank + rot_dim`` whose value row is
the latent followed by ``rot_dim`` zeros, which lets keys and values share one head size.

``own_latent=False``: the layer has no ``W_dkv``; it reads the cache that another layer of equal
``kv_rank``, ``rot_dim`` and rotation wrote in the same pass (the plan's step names that cache and
does not write it), with matrices, queries and window of its own. ``cache_window`` is then the
window of the cache's owner, which keeps what its widest reader sees.
"""

from __future__ import annotations

import math

import torch

from ..registry import register_part
from .base import Mixer
from .plan import CacheSpec, TensorDecl


def stretched_frequencies(dims: int, base: float, scaling=None) -> tuple[torch.Tensor, float]:
    """(float32 [dims / 2], what multiplies cosines and sines): ``base^(-2i/dims)``, stretched by
    ``scaling`` = (factor, original, fast, slow) as the module's text says. Computed in float64 and
    rounded once."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / max(dims, 1))
    if scaling is None:
        return f.to(torch.float32), 1.0
    factor, original, fast, slow = (float(v) for v in scaling)

    def pair(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo, hi = max(math.floor(pair(fast)), 0), min(math.ceil(pair(slow)), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return (f / factor * ramp + f * (1.0 - ramp)).to(torch.float32), 0.1 * math.log(factor) + 1.0


@register_part("mixer", "latent_attention")
class LatentAttention(Mixer):
    """``tensors``: ``dq``, ``dq_norm``, ``uq`` (or ``q``), ``dkv``, ``dkv_norm`` (a latent of its own), ``uk``, ``uv``,
    ``g`` (an output gate), ``o``."""

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, value_dim: int, q_rank: int | None,
                 kv_rank: int, scale: float, norm_eps: float, rot_dims: int, rot_base: float, output_gate: bool = True,
                 window: int | None = None, cache_window=..., rotation: str = "half", rot_scaling=None,
                 own_latent: bool = True, tensors=None):
        super().__init__(tensors)
        self.hidden_size, self.heads = int(hidden_size), int(num_heads)
        self.dim, self.rot_dim, self.vdim = int(head_dim), int(rot_dim), int(value_dim)
        self.q_rank, self.kv_rank = None if q_rank is None else int(q_rank), int(kv_rank)
        self.scale, self.eps = float(scale), float(norm_eps)
        self.rot_dims, self.rot_base = int(rot_dims), float(rot_base)
        if self.rot_dims % 2 or not 0 <= self.rot_dims <= self.rot_dim:
            raise ValueError(f"{rot_dims} rotated elements in a part of {rot_dim}: even, and no more than the part")
        if rotation not in ("half", "pairs"):
            raise ValueError(f"unknown rotation {rotation!r} (half, pairs)")
        self.output_gate, self.own_latent, self.neighbours = bool(output_gate), bool(own_latent), rotation == "pairs"
        self.window = None if window is None else int(window)
        self.cache_window = self.window if cache_window is ... else (None if cache_window is None else int(cache_window))
        if self.cache_window is not None and (self.window is None or self.window > self.cache_window):
            raise ValueError(f"a cache that keeps {self.cache_window} tokens under a window of {self.window}")
        # frequencies in float64, rounded once; angles are float32 products of position and frequency
        self.freq_cpu, self.magnitude = stretched_frequencies(self.rot_dims, self.rot_base, rot_scaling)
        self.down = self.uq = self.uk_t = self.uv = self.o = None
        self.dq_norm = self.dkv_norm = self.freq = None

    @property
    def latent_width(self) -> int:
        return self.kv_rank + self.rot_dim

    def cache_spec(self):
        # one key/value head: the row [c | k_rot] as key, [c | 0] as value
        return CacheSpec("paged_kv", heads=1, head_dim=self.latent_width, window=self.cache_window)

    @property
    def query_width(self) -> int:
        return self.heads * (self.dim + self.rot_dim)

    def _first(self) -> list[str]:
        """The matrices that multiply the mixer's input, in the order of the fused product's columns:
        queries (or their latent) | key/value latent and rotated key part | gate."""
        names = ["q" if self.q_rank is None else "dq"]
        return names + (["dkv"] if self.own_latent else []) + (["g"] if self.output_gate else [])

    def tensor_decls(self):
        h, n = self.hidden_size, self.heads
        if self.q_rank is None:
            decls = [TensorDecl(self._name("q"), (self.query_width, h))]
        else:
            decls = [TensorDecl(self._name("dq"), (self.q_rank, h)),
                     TensorDecl(self._name("dq_norm"), (self.q_rank,), init="norm"),
                     TensorDecl(self._name("uq"), (self.query_width, self.q_rank))]
        if self.own_latent:
            decls += [TensorDecl(self._name("dkv"), (self.latent_width, h)),
                      TensorDecl(self._name("dkv_norm"), (self.kv_rank,), init="norm")]
        decls += [TensorDecl(self._name("uk"), (n * self.dim, self.kv_rank)),
                  TensorDecl(self._name("uv"), (n * self.vdim, self.kv_rank))]
        if self.output_gate:
            decls.append(TensorDecl(self._name("g"), (n * self.vdim, h)))
        return decls + [TensorDecl(self._name("o"), (h, n * self.vdim))]

    def load(self, fetch):
        n = self.heads
        # one product of the mixer's input
        first = [self._name(name) for name in self._first()]
        self.down = fetch.fused(first, dim=0) if len(first) > 1 else fetch.matrix(first[0])
        if self.q_rank is not None:
            self.uq = fetch.matrix(self._name("uq"))
            self.dq_norm = fetch.vector_f32(self._name("dq_norm"))
        # per head [kv_rank, dim]: the plain key's matrix transposed, which takes a query to the latent
        uk = fetch.matrix(self._name("uk")).view(n, self.dim, self.kv_rank)
        self.uk_t = fetch.constant(uk.transpose(1, 2).contiguous())
        self.uv = fetch.matrix(self._name("uv")).view(n, self.vdim, self.kv_rank)
        self.o = fetch.matrix(self._name("o"))
        if self.own_latent:
            self.dkv_norm = fetch.vector_f32(self._name("dkv_norm"))
        self.freq = fetch.constant(self.freq_cpu) if self.rot_dims else None

    def step_cost(self, spans, rows, elem_bytes):
        cost = super().step_cost(spans, rows, elem_bytes)
        for q, kv in spans:  # scores over the latent row, values of the latent
            if self.window:
                pairs = sum(min(kv - q + i + 1, self.window) for i in range(q))
            else:
                pairs = q * (kv - q) + q * (q + 1) // 2
            cost.flop += 2.0 * self.heads * (self.latent_width + self.kv_rank) * pairs
        return cost

    def forward(self, ctx, x, cache):
        ops = ctx.ops
        n, w, dr = self.heads, self.latent_width, self.dim + self.rot_dim
        turn = {"neighbours": True, "magnitude": self.magnitude} if self.neighbours or self.magnitude != 1.0 else {}
        y = ops.linear(x, self.down)
        if self.q_rank is None:
            q, at = y, self.query_width  # the queries are the product's first columns
        else:
            q, at = ops.linear(ops.rmsnorm_columns(y, 0, self.q_rank, self.dq_norm, self.eps), self.uq), self.q_rank
        if self.own_latent:
            # norm of the latent, rotation of the shared key part, and the cache write, in one pass
            ops.latent_store(y, at, self.kv_rank, self.rot_dim, self.dkv_norm, self.eps, ctx.positions, self.freq,
                             cache if cache.writes else None, **turn)
            at += w
        elif cache.writes:
            raise ValueError("a layer without a latent of its own reads a cache that another layer writes")
        # queries as the cached rows see them: [W_uk^T q_plain | rotated part] per head
        ql = ops.new_rows(ctx.num_tokens, n * w, q.dtype, x.device)
        ops.heads_linear(q, dr, 0, self.uk_t, ql, w, 0)
        ops.rotate_half(q, dr, self.dim, ql, w, self.kv_rank, n, self.rot_dim, ctx.positions, self.freq, **turn)
        attn = ops.paged_attention(ql, cache, ctx, n, 1, w, self.scale, self.window)
        out = ops.new_rows(ctx.num_tokens, n * self.vdim, q.dtype, x.device)
        ops.heads_linear(attn, w, 0, self.uv, out, self.vdim, 0)
        if self.output_gate:
            ops.sigmoid_gate(out, y[:, at: at + n * self.vdim])
        return ops.linear_for_residual(out, self.o)
