"""Grouped-query attention over a paged cache, with optional per-head q/k norm.

Order of operations (reference: qwen3_runtime/models/qwen3.py:96-117):
one fused projection to q | k | v, reshape to heads, RMSNorm of every q head and
every k head over the head dimension with one weight per layer, position
encoding of q and k, keys (normed, rotated) and values (raw) written to the
cache before anything reads it, attention of every query over its sequence's
cache, output projection. Query head ``h`` reads key/value head ``h // g``,
``g = heads / kv_heads``; scores are ``q.k / sqrt(D)``, key ``j`` is visible
to the query at position ``i`` iff ``j <= i`` (and ``j > i - window`` when the
mixer has a window); softmax in float32
(reference: qwen3_runtime/attention/pytorch.py:12-47).

Options beyond that form, each a constructor argument: values of another size than keys
(``value_dim``); the q/k norm without weights (``qk_norm_weight=False``: the heads are divided
by their root mean square); a fixed score ``scale``; a cap on the scaled scores,
``softcap * tanh(score / softcap)``, before the softmax; a mask of chunks instead of a window
(``chunk``: key ``j`` is visible iff ``j <= i`` and ``j // chunk == i // chunk``, chunks counted
from position 0 of the sequence); an output gate (``output_gate``: one more projection ``g`` of
the mixer's input, whose sigmoid multiplies the concatenated heads before the output projection);
biases on the q, k and v projections (``bias``: tensors ``q_bias``, ``k_bias``, ``v_bias``, added to the
product's output in float32, before any rotation); beside a window, the sequence's first
``keep_first`` tokens stay visible to every later query (key ``j`` is visible iff ``j <= i`` and
``i - j < window or j < keep_first``; the cache keeps their pages); a ``sink`` in the softmax, one more
term of score 0 and no value in its denominator (``p_j = exp(s_j) / (1 + sum exp(s_j))``); the q/k norm
over the whole projection instead of per head (``qk_norm_scope="projection"``: all heads' query
elements of a token are divided by their one root mean square, weights ``q_norm`` of that whole
size, and likewise the keys); values that are the keys (``values_are_keys``: there is no ``v``
projection, a key head's value is that head's key as projected, bias included, before any norm); a
query temperature (``q_temp`` = (coef, every): the normed queries at position ``p`` are multiplied by
``1 + coef * ln(floor((p + 1) / every) + 1)``, float32).
"""

from __future__ import annotations

import math

import torch

from ..registry import part_class, register_part
from .base import Mixer
from .plan import CacheSpec, PartSpec, TensorDecl


@register_part("mixer", "gqa_attention")
class GroupedQueryAttention(Mixer):
    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        qk_norm_eps: float | None = None,
        position: PartSpec | None = None,
        window: int | None = None,
        scale: float | None = None,
        value_dim: int | None = None,
        qk_norm_weight: bool = True,
        softcap: float | None = None,
        chunk: int | None = None,
        output_gate: bool = False,
        bias: bool = False,
        keep_first: int = 0,
        sink: bool = False,
        qk_norm_scope: str = "head",
        values_are_keys: bool = False,
        q_temp: tuple[float, int] | None = None,
        tensors=None,
    ):
        super().__init__(tensors)
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads do not divide into {num_kv_heads} key/value heads")
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.qk_norm_eps = None if qk_norm_eps is None else float(qk_norm_eps)
        self.window = None if window is None else int(window)
        self.chunk = None if chunk is None else int(chunk)
        if self.window is not None and self.chunk is not None:
            raise ValueError("a mixer has a window or a mask of chunks, not both")
        self.value_dim = self.head_dim if value_dim is None else int(value_dim)
        self.qk_norm_weight = bool(qk_norm_weight)
        self.softcap = None if softcap is None else float(softcap)
        self.output_gate = bool(output_gate)
        self.has_bias = bool(bias)
        self.bias = None
        self.keep_first, self.sink = int(keep_first), bool(sink)
        if self.keep_first < 0 or (self.keep_first and self.window is None):
            raise ValueError("first tokens are kept in sight beside a window")
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        if qk_norm_scope not in ("head", "projection"):
            raise ValueError(f"unknown scope of the q/k norm {qk_norm_scope!r} (head, projection)")
        self.joint_norm = qk_norm_scope == "projection"
        self.values_are_keys = bool(values_are_keys)
        self.q_temp = None if q_temp is None else (float(q_temp[0]), int(q_temp[1]))
        if self.q_temp is not None and self.q_temp[1] < 1:
            raise ValueError(f"the query temperature counts positions in units of {self.q_temp[1]}")
        if self.joint_norm:
            # the form that one kernel serves: bias, norm over the projection, temperature, cache write
            if (self.qk_norm_eps is None or not self.qk_norm_weight or position is not None or output_gate
                    or self.value_dim != self.head_dim):
                raise ValueError("the q/k norm over the whole projection has weights and an eps, and goes without "
                                 "position encoding, output gate and values of another size than keys")
        elif self.values_are_keys or self.q_temp is not None:
            raise NotImplementedError("values that are the keys, and a query temperature, come with the q/k norm "
                                      "over the whole projection")
        if self.values_are_keys and self.value_dim != self.head_dim:
            raise ValueError("values that are the keys have the keys' size")
        self.position = None
        if position is not None:
            self.position = part_class("position", position.kind)(**position.args, tensors=position.tensors)
        self.qkv = self.o = self.q_norm = self.k_norm = None

    def children(self):
        return (self.position,) if self.position is not None else ()

    def cache_spec(self):
        return CacheSpec("paged_kv", heads=self.num_kv_heads, head_dim=self.head_dim, window=self.window,
                         chunk=self.chunk, value_dim=None if self.value_dim == self.head_dim else self.value_dim,
                         keep_first=self.keep_first)

    def tensor_decls(self):
        h, d, dv = self.hidden_size, self.head_dim, self.value_dim
        decls = [
            TensorDecl(self._name("q"), (self.num_heads * d, h)),
            TensorDecl(self._name("k"), (self.num_kv_heads * d, h)),
        ]
        if not self.values_are_keys:
            decls.append(TensorDecl(self._name("v"), (self.num_kv_heads * dv, h)))
        decls.append(TensorDecl(self._name("o"), (h, self.num_heads * dv)))
        if self.output_gate:
            decls.append(TensorDecl(self._name("g"), (self.num_heads * dv, h)))
        if self.has_bias:
            decls += [TensorDecl(self._name("q_bias"), (self.num_heads * d,)),
                      TensorDecl(self._name("k_bias"), (self.num_kv_heads * d,))]
            if not self.values_are_keys:
                decls.append(TensorDecl(self._name("v_bias"), (self.num_kv_heads * dv,)))
        if self.qk_norm_eps is not None and self.qk_norm_weight:
            nq, nk = (self.num_heads, self.num_kv_heads) if self.joint_norm else (1, 1)
            decls += [
                TensorDecl(self._name("q_norm"), (nq * d,), init="norm"),
                TensorDecl(self._name("k_norm"), (nk * d,), init="norm"),
            ]
        return decls

    def load(self, fetch):
        # one product for q | k | v (| gate): the gate reads the same input
        names = [self._name("q"), self._name("k")] + ([] if self.values_are_keys else [self._name("v")]) \
            + ([self._name("g")] if self.output_gate else [])
        self.qkv = fetch.fused(names, dim=0)
        self.o = fetch.matrix(self._name("o"))
        if self.has_bias:  # one vector over the product's columns; a gate's columns get zeros
            pieces = [fetch.vector_f32(self._name(n)) for n in ("q_bias", "k_bias", "v_bias")[: 2 if self.values_are_keys else 3]]
            if self.output_gate:
                pieces.append(torch.zeros(self.num_heads * self.value_dim, dtype=torch.float32, device=pieces[0].device))
            self.bias = fetch.constant(torch.cat(pieces))
        if self.qk_norm_eps is not None and self.qk_norm_weight:
            self.q_norm = fetch.vector_f32(self._name("q_norm"))
            self.k_norm = fetch.vector_f32(self._name("k_norm"))
        elif self.qk_norm_eps is not None:  # a norm without weights: weights of one
            self.q_norm = self.k_norm = fetch.constant(torch.ones(self.head_dim, dtype=torch.float32))

    def step_cost(self, spans, rows, elem_bytes):
        cost = super().step_cost(spans, rows, elem_bytes)  # the projections
        for q, kv in spans:  # scores and weighted values: 4 D operations per (query head, visible key)
            first = kv - q
            if self.window:
                pairs = sum(min(first + i + 1, self.window + self.keep_first) for i in range(q))
            elif self.chunk:
                pairs = sum((first + i) % self.chunk + 1 for i in range(q))
            else:
                pairs = q * first + q * (q + 1) // 2
            cost.flop += 2.0 * self.num_heads * (self.head_dim + self.value_dim) * pairs
        return cost

    def forward(self, ctx, x, cache):
        ops = ctx.ops
        nq, nkv, d, dv = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        qkv = ops.linear(x, self.qkv)
        eps = self.qk_norm_eps if self.qk_norm_eps is not None else 0.0
        if self.joint_norm:
            # biases, the norm over each whole projection, the queries' temperature and the cache
            # write (keys normed, values raw: the keys themselves, or the v columns) in one pass
            q = ops.qk_joint_norm_store(qkv, nq, nkv, d, self.bias, self.q_norm, self.k_norm, eps, ctx.positions,
                                        self.q_temp, self.values_are_keys, cache if cache.writes else None)
            more = {name: value for name, value in (("chunk", self.chunk), ("softcap", self.softcap),
                                                    ("keep_first", self.keep_first), ("sink", self.sink)) if value}
            attn = ops.paged_attention(q, cache, ctx, nq, nkv, d, self.scale, self.window, **more)
            return ops.linear_for_residual(attn, self.o)
        in_place = getattr(self.position, "in_place", False)
        if in_place:
            # biases and an encoding that works on the product where it lies: after it the mixer
            # goes on as one without encoding
            if self.qk_norm_eps is not None:
                raise NotImplementedError("a q/k norm in front of an encoding that works in place")
            self.position.rotate_in_place(ctx, qkv, nq + nkv, self.bias)
        elif self.bias is not None:
            ops.bias_rotate_pairs(qkv, self.bias, ctx.positions, None, 0, d)
        fused = self.position is None or in_place or self.position.fused_form == "neox_full"
        inv_freq = None if self.position is None or in_place or not fused else self.position.inv_freq
        # what only some designs have travels by name, and only where it is set
        more = {}
        if dv != d:
            more["value_dim"] = dv
        if self.chunk is not None:
            more["chunk"] = self.chunk
        if self.softcap is not None:
            more["softcap"] = self.softcap
        if self.keep_first:
            more["keep_first"] = self.keep_first
        if self.sink:
            more["sink"] = True
        gate_width = nq * dv if self.output_gate else 0
        if gate_width:
            # the gate's columns stay where the product put them: the attention reads them there
            more["gate"] = qkv[:, qkv.shape[1] - gate_width:]
        if fused and ops.fuses_decode_attention(ctx, qkv, nq, nkv, d, cache, **more):
            # a step of single tokens: all of it inside the attention kernel
            attn = ops.decode_attention(qkv, cache, ctx, nq, nkv, d, self.scale, self.window,
                                        self.q_norm, self.k_norm, eps, inv_freq,
                                        None if inv_freq is None else self.position.angles_key, **more)
            return ops.linear_for_residual(attn, self.o)
        if fused:
            # norm, rotation and the cache write in one pass over qkv
            shape = {k: more[k] for k in ("value_dim",) if k in more}
            if gate_width:
                shape["extra"] = gate_width
            q = ops.qk_norm_rope_store(
                qkv, nq, nkv, d, self.q_norm, self.k_norm, eps, inv_freq, ctx.positions,
                cache if cache.writes else None, ctx=ctx,
                angles_key=None if inv_freq is None else self.position.angles_key, **shape,
            )
        elif dv != d or gate_width:
            raise NotImplementedError("a position encoding without a fused form, with values of another size "
                                      "than keys or an output gate: the unfused steps do not take these")
        else:
            # an encoding the fused kernel has no form for: norm, let it rotate, then store
            q, k, v = ops.qk_norm_split(qkv, nq, nkv, d, self.q_norm, self.k_norm, eps)
            q, k = self.position.rotate(ctx, q, k)
            if cache.writes:
                ops.kv_store(k, v, cache)
            q = q.reshape(ctx.num_tokens, nq * d)
        attn = ops.paged_attention(q, cache, ctx, nq, nkv, d, self.scale, self.window, **more)
        return ops.linear_for_residual(attn, self.o)
