"""Arrangements of a layer's parts: the pre-norm residual block, over one residual stream or
over several (hyper-connections), the block with a norm on both sides of each sub-layer, and
the block whose mixer and feed-forward read one norm and join the stream in one scaled sum.

``x += mixer(norm_in(x)); x += feed_forward(norm_post(x))``: the form the
reference's oracle writes (tests/cpu/reference_qwen3.py:79-110) and its model
computes as a chain of fused add-norms (qwen3_runtime/models/qwen3.py:165-187).
Here the block receives the residual stream and the previous sub-layer's
output that is still to be added, and hands both on, so that each add fuses
with the norm that follows it without a block knowing its neighbour.
"""

from __future__ import annotations

from ..registry import register_part
from .base import Block, NormedUpdate, ScaledUpdate, StreamUpdate
from .plan import TensorDecl


@register_part("block", "pre_norm")
class PreNormBlock(Block):
    norm_names = ("input", "post_mixer")

    def __init__(self, mixer, feed_forward, norms, tensors=None):
        super().__init__(tensors)
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norm_in = norms["input"]
        self.norm_post = norms.get("post_mixer")

    def children(self):
        return tuple(p for p in (self.norm_in, self.mixer, self.norm_post, self.feed_forward) if p is not None)

    def forward(self, ctx, residual, delta, cache):
        x = self.norm_in.forward(ctx, residual, delta)
        mixed = self.mixer.forward(ctx, x, cache)
        if self.feed_forward is None:  # a layer of a mixer alone
            return residual, mixed
        x = self.norm_post.forward(ctx, residual, mixed)
        return residual, self.feed_forward.forward(ctx, x)


@register_part("block", "sandwich_norm")
class SandwichNormBlock(Block):
    """A norm on both sides of each sub-layer: ``x += norm_after(mixer(norm_in(x)))``, then
    ``x += norm_after_ff(feed_forward(norm_post(x)))``. The norm behind a sub-layer goes with its
    output as a ``NormedUpdate``, so that the norm in front of the next sub-layer applies it, adds
    and normalises in one pass over the stream."""

    norm_names = ("input", "after_mixer", "post_mixer", "after_ff")

    def __init__(self, mixer, feed_forward, norms, tensors=None):
        super().__init__(tensors)
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norm_in, self.after_mixer = norms["input"], norms["after_mixer"]
        self.norm_post, self.after_ff = norms.get("post_mixer"), norms.get("after_ff")
        if feed_forward is not None and (self.norm_post is None or self.after_ff is None):
            raise ValueError("a feed-forward comes with the norms in front of it and behind it")

    def children(self):
        return tuple(p for p in (self.norm_in, self.mixer, self.after_mixer, self.norm_post, self.feed_forward,
                                 self.after_ff) if p is not None)

    def forward(self, ctx, residual, delta, cache):
        x = self.norm_in.forward(ctx, residual, delta)
        pending = NormedUpdate(self.mixer.forward(ctx, x, cache), self.after_mixer.weight, self.after_mixer.eps)
        if self.feed_forward is None:
            return residual, pending
        x = self.norm_post.forward(ctx, residual, pending)
        return residual, NormedUpdate(self.feed_forward.forward(ctx, x), self.after_ff.weight, self.after_ff.eps)


@register_part("block", "hyper_connections")
class HyperConnectionBlock(Block):
    """Pre-norm sub-layers over ``streams`` residual streams ``x[T, S, H]`` that all start as the
    embedding. Sub-layer ``q`` (1 the mixer, 2 the feed-forward) reads ``u = sum_s in_q[s] x_s``,
    computes ``y = f(norm(u))``, and leaves ``x_t <- sum_s mix_q[s, t] x_s + out_q[t] y`` to the
    norm that comes next, which applies it in the pass in which it reads the streams: the one
    kernel between two sub-layers does the write of one and the read of the other. A block without
    feed-forward has the first sub-layer only. The model's last norm sums the streams."""

    norm_names = ("input", "post_mixer")

    def __init__(self, mixer, feed_forward, norms, streams: int, tensors=None):
        super().__init__(tensors)
        self.streams = int(streams)
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norm_in = norms["input"]
        self.norm_post = norms.get("post_mixer")
        if (feed_forward is None) != (self.norm_post is None):
            raise ValueError("a feed-forward and the norm in front of it come together")
        self.coeff: dict[str, object] = {}

    def children(self):
        return tuple(p for p in (self.norm_in, self.mixer, self.norm_post, self.feed_forward) if p is not None)

    def _sublayers(self):
        return ("1",) if self.feed_forward is None else ("1", "2")

    def tensor_decls(self):
        s = self.streams
        decls = []
        for q in self._sublayers():
            decls += [TensorDecl(self._name(f"in{q}"), (s,), init="norm"),
                      TensorDecl(self._name(f"out{q}"), (s,), init="norm"),
                      TensorDecl(self._name(f"mix{q}"), (s, s), init="mixing")]
        return decls

    def load(self, fetch):
        for q in self._sublayers():
            for name in (f"in{q}", f"out{q}", f"mix{q}"):
                self.coeff[name] = fetch.vector_f32(self._name(name))

    def step_cost(self, spans, rows, elem_bytes):
        cost = super().step_cost(spans, rows, elem_bytes)
        cost.flop = 0.0  # coefficients, not matrices that multiply tokens
        return cost

    def forward(self, ctx, residual, delta, cache):
        if residual.dim() == 2:
            # the one stream that the embedding began: every stream starts as a copy of it
            if delta is not None:
                raise ValueError("the residual streams begin at the embedding, with nothing pending")
            t, h = residual.shape
            residual = residual[:, None, :].expand(t, self.streams, h).contiguous()
        c = self.coeff
        x = self.norm_in.forward(ctx, residual, delta, read=c["in1"])
        pending = StreamUpdate(self.mixer.forward(ctx, x, cache), c["mix1"], c["out1"])
        if self.feed_forward is None:
            return residual, pending
        x = self.norm_post.forward(ctx, residual, pending, read=c["in2"])
        return residual, StreamUpdate(self.feed_forward.forward(ctx, x), c["mix2"], c["out2"])


@register_part("block", "parallel_scaled")
class ParallelScaledBlock(Block):
    """Mixer and feed-forward side by side: one norm, ``n = norm_in(x)``, both read it, and
    ``x <- x + s1 * mixer(n) + s2 * feed_forward(n)`` with a vector per sub-layer (tensors ``scale1``,
    ``scale2``; ``layer_scale=False``: no vectors, the plain sum). The two outputs go on as one
    ``ScaledUpdate``, which the next layer's norm adds in the pass in which it normalises. A block
    without feed-forward has the first term only."""

    norm_names = ("input",)

    def __init__(self, mixer, feed_forward, norms, hidden_size: int, layer_scale: bool = True, tensors=None):
        super().__init__(tensors)
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norm_in = norms["input"]
        self.hidden_size, self.layer_scale = int(hidden_size), bool(layer_scale)
        self.scale1 = self.scale2 = None

    def children(self):
        return tuple(p for p in (self.norm_in, self.mixer, self.feed_forward) if p is not None)

    def tensor_decls(self):
        if not self.layer_scale:
            return []
        names = ("scale1",) if self.feed_forward is None else ("scale1", "scale2")
        return [TensorDecl(self._name(n), (self.hidden_size,), init="norm") for n in names]

    def load(self, fetch):
        if self.layer_scale:
            self.scale1 = fetch.vector_f32(self._name("scale1"))
            if self.feed_forward is not None:
                self.scale2 = fetch.vector_f32(self._name("scale2"))
        else:
            import torch

            self.scale1 = self.scale2 = fetch.constant(torch.ones(self.hidden_size, dtype=torch.float32))

    def step_cost(self, spans, rows, elem_bytes):
        cost = super().step_cost(spans, rows, elem_bytes)
        cost.flop = 0.0  # vectors, not matrices that multiply tokens
        return cost

    def forward(self, ctx, residual, delta, cache):
        x = self.norm_in.forward(ctx, residual, delta)
        parts = [(self.mixer.forward(ctx, x, cache), self.scale1)]
        if self.feed_forward is not None:
            parts.append((self.feed_forward.forward(ctx, x), self.scale2))
        return residual, ScaledUpdate(parts)
