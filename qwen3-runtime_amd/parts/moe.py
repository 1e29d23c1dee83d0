"""Routed mixture of gated experts.

A router scores every token against ``num_experts`` experts in float32 (``z = W_r h + b_r``);
the token takes the ``top`` experts with the largest logits, weighted by the softmax over
those logits alone, and the output is the weighted sum of the chosen experts' outputs, each
``down_e( silu(gate_e(x)) * up_e(x) )``. Experts have no biases. On the device all experts'
matrices lie in two tensors, ``[E, 2I, H]`` (gate rows, then up rows) and ``[E, H, I]``, so that
one launch serves every (token, chosen expert) pair.

Options beyond that form. ``scoring="sigmoid"``: scores ``s = sigmoid(z)``; the ``top`` largest are
chosen and weigh the experts' outputs as they are, not renormalised. ``scoring="softmax_all"``: scores
``s = softmax(z)`` over all experts; the ``top`` largest are chosen and weigh the outputs as they are.
``groups`` and ``keep``: the experts form ``groups`` equal groups of neighbours, a group's score is the
sum of its two largest scores (``group_score="top2"``) or its largest score (``"max"``), and only
experts of the ``keep`` best groups can be chosen. ``activation="clamped"`` with
``limit``: ``g = min(gate x, limit)``, ``u = clamp(up x, -limit, limit)``, ``y = g sigmoid(1.702 g) (u + 1)``
in place of ``silu(g) u``. ``shared_size``: one more expert of that inner width (tensors
``shared_gate``, ``shared_up``, ``shared_down``; ``shared_limit`` its clamp) that every token passes
and whose output is added unweighted. ``correction`` (with ``softmax_all`` or ``sigmoid`` scores): a
tensor ``correction`` [experts] is added to the scores for the choice alone; the weights are the
chosen experts' scores without it. ``renormalise``: the chosen scores are divided by their sum
(plus 1e-20). ``weight_scale``: the weights are multiplied by it at the end.
``activation="relu2"``: experts without a gate, ``down_e( relu(up_e(x))^2 )``, tensors ``up`` and ``down``.
"""

from __future__ import annotations

from ..registry import register_part
from .base import FeedForward, StepCost
from .plan import TensorDecl


@register_part("feed_forward", "routed_experts")
@register_part("feed_forward", "moe_swiglu")
class RoutedSwiGLU(FeedForward):
    """``tensors``: ``router``, ``router_bias`` (with ``router_bias=True``), and ``gate``, ``up``,
    ``down`` as patterns in which ``{e}`` stands for the expert's number."""

    def __init__(self, hidden_size: int, intermediate_size: int, num_experts: int, top: int,
                 router_bias: bool = True, scoring: str = "softmax_top", groups: int = 1, keep: int | None = None,
                 activation: str = "swiglu", limit: float = 0.0, shared_size: int | None = None,
                 shared_limit: float | None = None, group_score: str = "top2", correction: bool = False,
                 renormalise: bool = False, weight_scale: float = 1.0, tensors=None):
        super().__init__(tensors)
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.num_experts = int(num_experts)
        self.top = int(top)
        if not 1 <= self.top <= self.num_experts:
            raise ValueError(f"each token takes {self.top} of {self.num_experts} experts")
        self.has_router_bias = bool(router_bias)
        if scoring not in ("softmax_top", "sigmoid", "softmax_all") or activation not in ("swiglu", "clamped", "relu2") \
                or group_score not in ("top2", "max"):
            raise ValueError(f"unknown scoring {scoring!r} (softmax_top, sigmoid, softmax_all), activation {activation!r} "
                             f"(swiglu, clamped, relu2) or group score {group_score!r} (top2, max)")
        self.scoring, self.activation, self.limit = scoring, activation, float(limit)
        self.group_score = group_score
        self.gated = activation != "relu2"
        self.has_correction, self.renormalise, self.weight_scale = bool(correction), bool(renormalise), float(weight_scale)
        if (self.has_correction or self.renormalise) and scoring == "softmax_top":
            raise ValueError("a correction of the choice and renormalised weights go with scores over all experts")
        if not self.gated and shared_size:
            raise NotImplementedError("a shared expert beside experts without a gate")
        self.groups = int(groups)
        self.keep = self.groups if keep is None else int(keep)
        if self.groups < 1 or self.num_experts % self.groups or not 1 <= self.keep <= self.groups:
            raise ValueError(f"{self.num_experts} experts in {self.groups} groups of which {self.keep} stay")
        if self.keep * (self.num_experts // self.groups) < self.top:
            raise ValueError(f"{self.keep} groups of {self.num_experts // self.groups} experts hold fewer than the {self.top} chosen")
        self.shared_size = None if shared_size is None else int(shared_size)
        self.shared_limit = self.limit if shared_limit is None else float(shared_limit)
        self.router = self.router_bias = self.gate_up = self.down = None
        self.shared_gate_up = self.shared_down = self.correction = None

    def _expert(self, logical: str, e: int) -> str:
        return self._name(logical).format(e=e)

    def tensor_decls(self):
        h, i = self.hidden_size, self.intermediate_size
        decls = [TensorDecl(self._name("router"), (self.num_experts, h))]
        if self.has_router_bias:
            decls.append(TensorDecl(self._name("router_bias"), (self.num_experts,)))
        for e in range(self.num_experts):
            decls += ([TensorDecl(self._expert("gate", e), (i, h))] if self.gated else []) + \
                     [TensorDecl(self._expert("up", e), (i, h)), TensorDecl(self._expert("down", e), (h, i))]
        if self.has_correction:
            decls.append(TensorDecl(self._name("correction"), (self.num_experts,)))
        if self.shared_size:
            s = self.shared_size
            decls += [TensorDecl(self._name("shared_gate"), (s, h)), TensorDecl(self._name("shared_up"), (s, h)),
                      TensorDecl(self._name("shared_down"), (h, s))]
        return decls

    def load(self, fetch):
        h, i, n = self.hidden_size, self.intermediate_size, self.num_experts
        # the router stays in float32 in every mode
        self.router = fetch.vector_f32(self._name("router"))
        if self.has_router_bias:
            self.router_bias = fetch.vector_f32(self._name("router_bias"))
        if self.has_correction:
            self.correction = fetch.vector_f32(self._name("correction"))
        halves = ("gate", "up") if self.gated else ("up",)  # without a gate the tensor holds the up rows alone
        names = [self._expert(part, e) for e in range(n) for part in halves]
        self.gate_up = fetch.fused(names, dim=0).view(n, len(halves) * i, h)
        self.down = fetch.fused([self._expert("down", e) for e in range(n)], dim=0).view(n, h, i)
        if self.shared_size:
            self.shared_gate_up = fetch.fused([self._name("shared_gate"), self._name("shared_up")], dim=0)
            self.shared_down = fetch.matrix(self._name("shared_down"))

    def step_cost(self, spans, rows, elem_bytes):
        # only the experts that some token chose are read, and each token multiplies `top` of them
        tokens = sum(q for q, _ in spans)
        h, i, n = self.hidden_size, self.intermediate_size, self.num_experts
        used = min(n, tokens * self.top)
        cost = StepCost()
        cost.weight_bytes[self._name("router")] = n * h * 4
        for e in range(used):  # which ones is not known here: the first `used` stand for them
            for part, size in (("gate", i * h), ("up", i * h), ("down", h * i))[0 if self.gated else 1:]:
                cost.weight_bytes[self._expert(part, e)] = size * elem_bytes
        cost.flop = 2.0 * tokens * (n * h + self.top * (3 if self.gated else 2) * h * i)
        if self.shared_size:
            for part in ("shared_gate", "shared_up", "shared_down"):
                cost.weight_bytes[self._name(part)] = self.shared_size * h * elem_bytes
            cost.flop += 2.0 * tokens * 3 * h * self.shared_size
        return cost

    def forward(self, ctx, x):
        ops = ctx.ops
        plain = self.scoring == "softmax_top" and self.groups == 1 and self.activation == "swiglu"
        if plain:
            index, weight = ops.route_top(x, self.router, self.router_bias, self.top)
            return ops.moe_swiglu(x, self.gate_up, self.down, index, weight)
        how = {"group_score": self.group_score} if self.group_score != "top2" else {}
        if self.has_correction or self.renormalise or self.weight_scale != 1.0:
            how.update(correction=self.correction, renormalise=self.renormalise, weight_scale=self.weight_scale)
        index, weight = ops.route_top(x, self.router, self.router_bias, self.top, scoring=self.scoring,
                                      groups=self.groups, keep=self.keep, **how)
        more = {"activation": self.activation, "limit": self.limit}
        if not self.shared_size:
            return ops.moe_swiglu(x, self.gate_up, self.down, index, weight, **more)
        act = ops.gated_linear(x, self.shared_gate_up, activation=self.activation, limit=self.shared_limit)
        # few tokens: the shared expert's product leaves float32 planes with one to spare, the routed
        # experts write theirs into it, and the norm that comes next adds them all up
        planes = ops.linear_planes_with_spare(act, self.shared_down)
        if planes is not None:
            ops.moe_swiglu(x, self.gate_up, self.down, index, weight, out=planes[-1], **more)
            return planes
        out = ops.moe_swiglu(x, self.gate_up, self.down, index, weight, **more)
        return ops.accumulate(out, ops.linear_for_residual(act, self.shared_down))
