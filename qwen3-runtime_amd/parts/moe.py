"""Routed mixture of SwiGLU experts.

A router scores every token against ``num_experts`` experts in float32 (``z = W_r h + b_r``);
the token takes the ``top`` experts with the largest logits, weighted by the softmax over
those logits alone, and the output is the weighted sum of the chosen experts' outputs, each
``down_e( silu(gate_e(x)) * up_e(x) )``. Experts have no biases. On the device all experts'
matrices lie in two tensors, ``[E, 2I, H]`` (gate rows, then up rows) and ``[E, H, I]``, so that
one launch serves every (token, chosen expert) pair.
"""

from __future__ import annotations

from ..registry import register_part
from .base import FeedForward, StepCost
from .plan import TensorDecl


@register_part("feed_forward", "moe_swiglu")
class RoutedSwiGLU(FeedForward):
    """``tensors``: ``router``, ``router_bias`` (with ``router_bias=True``), and ``gate``, ``up``,
    ``down`` as patterns in which ``{e}`` stands for the expert's number."""

    def __init__(self, hidden_size: int, intermediate_size: int, num_experts: int, top: int,
                 router_bias: bool = True, tensors=None):
        super().__init__(tensors)
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.num_experts = int(num_experts)
        self.top = int(top)
        if not 1 <= self.top <= self.num_experts:
            raise ValueError(f"each token takes {self.top} of {self.num_experts} experts")
        self.has_router_bias = bool(router_bias)
        self.router = self.router_bias = self.gate_up = self.down = None

    def _expert(self, logical: str, e: int) -> str:
        return self._name(logical).format(e=e)

    def tensor_decls(self):
        h, i = self.hidden_size, self.intermediate_size
        decls = [TensorDecl(self._name("router"), (self.num_experts, h))]
        if self.has_router_bias:
            decls.append(TensorDecl(self._name("router_bias"), (self.num_experts,)))
        for e in range(self.num_experts):
            decls += [TensorDecl(self._expert("gate", e), (i, h)), TensorDecl(self._expert("up", e), (i, h)),
                      TensorDecl(self._expert("down", e), (h, i))]
        return decls

    def load(self, fetch):
        h, i, n = self.hidden_size, self.intermediate_size, self.num_experts
        # the router stays in float32 in every mode
        self.router = fetch.vector_f32(self._name("router"))
        if self.has_router_bias:
            self.router_bias = fetch.vector_f32(self._name("router_bias"))
        names = [self._expert(part, e) for e in range(n) for part in ("gate", "up")]
        self.gate_up = fetch.fused(names, dim=0).view(n, 2 * i, h)
        self.down = fetch.fused([self._expert("down", e) for e in range(n)], dim=0).view(n, h, i)

    def step_cost(self, spans, rows, elem_bytes):
        # only the experts that some token chose are read, and each token multiplies `top` of them
        tokens = sum(q for q, _ in spans)
        h, i, n = self.hidden_size, self.intermediate_size, self.num_experts
        used = min(n, tokens * self.top)
        cost = StepCost()
        cost.weight_bytes[self._name("router")] = n * h * 4
        for e in range(used):  # which ones is not known here: the first `used` stand for them
            for part, size in (("gate", i * h), ("up", i * h), ("down", h * i)):
                cost.weight_bytes[self._expert(part, e)] = size * elem_bytes
        cost.flop = 2.0 * tokens * (n * h + self.top * 3 * h * i)
        return cost

    def forward(self, ctx, x):
        index, weight = ctx.ops.route_top(x, self.router, self.router_bias, self.top)
        return ctx.ops.moe_swiglu(x, self.gate_up, self.down, index, weight)
