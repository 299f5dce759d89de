"""Mixers side by side: several mixers read the same input, and the layer's mixer output is the
mean of their outputs, each RMS-normed over the model width first (``x / sqrt(mean x^2 + eps) * w``
with a plain weight per branch). Every branch keeps its own caches; together they are the
mixer's, in the branches' order.
"""

from __future__ import annotations

from ..registry import part_class, register_part
from .base import Mixer
from .plan import PartSpec, TensorDecl


@register_part("mixer", "side_by_side")
class SideBySide(Mixer):
    """``branches``: the mixers' ``PartSpec``s (two of them). ``tensors``: ``out0``, ``out1``: the
    weights of the norms on the branches' outputs."""

    def __init__(self, hidden_size: int, eps: float, branches, tensors=None):
        super().__init__(tensors)
        self.hidden_size = int(hidden_size)
        self.eps = float(eps)
        if len(branches) != 2:
            raise ValueError(f"two mixers stand side by side, not {len(branches)}")
        self.branches = [part_class("mixer", b.kind)(**b.args, tensors=b.tensors) for b in branches]
        self.out_weights = None

    def children(self):
        return tuple(self.branches)

    def cache_specs(self):
        return tuple(spec for b in self.branches for spec in b.cache_specs())

    def tensor_decls(self):
        return [TensorDecl(self._name(f"out{i}"), (self.hidden_size,), init="norm") for i in range(len(self.branches))]

    def load(self, fetch):
        self.out_weights = [fetch.vector_f32(self._name(f"out{i}")) for i in range(len(self.branches))]

    def step_cost(self, spans, rows, elem_bytes):
        cost = super().step_cost(spans, rows, elem_bytes)
        cost.flop = 0.0
        return cost

    def forward(self, ctx, x, cache):
        outs, at = [], 0
        views = cache if isinstance(cache, tuple) else (cache,)
        for b in self.branches:
            n = len(b.cache_specs())
            own = views[at: at + n]
            at += n
            outs.append(b.forward(ctx, x, None if n == 0 else own[0] if n == 1 else tuple(own)))
        return ctx.ops.norm_mean(outs[0], self.out_weights[0], outs[1], self.out_weights[1], self.eps)
