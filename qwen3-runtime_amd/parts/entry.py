"""Parts that work on the residual stream between two layers.

``origin_mix``: the stream is replaced by a product of itself joined with the embedding's
output, ``x <- W [x; x0]`` with ``W`` ``[width, 2 width]`` (the stream's columns first): how a pass
over a looped span of layers begins. What the layer before left pending is added first
(``x + scale * delta``), in float32; the product's result is the new float32 stream.
"""

from __future__ import annotations

from ..registry import register_part
from .base import Entry
from .plan import TensorDecl


@register_part("entry", "origin_mix")
class OriginMix(Entry):
    def __init__(self, hidden_size: int, delta_scale: float = 1.0, tensors=None):
        super().__init__(tensors)
        self.hidden_size = int(hidden_size)
        self.delta_scale = float(delta_scale)
        self.weight = None

    def tensor_decls(self):
        return [TensorDecl(self._name("weight"), (self.hidden_size, 2 * self.hidden_size))]

    def load(self, fetch):
        self.weight = fetch.matrix(self._name("weight"))

    def forward(self, ctx, residual, delta, origin):
        joined = ctx.ops.add_concat(residual, delta, self.delta_scale, origin, ctx.dtype)
        return ctx.ops.linear(joined, self.weight, out_f32=True), None
