"""Rotary position encodings: NeoX pairing, and interleaved pairs over part of a head.

``inv_j = theta^(-2j/D)``, angle ``pos * inv_j``; the head vector is split
into its first and second half ``x1 | x2`` and rotated pairwise:
``y1 = x1 cos - x2 sin``, ``y2 = x2 cos + x1 sin``
(reference: qwen3_runtime/layers/rope.py:7-21). Angles, sine and cosine are
float32. The same angles serve every head; values are not rotated.

``rope_pairs``: only the first ``dims`` elements of a head turn, element ``2i`` paired with
``2i + 1`` (the interleaved layout): ``(u, v) -> (u cos a - v sin a, v cos a + u sin a)`` with
``a = pos * f_i``, ``f_i = base^(-2i/dims)``; the rest of the head passes unchanged. The
frequencies may be scaled by wavelength ``l = 2 pi / f`` (``scaling``: ``factor``, ``low``, ``high``,
``original``): kept where ``l < original / high``, divided by ``factor`` where ``l > original / low``,
and between the two blended, ``(1 - s) f / factor + s f`` with
``s = (original / l - low) / (high - low)``. The encoding works on the q | k | v product where
it lies (``in_place``), together with the projections' biases.
"""

from __future__ import annotations

import math

import torch

from ..registry import register_part
from .base import PositionEncoding


@register_part("position", "rope_neox")
class RotaryNeox(PositionEncoding):
    fused_form = "neox_full"

    def __init__(self, head_dim: int, theta: float, tensors=None):
        super().__init__(tensors)
        if head_dim % 2:
            raise ValueError(f"rotary encoding needs an even head size, got {head_dim}")
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        # float32 throughout, as the table of the reference is built
        # (reference: qwen3_runtime/layers/rope.py:18)
        self.inv_freq_cpu = 1.0 / (
            self.theta ** (torch.arange(0, self.head_dim, 2, dtype=torch.float32) / self.head_dim)
        )
        self.inv_freq = None
        # layers whose encodings have equal keys rotate by equal angles and share a step's table
        self.angles_key = ("rope_neox", self.head_dim, self.theta)

    def load(self, fetch):
        self.inv_freq = fetch.constant(self.inv_freq_cpu)

    def rotate(self, ctx, q, k):
        """Unfused form: rotate already-normed q ``[T, nq, D]`` and k ``[T, nkv, D]``."""
        return ctx.ops.rope_neox(q, k, ctx.positions, self.inv_freq)


@register_part("position", "rope_pairs")
class RotaryPairs(PositionEncoding):
    # the attention mixer hands this encoding the fused product (and its biases) to work on where
    # it lies, then stores and attends as for a mixer without encoding
    in_place = True

    def __init__(self, head_dim: int, dims: int, base: float, scaling=None, tensors=None):
        super().__init__(tensors)
        if dims % 2 or not 0 <= dims <= head_dim or head_dim % 2:
            raise ValueError(f"{dims} rotated elements in heads of {head_dim}: both even, the first no larger")
        self.head_dim, self.dims, self.base = int(head_dim), int(dims), float(base)
        self.scaling = None if scaling is None else {k: float(scaling[k]) for k in ("factor", "low", "high", "original")}
        # the table in float64, then rounded once: angles are float32 products of position and frequency
        i = torch.arange(self.dims // 2, dtype=torch.float64)
        f = self.base ** (-2.0 * i / max(self.dims, 1))
        if self.scaling is not None:
            sc = self.scaling
            wavelength = 2.0 * math.pi / f
            s = (sc["original"] / wavelength - sc["low"]) / (sc["high"] - sc["low"])
            blended = (1.0 - s) * f / sc["factor"] + s * f
            f = torch.where(wavelength < sc["original"] / sc["high"], f,
                            torch.where(wavelength > sc["original"] / sc["low"], f / sc["factor"], blended))
        self.freq_cpu = f.to(torch.float32)
        self.freq = None

    def load(self, fetch):
        self.freq = fetch.constant(self.freq_cpu)

    def rotate_in_place(self, ctx, qkv, num_rotated_heads: int, bias=None):
        """Add ``bias`` to every column of ``qkv`` and turn the first ``num_rotated_heads`` heads."""
        ctx.ops.bias_rotate_pairs(qkv, bias, ctx.positions, self.freq if self.dims else None,
                                  num_rotated_heads, self.head_dim)
