"""Gated delta rule: a recurrent mixer with a matrix-valued state per head.

From the mixer's input ``h``: queries and keys ``kv_heads x dim`` and values ``heads x vdim``
by projections without bias (head ``j`` reads query/key head ``j // (heads / kv_heads)``), each
passed through a short causal convolution over time per channel (``taps`` taps, the last one on
the current token, zeros before the sequence's start) and silu; queries and keys are then scaled
to unit vectors per head (``x / sqrt(sum x^2 + 1e-6)``), queries also by ``dim^(-1/2)``. A step
size ``beta = sigmoid(b h)`` per head, and a decay ``g = exp(-exp(A_log) softplus(a h + dt_bias))``,
one number per head, or (``decay="channel"``) one per head and key channel from a low-rank pair
``a2 (a1 h)``. Per head and token, in this order::

    S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q

so the read-out sees the token's own write. Each head's ``o`` is divided by its root mean square
over ``vdim``, multiplied by one weight vector shared by the heads and by a gate of ``h``
(``gate="silu"``: ``silu(g h)``; ``gate="sigmoid_low_rank"``: ``sigmoid(g2 (g1 h))``), then projected
out. ``S`` starts at zero and is float32; it and the convolutions' last ``taps - 1`` inputs are
the request's state, kept in its slot from step to step. Everything that enters the recurrence
besides the projections and convolutions is float32.

All projections of ``h`` are one fused product; the low-rank pairs' second factors follow as
products of their own, in float32 where they feed the decay.
"""

from __future__ import annotations

from ..registry import register_part
from .base import Mixer, StepCost
from .plan import CacheSpec, TensorDecl

UNIT_EPS = 1e-6


@register_part("mixer", "gated_delta")
class GatedDeltaRule(Mixer):
    """``tensors``: ``q``, ``k``, ``v`` (their convolutions under the same file names with
    ``.conv`` added), ``b``, ``A_log``, ``dt_bias``, ``norm``, ``o``; with ``decay="head"`` ``a``, with
    ``"channel"`` ``a1`` and ``a2``; with ``gate="silu"`` ``g``, with ``"sigmoid_low_rank"`` ``g1``, ``g2``."""

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                 taps: int, norm_eps: float, decay: str = "head", gate: str = "silu",
                 decay_rank: int | None = None, gate_rank: int | None = None, tensors=None):
        super().__init__(tensors)
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads do not divide into {num_kv_heads} query/key heads")
        if decay not in ("head", "channel") or gate not in ("silu", "sigmoid_low_rank"):
            raise ValueError(f"unknown decay {decay!r} (head, channel) or gate {gate!r} (silu, sigmoid_low_rank)")
        if not 1 <= int(taps) <= 16:
            raise ValueError(f"the convolution has 1 to 16 taps, not {taps}")
        if not 1 <= int(head_dim) <= 512:
            raise ValueError(f"the state's rows are held in registers: key size 1 to 512, not {head_dim}")
        self.hidden_size = int(hidden_size)
        self.heads, self.kv_heads = int(num_heads), int(num_kv_heads)
        self.dim, self.vdim = int(head_dim), int(value_dim)
        self.taps = int(taps)
        self.norm_eps = float(norm_eps)
        self.decay, self.gate = decay, gate
        self.proj = self.conv = self.a2 = self.g2 = self.o = None
        self.a_log = self.dt_bias = self.norm = None
        # inner sizes of the low-rank pairs; None: whatever the model file's tensors have
        self.decay_rank = None if decay_rank is None else int(decay_rank)
        self.gate_rank = None if gate_rank is None else int(gate_rank)
        self.columns: dict[str, tuple[int, int]] = {}

    # ---- sizes ---------------------------------------------------------------
    @property
    def channels(self) -> int:
        """Convolved channels: queries, keys, values."""
        return 2 * self.kv_heads * self.dim + self.heads * self.vdim

    def cache_specs(self):
        # the state transposed, [heads, vdim, dim]: a value channel's column of S is contiguous
        return (CacheSpec("state", shape=(self.heads, self.vdim, self.dim), dtype="float32"),
                CacheSpec("state", shape=(self.channels, max(self.taps - 1, 1)), dtype="float32"))

    def _head_rows(self) -> list[tuple[str, int]]:
        """Projections of the mixer's input, in the order of the fused product's columns."""
        rows = [("q", self.kv_heads * self.dim), ("k", self.kv_heads * self.dim), ("v", self.heads * self.vdim),
                ("b", self.heads)]
        # a size of -1 in a declaration stands for "as the file has it"
        rows.append(("a", self.heads) if self.decay == "head" else ("a1", self.decay_rank or -1))
        rows.append(("g", self.heads * self.vdim) if self.gate == "silu" else ("g1", self.gate_rank or -1))
        return rows

    def tensor_decls(self):
        h = self.hidden_size
        decls = [TensorDecl(self._name(n), (rows, h)) for n, rows in self._head_rows()]
        for n, rows in self._head_rows()[:3]:
            decls.append(TensorDecl(self._name(n) + ".conv", (rows, self.taps)))
        per = self.heads if self.decay == "head" else self.heads * self.dim
        decls += [TensorDecl(self._name("A_log"), (self.heads,), init="log_rate"),
                  TensorDecl(self._name("dt_bias"), (per,)),
                  TensorDecl(self._name("norm"), (self.vdim,), init="norm"),
                  TensorDecl(self._name("o"), (h, self.heads * self.vdim))]
        if self.decay == "channel":
            decls.append(TensorDecl(self._name("a2"), (self.heads * self.dim, self.decay_rank or -1)))
        if self.gate == "sigmoid_low_rank":
            decls.append(TensorDecl(self._name("g2"), (self.heads * self.vdim, self.gate_rank or -1)))
        return decls

    def load(self, fetch):
        import torch

        if self.decay == "channel":
            self.a2 = fetch.matrix(self._name("a2"))
            self.decay_rank = int(self.a2.shape[1])
        if self.gate == "sigmoid_low_rank":
            self.g2 = fetch.matrix(self._name("g2"))
            self.gate_rank = int(self.g2.shape[1])
        rows = self._head_rows()
        self.proj = fetch.fused([self._name(n) for n, _ in rows], dim=0)
        self.columns, at = {}, 0
        for n, r in rows:
            self.columns[n] = (at, r)
            at += r
        if at != self.proj.shape[0]:
            raise ValueError(f"{self._name('q')}: the low-rank pairs' two factors do not fit each other "
                             f"({self.proj.shape[0]} rows in all, {at} expected)")
        self.conv = fetch.constant(torch.cat([fetch.vector_f32(self._name(n) + ".conv") for n, _ in rows[:3]], dim=0))
        self.second = None
        if self.a2 is not None and self.g2 is not None:
            # both low-rank pairs: their second factors as one block-diagonal matrix, so that one
            # product (float32 out) of the neighbouring columns a1 | g1 serves decay and gate. The
            # zeros add nothing to either sum.
            ra, rg = self.decay_rank, self.gate_rank
            both = torch.zeros((self.a2.shape[0] + self.g2.shape[0], ra + rg), dtype=self.a2.dtype, device=self.a2.device)
            both[: self.a2.shape[0], :ra] = self.a2
            both[self.a2.shape[0]:, ra:] = self.g2
            self.second = fetch.constant(both)
        self.a_log = fetch.vector_f32(self._name("A_log"))
        self.dt_bias = fetch.vector_f32(self._name("dt_bias"))
        self.norm = fetch.vector_f32(self._name("norm"))
        self.o = fetch.matrix(self._name("o"))

    def step_cost(self, spans, rows, elem_bytes):
        cost = super().step_cost(spans, rows, elem_bytes)
        tokens = sum(q for q, _ in spans)
        # per token and head: decay, two sums over the state's rows, one write: 4 passes over D x Dv
        cost.flop += 2.0 * 4 * tokens * self.heads * self.dim * self.vdim
        return cost

    def forward(self, ctx, x, cache):
        ops = ctx.ops
        state, tail = cache
        y = ops.linear(x, self.proj)
        cols = self.columns
        qkv = ops.delta_conv(ctx, y, self.channels, self.conv, tail.state,
                             ((self.kv_heads, self.dim, 2), (self.kv_heads, self.dim, 1), (self.heads, self.vdim, 0)),
                             UNIT_EPS)
        beta = y[:, cols["b"][0]: cols["b"][0] + self.heads]  # columns of the product, where they lie
        def columns(name):
            first, width = cols[name]
            return y[:, first: first + width]

        if self.second is not None:  # decay logits and gate from one product, float32 out
            low = y[:, cols["a1"][0]: cols["g1"][0] + cols["g1"][1]].contiguous()
            both = ops.linear(low, self.second, out_f32=True)
            a, gate = both[:, : self.heads * self.dim], both[:, self.heads * self.dim:]
        else:
            # the decay's logits stay float32 from the second factor on
            a = columns("a") if self.decay == "head" else ops.linear(columns("a1").contiguous(), self.a2, out_f32=True)
            gate = columns("g") if self.gate == "silu" else ops.linear(columns("g1").contiguous(), self.g2)
        o = ops.delta_rule(ctx, qkv, beta, a, self.a_log, self.dt_bias, state.state, self.heads, self.kv_heads,
                           self.dim, self.vdim, self.decay == "channel")
        out = ops.delta_out(o, self.norm, gate, self.norm_eps, "silu" if self.gate == "silu" else "sigmoid", ctx.dtype)
        return ops.linear_for_residual(out, self.o)
