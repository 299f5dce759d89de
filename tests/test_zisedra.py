"""Zisedra: every mechanism alone against its plain function, and whole models under every cutting.

Each test runs with the plain torch ops on the CPU (which pins the host side: plan, packing,
pages, windows, state slots, the loop) and with the HIP ops on the GPU (marked ``gpu``; float32
and bfloat16). The oracle is ``plain/zisedra_plain.py``: whole sequences, no cache, no state
carried, float64. Configurations are made here and differ from each other in every size and
option, also in values that a model may happen to make equal or 1.
"""

from __future__ import annotations

import math
from types import SimpleNamespace

import pytest
import torch

import traces
from plain import zisedra_plain as P
from plain.ops_ref import TorchOps

GPU = pytest.mark.gpu
BACKENDS = [pytest.param(("cpu", "float32"), id="host-f32"),
            pytest.param(("cuda:0", "float32"), id="gpu-f32", marks=GPU),
            pytest.param(("cuda:0", "bfloat16"), id="gpu-bf16", marks=GPU)]
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def make_ops(device):
    if device == "cpu":
        return TorchOps()
    from qwen3_runtime_amd.ops.hip import HipOps

    return HipOps()


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def tol(dtype):
    return dict(atol=3e-5, rtol=3e-5) if dtype == "float32" else dict(atol=4e-2, rtol=4e-2)


def spans_ctx(ops, device, dtype, q_lens, starts, slots):
    """A step's context for sequences that bring ``q_lens`` tokens after ``starts`` earlier ones."""
    from qwen3_runtime_amd.parts.base import StepContext

    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)  # noqa: E731
    cu = [0]
    for n in q_lens:
        cu.append(cu[-1] + n)
    kv = [s + n for s, n in zip(starts, q_lens)]
    return StepContext(ops=ops, dtype=dtype, device=torch.device(device), num_tokens=cu[-1], num_seqs=len(q_lens),
                       positions=i32([s + i for s, n in zip(starts, q_lens) for i in range(n)]), cu_q=i32(cu),
                       kv_lens=i32(kv), seq_of_token=i32([j for j, n in enumerate(q_lens) for _ in range(n)]),
                       state_slots=i32(slots), first_span=i32([int(s == 0) for s in starts]), q_lens_host=list(q_lens),
                       kv_lens_host=kv, max_q_len=max(q_lens), max_kv_len=max(kv))


def in_steps(total, sizes):
    """Cut ``total`` tokens into portions of the given sizes, repeated."""
    out, p, i = [], 0, 0
    while p < total:
        n = min(sizes[i % len(sizes)], total - p)
        out.append((p, n))
        p += n
        i += 1
    return out


# ------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("taps,segments", [(4, ((2, 16, 2), (2, 16, 1), (4, 24, 0))), (2, ((1, 40, 2), (1, 40, 1), (3, 8, 0))),
                                           (5, ((3, 72, 2), (3, 72, 1), (3, 130, 0))), (1, ((2, 32, 2), (2, 32, 1), (2, 32, 0)))])
@pytest.mark.parametrize("sizes", [(150,), (1,), (2, 1, 3, 1, 1, 17), (7, 2), (64, 3, 70)])
def test_convolution_silu_and_unit_vectors_carry_their_tail(backend, taps, segments, sizes):
    """Two sequences of unequal lengths in slots 2 and 0 of 3, fed in portions down to one token: the
    convolution of a portion's first tokens reads the inputs the portion before left in the slot.
    Steps of 64 tokens and more take the kernel that walks eight tokens a wave, where a sequence
    may begin in the middle of a wave's tokens."""
    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    c = sum(h * w for h, w, _ in segments)
    lengths, slots = ([150, 90], [2, 0]) if len(sizes) != 6 else ([50, 23], [2, 0])
    x = [rnd(n, c + 6, seed=3 + i).to(dt) for i, n in enumerate(lengths)]  # columns of a wider matrix
    w = rnd(c, taps, seed=9, scale=0.6)
    tail = torch.zeros(3, c, max(taps - 1, 1), dtype=torch.float32, device=device)
    tail[1] = float("nan")  # a slot nobody holds
    got = [torch.zeros(n, c) for n in lengths]
    steps = [in_steps(n, sizes) for n in lengths]
    for r in range(max(len(s) for s in steps)):
        live = [i for i in range(2) if r < len(steps[i])]
        ctx = spans_ctx(ops, device, dt, [steps[i][r][1] for i in live], [steps[i][r][0] for i in live], [slots[i] for i in live])
        y = torch.cat([x[i][steps[i][r][0]: steps[i][r][0] + steps[i][r][1]] for i in live]).to(device)
        out = ops.delta_conv(ctx, y, c, w.to(device), tail, segments, 1e-6).cpu()
        at = 0
        for i in live:
            p, n = steps[i][r]
            got[i][p: p + n] = out[at: at + n]
            at += n
    for i, n in enumerate(lengths):
        conv = P.causal_conv_silu(x[i][:, :c].double(), w.double())
        first, parts = 0, []
        for heads, width, mode in segments:
            seg = conv[:, first: first + heads * width].view(n, heads, width)
            if mode:
                seg = P.unit_vector(seg) * (width ** -0.5 if mode == 2 else 1.0)
            parts.append(seg.reshape(n, -1))
            first += heads * width
        torch.testing.assert_close(got[i].double(), torch.cat(parts, 1), atol=2e-5, rtol=2e-5)


def rule_inputs(t, heads, kv_heads, d, dv, per_channel, seed, slow=False):
    q = P.unit_vector(rnd(t, kv_heads, d, seed=seed)) * d ** -0.5
    k = P.unit_vector(rnd(t, kv_heads, d, seed=seed + 1))
    v = rnd(t, heads, dv, seed=seed + 2)
    beta = rnd(t, heads, seed=seed + 3, scale=2.0)
    a = rnd(t, heads * d if per_channel else heads, seed=seed + 4, scale=2.0)
    a_log = rnd(heads, seed=seed + 5) - (6.0 if slow else 1.0)
    dt_bias = rnd(heads * d if per_channel else heads, seed=seed + 6)
    return q, k, v, beta, a, a_log, dt_bias


def plain_rule(q, k, v, beta, a, a_log, dt_bias, per_channel):
    t, heads, dv = v.shape
    kv_heads, d = k.shape[1], k.shape[2]
    q, k, v, beta, a, a_log, dt_bias = (x.double() for x in (q, k, v, beta, a, a_log, dt_bias))
    sp = P.softplus(a + dt_bias)
    decay = torch.exp(-torch.exp(a_log)[None, :, None] * sp.view(t, heads, d)) if per_channel else \
        torch.exp(-torch.exp(a_log)[None, :] * sp)
    b = torch.sigmoid(beta)
    g = heads // kv_heads
    return torch.stack([P.delta_rule(q[:, h // g], k[:, h // g], v[:, h], b[:, h], decay[:, h]) for h in range(heads)], 1)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("heads,kv_heads,d,dv", [(4, 2, 32, 48), (8, 4, 64, 32), (3, 1, 40, 20), (2, 2, 128, 128), (1, 1, 16, 8),
                                                 (2, 1, 72, 17), (2, 2, 256, 16), (5, 5, 1, 1), (1, 1, 320, 24), (2, 1, 512, 8)])
@pytest.mark.parametrize("per_channel", [False, True])
@pytest.mark.parametrize("sizes", [(300,), (37, 2, 1, 1, 16, 5)])
def test_delta_rule_against_the_recurrence_written_out(backend, heads, kv_heads, d, dv, per_channel, sizes):
    """Random inputs, float32 everywhere; the state is carried from portion to portion in a slot.
    The step sizes and decay logits come as columns of wider matrices, as the mixer hands them."""
    device, dtype = backend
    ops = make_ops(device)
    t = 70 if device == "cpu" else 300
    q, k, v, beta, a, a_log, dt_bias = rule_inputs(t, heads, kv_heads, d, dv, per_channel, seed=d + dv)
    dt = DT[dtype]
    beta, a = beta.to(dt), (a if per_channel else a.to(dt))  # the decay's low-rank product stays float32
    want = plain_rule(q, k, v, beta, a, a_log, dt_bias, per_channel)
    state = torch.full((4, heads, dv, d), float("nan"), device=device)
    state[3] = 0.0
    qkv = torch.cat([q.reshape(t, -1), k.reshape(t, -1), v.reshape(t, -1)], 1).float()
    wide_b, wide_a = torch.cat([rnd(t, 3).to(dt), beta], 1).to(device), torch.cat([rnd(t, 5).to(a.dtype), a], 1).to(device)
    got = torch.zeros(t, heads, dv)
    for p, n in in_steps(t, sizes):
        ctx = spans_ctx(ops, device, dt, [n], [p], [3])
        got[p: p + n] = ops.delta_rule(ctx, qkv[p: p + n].contiguous().to(device), wide_b[p: p + n, 3:], wide_a[p: p + n, 5:],
                                       a_log.to(device), dt_bias.to(device), state, heads, kv_heads, d, dv, per_channel).cpu()
    torch.testing.assert_close(got.double(), want, atol=3e-5, rtol=3e-4)
    assert torch.isnan(state[:3]).all()  # other slots are left alone


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("per_channel", [False, True])
def test_a_write_far_back_is_read_and_a_slot_taken_again_starts_empty(backend, per_channel):
    """Slow decays; one token far back writes a marker value under a key that a query hundreds of
    tokens later asks for, across many portions and beside a second sequence. Then the slot is
    zeroed as when it is taken again, and the same query reads nothing."""
    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    heads, kv_heads, d, dv, t = 2, 1, 32, 16, 420
    q, k, v, beta, a, a_log, dt_bias = rule_inputs(t, heads, kv_heads, d, dv, per_channel, seed=1, slow=True)
    direction = P.unit_vector(rnd(d, seed=77))
    k = k - (k @ direction)[..., None] * direction  # nobody else writes under the marker's key
    k = P.unit_vector(k)
    k[5, 0], v[5], beta[5] = direction, 9.0, 30.0   # step size 1: the marker is stored whole
    q[:] = 0.0
    q[-1, 0] = direction
    want = plain_rule(q, k, v, beta, a, a_log, dt_bias, per_channel)[-1]
    assert want.abs().min() > 3.0  # the marker survives the decays
    state = torch.zeros(2, heads, dv, d, device=device)
    qkv = torch.cat([q.reshape(t, -1), k.reshape(t, -1), v.reshape(t, -1)], 1).float()
    other = rule_inputs(t, heads, kv_heads, d, dv, per_channel, seed=50)
    qkv2 = torch.cat([x.reshape(t, -1) for x in other[:3]], 1).float()
    for p, n in in_steps(t, (64, 3, 1, 100, 2)):
        ctx = spans_ctx(ops, device, dt, [n, n], [p, p], [1, 0])
        rows = torch.cat([qkv[p: p + n], qkv2[p: p + n]]).to(device)
        got = ops.delta_rule(ctx, rows, torch.cat([beta[p: p + n], other[3][p: p + n]]).to(device),
                             torch.cat([a[p: p + n], other[4][p: p + n]]).to(device), a_log.to(device), dt_bias.to(device),
                             state, heads, kv_heads, d, dv, per_channel).cpu()
    torch.testing.assert_close(got[n - 1].double(), want, atol=1e-4, rtol=1e-3)
    state[1].zero_()
    ctx = spans_ctx(ops, device, dt, [1], [0], [1])
    again = ops.delta_rule(ctx, qkv[-1:].to(device), beta[-1:].to(device), a[-1:].to(device), a_log.to(device),
                           dt_bias.to(device), state, heads, kv_heads, d, dv, per_channel).cpu()
    assert again.abs().max() < 1.0


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("heads,dv,kind", [(4, 64, "silu"), (3, 20, "sigmoid"), (1, 1, "silu"), (2, 130, "sigmoid")])
def test_read_out_norm_and_gate(backend, heads, dv, kind):
    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    o, w = rnd(9, heads, dv, seed=1), 1 + rnd(dv, seed=2, scale=0.2)
    gate = rnd(9, heads * dv + 4, seed=3).to(dt)
    got = ops.delta_out(o.to(device), w.to(device), gate.to(device)[:, 4:], 1e-5, kind, dt).double().cpu()
    z = gate[:, 4:].double().view(9, heads, dv)
    want = P.rms_norm(o.double(), w.double(), 1e-5) * (z * torch.sigmoid(z) if kind == "silu" else torch.sigmoid(z))
    torch.testing.assert_close(got, want.reshape(9, -1), **tol(dtype))


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("heads,kv_heads,d,dims,scaling", [(4, 1, 64, 24, (6.0, 1.0, 4.0, 512.0)), (3, 3, 16, 16, None),
                                                           (2, 1, 48, 12, (4.0, 1.0, 3.0, 64.0)), (2, 2, 32, 0, None),
                                                           (5, 1, 8, 2, (2.0, 0.5, 2.0, 16.0))])
def test_pair_rotation_biases_and_scaled_frequencies(backend, heads, kv_heads, d, dims, scaling):
    """The encoding part on a q | k | v product where it lies, with the projections' biases, at
    positions up to thousands; frequencies from all three regions of the scaling."""
    from qwen3_runtime_amd.parts.rope import RotaryPairs

    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    rot = {"dims": dims, "base": 10000.0 if scaling is None else 2e5}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    part = RotaryPairs(d, dims, rot["base"], rot.get("scaling"))
    part.freq = part.freq_cpu.to(device)
    freqs = P.scaled_frequencies(rot, torch.float64)
    if scaling and dims >= 12:
        wl = 2 * math.pi / (rot["base"] ** (-2.0 * torch.arange(dims // 2, dtype=torch.float64) / dims))
        assert (wl < scaling[3] / scaling[2]).any() and (wl > scaling[3] / scaling[1]).any()
    t, dv = 6, 24
    width = (heads + kv_heads) * d + kv_heads * dv
    x, bias = rnd(t, width, seed=1).to(dt), rnd(width, seed=2)
    positions = [0, 1, 71, 500, 1021, 3000]
    ctx = SimpleNamespace(ops=ops, positions=torch.tensor(positions, dtype=torch.int32, device=device))
    y = x.clone().to(device)
    part.rotate_in_place(ctx, y, heads + kv_heads, bias.to(device))
    full = x.double() + bias.double()
    qk = P.rotate_interleaved(full[:, : (heads + kv_heads) * d].view(t, heads + kv_heads, d), torch.tensor(positions), freqs)
    want = torch.cat([qk.reshape(t, -1), full[:, (heads + kv_heads) * d:]], 1)
    # an angle of thousands of radians held in float32 is good to some 1e-4 rad
    torch.testing.assert_close(y.double().cpu(), want, **(dict(atol=2e-3, rtol=1e-3) if dtype == "float32" else dict(atol=5e-2, rtol=3e-2)))


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("experts,top,groups,keep,width", [(18, 2, 3, 1, 200), (12, 3, 3, 2, 96), (6, 2, 1, 1, 64), (8, 4, 8, 4, 50),
                                                           (64, 6, 8, 3, 128), (4, 4, 2, 2, 31)])
def test_router_sigmoid_scores_and_groups(backend, experts, top, groups, keep, width):
    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    x, router = rnd(40, width, seed=1).to(dt), rnd(experts, width, seed=2, scale=0.2)
    index, weight = ops.route_top(x.to(device), router.to(device), None, top, scoring="sigmoid", groups=groups, keep=keep)
    want_i, want_w = P.route(x.double(), router.double(), top, groups, keep)
    assert torch.equal(index.cpu().long().sort(1).values, want_i.sort(1).values)
    torch.testing.assert_close(weight.cpu().double().sort(1).values, want_w.sort(1).values, atol=1e-5, rtol=1e-5)


def test_groups_keep_a_strong_expert_out():
    """The best expert of all lies in a group whose two best together lose: it is not chosen."""
    router = torch.zeros(6, 4)
    router[0, 0], router[3, 0], router[4, 0], router[5, 0] = 5.0, 2.0, 2.0, -9.0   # group 0: 5, 0, 0; group 1: 2, 2, -9
    x = torch.tensor([[1.0, 0, 0, 0]])
    router[1:3, 0] = -9.0
    index, _ = TorchOps().route_top(x, router, None, 2, scoring="sigmoid", groups=2, keep=1)
    want, _ = P.route(x.double(), router.double(), 2, 2, 1)
    assert sorted(index[0].tolist()) == sorted(want[0].tolist()) == [3, 4]


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("experts,top,width,inner,tokens,limit", [(6, 2, 64, 48, 9, 0.8), (16, 2, 256, 96, 3, 1.0), (4, 4, 96, 40, 70, 1.5),
                                                                  (5, 1, 128, 16, 300, 0.5)])
def test_clamped_experts_weighted_by_their_scores(backend, experts, top, width, inner, tokens, limit):
    """Inputs large enough that the clamps hold on both sides; few pairs, several pairs an expert,
    and steps long enough for the expert-by-expert forms."""
    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    x = rnd(tokens, width, seed=1).to(dt)
    gate, up, down = (rnd(experts, inner, width, seed=2, scale=0.15).to(dt), rnd(experts, inner, width, seed=3, scale=0.15).to(dt),
                      rnd(experts, width, inner, seed=4, scale=0.15).to(dt))
    g = torch.Generator().manual_seed(5)
    index = torch.stack([torch.randperm(experts, generator=g)[:top] for _ in range(tokens)]).to(torch.int32)
    weight = torch.rand(tokens, top, generator=g)
    got = ops.moe_swiglu(x.to(device), torch.cat([gate, up], 1).to(device), down.to(device), index.to(device), weight.to(device),
                         activation="clamped", limit=limit).double().cpu()
    want = torch.zeros(tokens, width, dtype=torch.float64)
    pre = x.double() @ gate[0].double().T
    assert (pre > limit).any() and (x.double() @ up[0].double().T < -limit).any()
    for t in range(tokens):
        for j in range(top):
            e = int(index[t, j])
            want[t] += weight[t, j].double() * P.expert(x[t].double(), gate[e].double(), up[e].double(), down[e].double(), limit)
    torch.testing.assert_close(got, want, **(tol(dtype) if dtype == "float32" else dict(atol=6e-2, rtol=6e-2)))


class DictFetch:
    """Hands a part its tensors from a dict, placed as the loader would place them."""

    def __init__(self, tensors, device, dtype):
        self.t, self.device, self.dtype = tensors, device, dtype

    def matrix(self, name):
        return self.t[name].to(self.dtype).to(self.device).contiguous()

    def fused(self, names, dim=0):
        return torch.cat([self.t[n] for n in names], dim=dim).to(self.dtype).to(self.device).contiguous()

    def vector_f32(self, name):
        return self.t[name].float().to(self.device)

    def constant(self, tensor):
        return tensor.to(self.device).contiguous()


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("width,inner,shared,experts,top,groups,keep", [(128, 64, 128, 8, 2, 2, 1), (384, 64, 128, 16, 2, 4, 2),
                                                                        (96, 48, 80, 12, 12, 3, 3), (256, 128, 256, 4, 1, 1, 1)])
def test_mixture_with_shared_expert_at_every_step_size(backend, width, inner, shared, experts, top, groups, keep):
    """The feed-forward part, routed and shared experts summed, over steps of 1 to 300 tokens: every
    form of the experts' and of the shared expert's products (few rows, rows in planes with the
    routed sum as one more plane, the library's)."""
    from qwen3_runtime_amd.parts.moe import RoutedSwiGLU

    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    names = {"router": "r", "gate": "e{e}.gate", "up": "e{e}.up", "down": "e{e}.down",
             "shared_gate": "shared.gate", "shared_up": "shared.up", "shared_down": "shared.down"}
    w = {"r": rnd(experts, width, seed=1, scale=0.3), "shared.gate": rnd(shared, width, seed=2, scale=0.15),
         "shared.up": rnd(shared, width, seed=3, scale=0.15), "shared.down": rnd(width, shared, seed=4, scale=0.15)}
    for e in range(experts):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = (rnd(inner, width, seed=10 + e, scale=0.15), rnd(inner, width, seed=40 + e, scale=0.15),
                                                            rnd(width, inner, seed=70 + e, scale=0.15))
    w = {n: x.to(dt).float() for n, x in w.items()}
    part = RoutedSwiGLU(width, inner, experts, top, router_bias=False, scoring="sigmoid", groups=groups, keep=keep,
                        activation="clamped", limit=0.9, shared_size=shared, shared_limit=1.1, tensors=names)
    part.load(DictFetch(w, device, dt))
    mlp = {"router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}, "expert": {"limit": 0.9},
           "shared": {"limit": 1.1}}
    for tokens in (1, 8, 17, 70, 100, 300):
        x = rnd(tokens, width, seed=tokens).to(dt)
        ctx = SimpleNamespace(ops=ops, dtype=dt)
        got = part.forward(ctx, x.to(device))
        got = (got.sum(0) if got.dim() == 3 else got).double().cpu()
        want = P.mixture(x.double(), {n: t.double() for n, t in w.items()} | {"router": w["r"].double()}, mlp)
        if dtype == "float32":
            torch.testing.assert_close(got, want, atol=3e-5, rtol=3e-5)
        else:  # a token whose choice falls the other way in bfloat16 is another token; all others are close
            close = ((got - want).abs() <= 6e-2 + 6e-2 * want.abs()).all(dim=1)
            assert int((~close).sum()) <= max(1, tokens // 10), (tokens, int((~close).sum()))


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("width,tokens,planes", [(96, 5, 1), (352, 3, 4), (2560, 2, 1), (50, 7, 2)])
def test_scaled_sum_mean_of_norms_and_the_entry_of_a_pass(backend, width, tokens, planes):
    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    res, origin = rnd(tokens, width, seed=1), rnd(tokens, width, seed=2)
    delta = rnd(planes, tokens, width, seed=3) if planes > 1 else rnd(tokens, width, seed=3).to(dt)
    total = delta.double().sum(0) if planes > 1 else delta.double()
    w1, w2 = 1 + rnd(width, seed=4, scale=0.2), 1 + rnd(width, seed=5, scale=0.2)
    # x + m * delta, then the norm
    r = res.clone().to(device)
    got = ops.add_rmsnorm(r, delta.to(device), w1.to(device), 1e-5, dt, delta_scale=0.3)
    x = res.double() + 0.3 * total
    torch.testing.assert_close(r.double().cpu(), x, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(got.double().cpu(), P.rms_norm(x, w1.double(), 1e-5), **tol(dtype))
    # half the sum of two normed outputs, one of them in planes
    other = rnd(tokens, width, seed=6, scale=3.0).to(dt)
    got = ops.norm_mean(other.to(device), w1.to(device), delta.to(device), w2.to(device), 1e-5)
    want = 0.5 * (P.rms_norm(other.double(), w1.double(), 1e-5) + P.rms_norm(total, w2.double(), 1e-5))
    torch.testing.assert_close(got.double().cpu(), want, atol=1e-5, rtol=1e-5)
    # the stream with what is pending, joined with the embedding
    got = ops.add_concat(res.to(device), delta.to(device), 0.3, origin.to(device), dt)
    torch.testing.assert_close(got.double().cpu(), torch.cat([x, origin.double()], 1), **(dict(atol=1e-5, rtol=1e-5) if dtype == "float32" else dict(atol=3e-2, rtol=1e-2)))
    acc = res.clone().to(device)
    torch.testing.assert_close(ops.accumulate(acc, delta.to(device)).double().cpu(), res.double() + total, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("heads,kv_heads,d,dv,window,page,dims", [(4, 2, 64, 64, 70, 16, 48), (2, 2, 32, 16, 9, 8, 32), (6, 2, 16, 16, 21, 16, 4),
                                                                  (2, 1, 128, 128, 130, 16, 64), (3, 3, 48, 48, 1, 8, 0)])
def test_window_attention_mixer_sees_a_key_inside_the_window_only(backend, heads, kv_heads, d, dv, window, page, dims):
    """The attention mixer itself (biased projections, pair rotation, window) over a paged cache whose
    early pages go back to the pool as the window passes: against the plain mixer on the whole
    sequence. One token's input is scaled up so that its key and value dominate wherever it is
    seen; queries just inside and just outside the window of it, in a prompt portion and decoded
    one by one, would differ grossly if the edge were one off."""
    from qwen3_runtime_amd.cache import CacheManager
    from qwen3_runtime_amd.parts.attention import GroupedQueryAttention
    from qwen3_runtime_amd.parts.plan import PartSpec

    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    width, t = 40, 3 * window + 37
    sizes = {"heads": heads, "kv_heads": kv_heads, "dim": d, "vdim": dv, "scale": 0.9 / math.sqrt(d), "mask": {"size": window},
             "rot": {"dims": dims, "base": 300.0, "scaling": {"factor": 4.0, "low": 1.0, "high": 3.0, "original": 40.0}}}
    w = {"q": rnd(heads * d, width, seed=1, scale=0.3), "k": rnd(kv_heads * d, width, seed=2, scale=0.3),
         "v": rnd(kv_heads * dv, width, seed=3, scale=0.3), "o": rnd(width, heads * dv, seed=4, scale=0.3),
         "q.b": rnd(heads * d, seed=5, scale=0.3), "k.b": rnd(kv_heads * d, seed=6, scale=0.3), "v.b": rnd(kv_heads * dv, seed=7, scale=0.3)}
    w = {n: x.to(dt).float() for n, x in w.items()}
    h = rnd(t, width, seed=8).to(dt)
    marked = t - window - 20
    h[marked] *= 6.0
    want = P.window_attention(h.double(), {n: x.double() for n, x in w.items()}, sizes)
    mixer = GroupedQueryAttention(width, heads, kv_heads, d, value_dim=dv, scale=sizes["scale"], window=window, bias=True,
                                  position=PartSpec("rope_pairs", {"head_dim": d, "dims": dims, "base": 300.0,
                                                                   "scaling": sizes["rot"]["scaling"]}))
    mixer.qkv = torch.cat([w["q"], w["k"], w["v"]]).to(dt).to(device)
    mixer.o = w["o"].to(dt).to(device)
    mixer.bias = torch.cat([w["q.b"], w["k.b"], w["v.b"]]).to(device)
    mixer.position.freq = mixer.position.freq_cpu.to(device)
    pages = -(-(window + 64) // page) + 2
    cache = CacheManager([mixer.cache_spec()], page_size=page, num_pages=pages, max_requests=2, device=device, dtype=dt)
    for g in cache.groups:
        for store in g.storage:
            store.fill_(float("nan"))
    cache.admit("a")
    got = torch.zeros(t, width)
    edge = marked + window
    cuts = in_steps(edge - 3, (64, 5)) + [(p, 1) for p in range(edge - 3, edge + 4)] + [(edge + 4, t - edge - 4)]
    from qwen3_runtime_amd.parts.base import GroupView

    for p, n in cuts:
        cache.reserve("a", n)
        ctx = spans_ctx(ops, device, dt, [n], [p], [0])
        table = torch.full((1, cache.table_width(["a"])), -1, dtype=torch.int32)
        cache.fill_tables(0, ["a"], table.numpy())
        slots = torch.from_numpy(cache.token_slots(0, "a", p, n))
        ctx.groups = [GroupView(page, window, table.to(device), slots.to(device))]
        out = mixer.forward(ctx, h[p: p + n].to(device), cache.view(0, ctx.groups))
        got[p: p + n] = (out.sum(0) if out.dim() == 3 else out).float().cpu()
        cache.commit("a", n)
    cache.release("a")
    inside, outside = marked + window - 1, marked + window
    # bfloat16: the marked token makes outputs of up to a hundred; queries, keys and probabilities
    # rounded to 8 bits move them by about a hundredth of that
    bound = dict(atol=2e-4, rtol=2e-4) if dtype == "float32" else dict(atol=0.015 * float(want.abs().max()), rtol=0.05)
    assert (want[inside] - want[outside]).abs().max() > max(0.5, 10 * bound["atol"])  # the edge shows
    torch.testing.assert_close(got.double(), want, **bound)


# ------------------------------------------------------------------ whole models
def moe(ff, limit, experts, top, groups, keep, shared=None):
    raw = {"kind": "moe", "expert": {"ff": ff, "limit": limit},
           "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}
    if shared:
        raw["shared"] = {"ff": shared[0], "limit": shared[1]}
    return raw


def delta(heads, kv_heads, dim, vdim, conv, ranks=None):
    raw = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}
    if ranks:
        raw.update(decay_rank=ranks[0], gate_rank=ranks[1])
    return raw


def window(heads, kv_heads, dim, vdim, scale, size, dims, base, scaling=None):
    rot = {"dims": dims, "base": base}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": size}, "rot": rot}


def config_a():
    """A looped span that begins with a parallel layer, entered three times; unequal sizes everywhere."""
    return {"architecture": "Zisedra", "vocab": 300, "width": 96, "norm": {"eps": 1e-5}, "residual_mult": 0.7,
            "loop": {"start": 1, "stop": 3, "times": 3},
            "layers": [
                {"type": "delta", "mixer": delta(6, 3, 16, 24, 3), "mlp": moe(48, 1.5, 12, 3, 3, 2, (80, 2.0))},
                {"type": "parallel", "mixer": {"left": window(6, 2, 32, 32, 0.2, 21, 12, 5000.0, (4.0, 1.0, 3.0, 64.0)),
                                               "right": delta(3, 3, 48, 20, 2, (8, 12))},
                 "mlp": moe(32, 0.8, 6, 2, 1, 1)},
                {"type": "delta", "mixer": delta(2, 1, 40, 40, 5), "mlp": None},
                {"type": "parallel", "mixer": {"left": window(4, 4, 16, 16, 0.25, 40, 16, 100.0),
                                               "right": delta(4, 2, 16, 16, 4, (4, 4))},
                 "mlp": moe(24, 1.0, 4, 4, 2, 2, (16, 0.5))}]}, 16


def config_b():
    """No loop, no scaling of the stream, values of another size than keys, a window of one page."""
    return {"architecture": "Zisedra", "vocab": 200, "width": 64, "norm": {"eps": 1e-6}, "residual_mult": 1.0,
            "layers": [
                {"type": "parallel", "mixer": {"left": window(4, 1, 32, 16, 0.3, 8, 32, 50.0),
                                               "right": delta(2, 2, 72, 8, 4, (6, 3))}, "mlp": moe(40, 1.2, 8, 2, 4, 2)},
                {"type": "delta", "mixer": delta(4, 4, 32, 32, 4), "mlp": moe(16, 2.0, 3, 1, 1, 1, (48, 1.0))}]}, 8


def config_c():
    """The whole model is one looped span; head size 64 (decoding through the one-kernel attention)."""
    return {"architecture": "Zisedra", "vocab": 150, "width": 128, "norm": {"eps": 1e-5}, "residual_mult": 0.6,
            "loop": {"start": 0, "stop": 2, "times": 2},
            "layers": [
                {"type": "parallel", "mixer": {"left": window(2, 1, 64, 64, 0.11, 50, 48, 100000.0, (8.0, 1.0, 4.0, 2048.0)),
                                               "right": delta(2, 1, 128, 64, 4, (16, 16))}, "mlp": moe(64, 1.0, 4, 2, 2, 1, (64, 1.0))},
                {"type": "delta", "mixer": delta(1, 1, 64, 128, 2), "mlp": None}]}, 16


def every_expert(make):
    """The same model with a router that has no choice to make (every expert of every group is taken,
    weighted by its score): for runs in bfloat16, where a choice between two experts whose scores
    lie within rounding of each other may fall the other way, which moves that position's logits by
    a large part of their spread, and later positions' through the recurrent state. The choice
    itself is held to the plain one in float32 here, and in both types in the router's own test."""
    def made():
        raw, page = make()
        for layer in raw["layers"]:
            if layer["mlp"]:
                router = layer["mlp"]["router"]
                router["top"], router["groups"]["keep"] = router["experts"], router["groups"]["count"]
        return raw, page
    return made


def config_d():
    """Odd sizes: a vocabulary of 123, width 88, heads of 24 (no multiple of 16), three query heads on one
    key head, a rotation of the whole head, one layer looped four times and entered each time, a
    parallel layer without feed-forward, groups of one expert, a stream scaled up, one tap."""
    return {"architecture": "Zisedra", "vocab": 123, "width": 88, "norm": {"eps": 1e-5}, "residual_mult": 1.3,
            "loop": {"start": 1, "stop": 2, "times": 4},
            "layers": [
                {"type": "parallel", "mixer": {"left": window(3, 1, 24, 40, 0.2, 17, 24, 1000.0, (2.0, 1.0, 2.0, 32.0)),
                                               "right": delta(2, 1, 24, 12, 2, (5, 7))}, "mlp": None},
                {"type": "delta", "mixer": delta(3, 3, 8, 56, 1), "mlp": moe(20, 0.7, 5, 2, 5, 3, (8, 0.9))},
                {"type": "parallel", "mixer": {"left": window(2, 2, 16, 16, 0.3, 64, 2, 7.0),
                                               "right": delta(1, 1, 100, 36, 3, (1, 2))}, "mlp": moe(12, 1.0, 2, 1, 2, 1)}]}, 8


def config_e():
    """Delta rules only: a model without a single page of cache; a loop that runs once."""
    return {"architecture": "Zisedra", "vocab": 90, "width": 48, "norm": {"eps": 1e-5},
            "loop": {"start": 0, "stop": 2, "times": 1},
            "layers": [{"type": "delta", "mixer": delta(2, 1, 16, 16, 4), "mlp": None},
                       {"type": "delta", "mixer": delta(3, 3, 8, 24, 2), "mlp": moe(16, 1.0, 4, 1, 2, 1)}]}, 16


def config_f():
    """Sizes that are multiples of nothing: width 90, values of 7 and 5 elements, keys of 10, 6 and 3,
    experts of 9 and 5, a shared expert of 11."""
    return {"architecture": "Zisedra", "vocab": 77, "width": 90, "norm": {"eps": 1e-5}, "residual_mult": 0.9,
            "loop": {"start": 0, "stop": 1, "times": 2},
            "layers": [{"type": "parallel", "mixer": {"left": window(3, 1, 10, 7, 0.3, 13, 6, 50.0), "right": delta(2, 1, 6, 5, 3, (3, 2))},
                        "mlp": moe(9, 1.0, 3, 2, 1, 1, (11, 1.0))},
                       {"type": "delta", "mixer": delta(5, 5, 3, 9, 2), "mlp": moe(5, 0.5, 2, 1, 2, 1)}]}, 8


def config_g():
    """Layers of a real model's proportions (heads of 128, a window of 256, experts of 512): the kernel
    forms that small sizes never reach."""
    return {"architecture": "Zisedra", "vocab": 500, "width": 1024, "norm": {"eps": 1e-5}, "residual_mult": 0.8,
            "layers": [{"type": "delta", "mixer": delta(8, 2, 128, 128, 4), "mlp": moe(512, 2.0, 8, 2, 4, 2, (512, 2.0))},
                       {"type": "parallel", "mixer": {"left": window(8, 2, 128, 128, 0.09, 256, 64, 10000.0),
                                                      "right": delta(8, 2, 128, 128, 4, (32, 32))},
                        "mlp": moe(512, 2.0, 8, 2, 4, 2, (512, 2.0))}]}, 16


CONFIGS = {"a": config_a, "b": config_b, "c": config_c, "d": config_d, "e": config_e, "f": config_f, "g": config_g}
CONFIGS.update({name + "_every": every_expert(make) for name, make in list(CONFIGS.items())})
# bfloat16: the bound on the largest error of a position's logits, in units of their deviation. The
# error has a long tail: over six seeds of "c" its median per position was 0.02 and the largest
# 0.13 to 0.46, at scattered positions; "a" (eight layer runs of width 96, a gain above one at
# every entry of its loop) measured 0.37, "b" 0.11. float32 showed no error in any of them.
NOISE = {"a": 0.6, "b": 0.3, "c": 0.6, "d": 0.6, "e": 0.3, "f": 0.6, "g": 0.3}
LENGTHS = {"a": [1, 7, 45, 130], "b": [3, 17, 50, 64, 101], "c": [2, 16, 17, 120], "d": [1, 5, 40, 83], "e": [1, 9, 40, 70], "f": [1, 9, 40, 70]}
_folders: dict = {}


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    from qwen3_runtime_amd.weights import write_model_folder

    def get(name, dtype="float32"):
        if dtype == "bfloat16":
            name += "_every"
        if name not in _folders:
            raw, _ = CONFIGS[name]()
            _folders[name] = write_model_folder(tmp_path_factory.mktemp("zisedra_" + name), raw, seed=71 + len(_folders),
                                                std=0.03 if name.startswith("g") else 0.08, norm_jitter=0.2)
        return _folders[name]

    return get


def load(folder, page, pages, backend, max_seqs=4, hip_graph=False):
    from qwen3_runtime_amd.config.engine import EngineConfig
    from qwen3_runtime_amd.engine.factory import load as load_model

    device, dtype = backend
    cfg = EngineConfig(page_size=page, num_pages=pages, max_num_seqs=max_seqs, dtype=dtype, device=device,
                       hip_graph=hip_graph)
    return load_model(folder, cfg, ops=TorchOps() if device == "cpu" else None)


def plain_logits(folder, requests):
    cfg, w = P.load(folder)
    out = {}
    for rid, toks in requests.items():
        logits = P.forward(cfg, w, toks).float()
        for p in range(len(toks)):
            out[(rid, p)] = logits[p]
    return out


def check(got, want, dtype, noise=0.2):
    """float32: to rounding of float32 sums, everywhere. bfloat16: as noise relative to the logits'
    own spread, no position over ``noise`` and their root mean square under a quarter of it; a wrong
    window, state or portion shows in float32, where the bound is rounding."""
    if dtype == "float32":
        traces.compare(got, want, atol=2e-4, rtol=2e-4)
        return
    keys = sorted(want)
    assert set(got) == set(want)
    w = torch.stack([want[k].double() for k in keys])
    err = torch.stack([got[k].double() for k in keys]) - w
    std = float(w.std())
    per_pos = err.abs().amax(dim=1)
    good = per_pos < noise * std
    assert bool(good.all()), \
        f"{int((~good).sum())} of {len(keys)} positions over the bound, the first {keys[int((~good).nonzero()[0])]}"
    rms = float(err.pow(2).mean().sqrt())
    assert rms < 0.25 * noise * std, f"rms error {rms:.4f} against a logit deviation of {std:.3f}"


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["a", "b", "c", "d", "e", "f"])
@pytest.mark.parametrize("cut", ["whole", "tail_one_by_one", "portions", "mixed"])
def test_cuttings_match_plain(folder, backend, name, cut):
    """Whole prompts; the last tokens one by one (across window edges); portions down to two tokens;
    up to four live requests mixed in a pool of the peak's size, so that pages and slots are used
    again (freed pages are poisoned first; a slot is zeroed when it is taken)."""
    raw, page = CONFIGS[name]()
    reqs = traces.make_requests(raw["vocab"], LENGTHS[name] + ([30, 9] if cut == "mixed" else []), seed=5)
    steps = getattr(traces, cut)(reqs)
    loaded = load(folder(name, backend[1]), page, traces.peak_tokens(steps, unit=page) // page, backend)
    got = traces.replay(loaded, steps, poison_freed=True)
    check(got, plain_logits(folder(name, backend[1]), reqs), backend[1], NOISE[name])
    assert (len(loaded.cache.groups) == 0) == (name == "e")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_of_a_real_model_s_proportions(folder, dtype):
    """A 330-token prompt in one step, then in portions with its last tokens one by one, beside a
    second request: prompt kernels with full tiles, the window passing, experts by expert."""
    raw, page = config_g()
    reqs = traces.make_requests(raw["vocab"], [330, 40], seed=9)
    want = plain_logits(folder("g", dtype), reqs)
    for steps in (traces.whole(reqs), traces.mixed(reqs, seed=2, decode_tail=12)):
        loaded = load(folder("g", dtype), page, traces.peak_tokens(steps, unit=page) // page, ("cuda:0", dtype))
        check(traces.replay(loaded, steps, poison_freed=True), want, dtype, NOISE["g"])


@pytest.mark.parametrize("backend", BACKENDS)
def test_long_decoding_in_a_pool_of_one_window(folder, backend):
    """A request far longer than the pool, decoded token by token: the windowed caches give their
    early pages back, the recurrent state has no pages, so a few pages serve 300 positions."""
    raw, page = config_b()
    reqs = traces.make_requests(raw["vocab"], [300], seed=8)
    steps = traces.tail_one_by_one(reqs, tail=290)
    loaded = load(folder("b", backend[1]), page, 4, backend)
    got = traces.replay(loaded, steps, poison_freed=True)
    check(got, plain_logits(folder("b", backend[1]), reqs), backend[1], NOISE["b"])


@pytest.mark.parametrize("backend", BACKENDS)
def test_batch_mates_do_not_change_a_request(folder, backend):
    """Unequal requests in one batch against each alone: the same logits within rounding."""
    raw, page = config_a()
    reqs = traces.make_requests(raw["vocab"], [9, 60, 121, 33], seed=2)
    together = [{"step": 0, "entries": [{"id": r, "tokens": t, "want": list(range(len(t)))} for r, t in reqs.items()],
                 "end": list(reqs)}]
    loaded = load(folder("a", backend[1]), page, 32, backend)
    both = traces.replay(loaded, together)
    alone = traces.replay(loaded, traces.whole(reqs))
    if backend[1] == "float32":
        traces.compare(both, alone, atol=2e-5, rtol=2e-5)
    else:
        check(both, alone, "bfloat16", NOISE["a"])


@pytest.mark.parametrize("backend", BACKENDS)
def test_a_restarted_request_computes_the_same_again(folder, backend):
    """Preemption by recompute: pages back, state and tails zeroed, the slot kept; the second pass
    over the same tokens gives the first one's logits."""
    from qwen3_runtime_amd.engine.batch import StepEntry

    raw, page = config_c()
    toks = traces.make_requests(raw["vocab"], [70], seed=3)["r0"]
    loaded = load(folder("c"), page, 16, backend)
    loaded.cache.admit("x")
    first = loaded.runner.step([StepEntry("x", toks[:50], [49])]).float().cpu()
    loaded.runner.step([StepEntry("x", toks[50:], [0])])
    loaded.cache.restart("x")
    again = loaded.runner.step([StepEntry("x", toks[:50], [49])]).float().cpu()
    loaded.cache.release("x")
    torch.testing.assert_close(again, first, atol=1e-6 if backend[1] == "float32" else 1e-2, rtol=0)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,graphs", [("float32", False), ("bfloat16", True), ("bfloat16", False)])
@pytest.mark.parametrize("name", ["a", "c", "e"])
def test_greedy_generation_through_the_entry_point(folder, name, dtype, graphs):
    """``LLM.generate`` (scheduler with a small token budget, sampler, graphs where they apply): the
    tokens chosen greedily are, by the plain model given the same context, the best ones or within
    rounding of the best. Requests of unequal lengths, more of them than fit at once."""
    from qwen3_runtime_amd.llm import LLM

    raw, page = CONFIGS[name]()
    llm = LLM(str(folder(name, dtype)), dtype=dtype, block_size=page, num_kv_blocks=64, max_num_seqs=3,
              max_num_batched_tokens=48, cuda_graph=graphs)
    prompts = list(traces.make_requests(raw["vocab"], [5, 61, 20, 90], seed=4).values())
    outs = llm.generate(prompts, max_tokens=40)
    cfg, w = P.load(folder(name, dtype))
    for prompt, tokens in zip(prompts, outs):
        assert len(tokens) == 40
        logits = P.forward(cfg, w, list(prompt) + list(tokens))[len(prompt) - 1: -1]
        below = logits.max(-1).values - logits[range(40), list(tokens)]
        bound = 1e-3 if dtype == "float32" else 2 * NOISE[name] * float(logits.std())
        assert int((below >= bound).sum()) == 0, (float(below.max()), int(below.argmax()))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_command_line_and_trace_replay(folder, tmp_path, dtype):
    """As a user runs them: ``python -m qwen3_runtime_amd.cli --model DIR`` generates greedily, and
    ``bin/trace_run`` replays a mixed schedule of seven requests from standard input, four live at
    most, with a pool that only holds what is live and state slots for four."""
    import ast
    import json
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np

    root = Path(__file__).resolve().parents[1]
    raw, page = config_c()
    where = folder("c", dtype)
    cfg, w = P.load(where)
    prompt = [5, 17, 3, 140, 9, 77, 2]
    proc = subprocess.run([sys.executable, "-m", "qwen3_runtime_amd.cli", "--model", str(where), "--dtype", dtype,
                           "--prompt-tokens", *map(str, prompt), "--max-tokens", "8"],
                          capture_output=True, text=True, timeout=600, cwd=str(root))
    assert proc.returncode == 0, proc.stderr[-3000:]
    lines = dict(line.split(" ", 1) for line in proc.stdout.splitlines() if " " in line)
    tokens = ast.literal_eval(lines["runtime"])
    assert len(tokens) == 8
    logits = P.forward(cfg, w, prompt + tokens)[len(prompt) - 1: -1]
    below = logits.max(-1).values - logits[range(8), tokens]
    assert float(below.max()) < (1e-3 if dtype == "float32" else 2 * NOISE["c"] * float(logits.std()))

    reqs = traces.make_requests(raw["vocab"], [70, 9, 41, 100, 35, 1, 66], seed=6)
    steps = traces.mixed(reqs, seed=1)
    out = tmp_path / "logits"
    proc = subprocess.run([str(root / "bin" / "trace_run"), "--model", str(where), "--dtype", dtype, "--out", str(out),
                           "--max-tokens", str(traces.peak_tokens(steps))],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True,
                          timeout=600, cwd=str(root))
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert [line for line in proc.stdout.splitlines() if line.startswith("done ")] == [f"done {s['step']}" for s in steps]
    got, pos = {}, {r: 0 for r in reqs}
    for s in steps:
        wanted = sum(len(e["want"]) for e in s["entries"])
        rows = np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(wanted, raw["vocab"]) if wanted else None
        i = 0
        for e in s["entries"]:
            for k in e["want"]:
                got[(e["id"], pos[e["id"]] + k)] = torch.from_numpy(rows[i].copy())
                i += 1
            pos[e["id"]] += len(e["tokens"])
    check(got, plain_logits(where, reqs), dtype, NOISE["c"])


# ------------------------------------------------------------------ configuration and plan
def test_config_reader_and_plan():
    from qwen3_runtime_amd.config.model import ConfigError
    from qwen3_runtime_amd.config.zisedra import ZisedraConfig
    from qwen3_runtime_amd.engine.factory import build_model

    raw, _ = config_a()
    cfg = ZisedraConfig.from_dict(raw)
    assert ZisedraConfig.from_dict(cfg.to_dict()) == cfg
    assert [i for i, _ in cfg.run_order()] == [0, 1, 2, 1, 2, 1, 2, 3]
    assert [e for _, e in cfg.run_order()] == [False, True, False, True, False, True, False, False]
    _, model = build_model(raw)
    # every run of a layer has caches of its own: pages of keys for an attention, two states a delta rule
    assert [len(s.cache_ids()) for s in model.plan.order] == [2, 3, 2, 3, 2, 3, 2, 3]
    assert len({c for s in model.plan.order for c in s.cache_ids()}) == len(model.plan.caches) == 20
    assert [s.entry for s in model.plan.order] == [None, 0, None, 0, None, 0, None, None]
    names = {d.file_name for d in model.tensor_decls()}
    assert {"loop.in", "l1.mix.left.q.b", "l1.mix.right.a2", "l1.mix.right.out", "l0.mlp.shared.up", "l0.mix.q.conv"} <= names
    assert "l2.norm2" not in names and "l2.norm2" in model.plan.ignorable
    for key, value in (("residual_mult", "x"), ("loop", {"start": 2, "stop": 1, "times": 1})):
        with pytest.raises((ConfigError, ValueError, TypeError)):
            ZisedraConfig.from_dict({**raw, key: value})
    bad = {**raw, "layers": [{"type": "attention", "mixer": {}, "mlp": None}]}
    with pytest.raises(ConfigError):
        ZisedraConfig.from_dict(bad)


def test_low_rank_sizes_come_from_the_file(folder, tmp_path):
    """A configuration as a model file carries it names no inner size of the low-rank pairs: the
    tensors' shapes give them."""
    import json
    import shutil

    src = folder("b")
    shutil.copy(src / "model.safetensors", tmp_path / "model.safetensors")
    raw = json.loads((src / "config.json").read_text())
    for layer in raw["layers"]:
        if layer["type"] == "parallel":
            del layer["mixer"]["right"]["decay_rank"], layer["mixer"]["right"]["gate_rank"]
    (tmp_path / "config.json").write_text(json.dumps(raw))
    reqs = traces.make_requests(raw["vocab"], [12], seed=1)
    got = traces.replay(load(tmp_path, 8, 8, ("cpu", "float32")), traces.whole(reqs))
    check(got, plain_logits(src, reqs), "float32")
