"""Deginex: every mechanism alone against its plain function, and whole models under every cutting.

Each test runs twice: with the plain torch ops on the CPU (which pins the host side: plan,
packing, pages, chunks, the loop) and with the HIP ops on the GPU (marked ``gpu``; float32 and
bfloat16). The oracle is ``plain/deginex_plain.py``: whole sequences, no cache, float64.
Configurations are made here and differ from each other in every size and option.
"""

from __future__ import annotations

import math
from types import SimpleNamespace

import pytest
import torch

import traces
from plain import deginex_plain as P
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


# ------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("streams,width,tokens,bias", [(1, 96, 5, True), (3, 128, 7, True), (4, 2560, 3, True),
                                                       (2, 1000, 4, False), (8, 64, 2, True)])
def test_streams_update_read_and_norm(backend, streams, width, tokens, bias):
    """new[t] = sum_s mix[s, t] old[s] + out[t] y; u = sum_t read[t] new[t]; norm(u). Also with
    picked rows (nothing written back) and with the output in planes."""
    device, dtype = backend
    ops = make_ops(device)
    x = rnd(tokens, streams, width, seed=1)
    y = rnd(tokens, width, seed=2).to(DT[dtype])
    mix = torch.eye(streams) + rnd(streams, streams, seed=3, scale=0.3)
    out, read = 1 + rnd(streams, seed=4, scale=0.3), 1 + rnd(streams, seed=5, scale=0.3)
    w, b = 1 + rnd(width, seed=6, scale=0.1), rnd(width, seed=7, scale=0.1)
    eps = 1e-5
    new = P.write_streams(x.permute(1, 0, 2).double(), mix.double(), out.double(), y.double())
    u = P.read_streams(new, read.double())
    want = P.layer_norm(u, w.double(), b.double(), eps) if bias else P.unit_rms(u, eps) * w.double()
    dev = lambda t: t.to(device)  # noqa: E731
    upd = SimpleNamespace(y=dev(y), mix=dev(mix), out=dev(out))
    xs = dev(x.clone())
    got = ops.mix_norm(xs, upd, dev(read), dev(w), dev(b) if bias else None, eps, DT[dtype])
    torch.testing.assert_close(got.double().cpu(), want, **tol(dtype))
    torch.testing.assert_close(xs.cpu().double(), new.permute(1, 0, 2), atol=1e-5, rtol=1e-5)
    # rows picked out: the same numbers, and the streams stay as they were
    xs = dev(x.clone())
    rows = torch.tensor([tokens - 1, 0], dtype=torch.int32, device=device)
    got = ops.mix_norm(xs, upd, dev(read), dev(w), dev(b) if bias else None, eps, DT[dtype], rows)
    torch.testing.assert_close(got.double().cpu(), want[[tokens - 1, 0]], **tol(dtype))
    assert torch.equal(xs.cpu(), x)
    # the output in float32 planes whose sum it is
    planes = torch.stack([y.float() * 0.25, y.float() * 0.75])
    xs = dev(x.clone())
    got = ops.mix_norm(xs, SimpleNamespace(y=dev(planes), mix=dev(mix), out=dev(out)), dev(read), dev(w),
                       dev(b) if bias else None, eps, DT[dtype])
    torch.testing.assert_close(got.double().cpu(), want, **tol(dtype))
    # nothing pending: only read and norm
    xs = dev(x.clone())
    got = ops.mix_norm(xs, None, dev(read), dev(w), dev(b) if bias else None, eps, DT[dtype])
    u0 = P.read_streams(x.permute(1, 0, 2).double(), read.double())
    want0 = P.layer_norm(u0, w.double(), b.double(), eps) if bias else P.unit_rms(u0, eps) * w.double()
    torch.testing.assert_close(got.double().cpu(), want0, **tol(dtype))


@pytest.mark.parametrize("backend", BACKENDS)
def test_layer_norm_of_one_stream_with_a_plain_delta(backend):
    device, dtype = backend
    ops = make_ops(device)
    x, d = rnd(6, 200, seed=1), rnd(6, 200, seed=2).to(DT[dtype])
    w, b = 1 + rnd(200, seed=3, scale=0.1), rnd(200, seed=4, scale=0.1)
    xs = x.clone().to(device)
    got = ops.mix_norm(xs, d.to(device), None, w.to(device), b.to(device), 1e-6, DT[dtype])
    want = P.layer_norm(x.double() + d.double(), w.double(), b.double(), 1e-6)
    torch.testing.assert_close(got.double().cpu(), want, **tol(dtype))
    torch.testing.assert_close(xs.cpu().double(), x.double() + d.double(), atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("experts,top,width", [(8, 2, 256), (5, 3, 96), (6, 1, 128), (4, 4, 64), (64, 6, 512)])
def test_router_takes_the_best_and_weighs_them_among_themselves(backend, experts, top, width):
    device, dtype = backend
    ops = make_ops(device)
    x = rnd(9, width, seed=1).to(DT[dtype])
    router, bias = rnd(experts, width, seed=2, scale=0.2), rnd(experts, seed=3)
    index, weight = ops.route_top(x.to(device), router.to(device), bias.to(device), top)
    want_i, want_w = P.route(x.double(), router.double(), bias.double(), top)
    assert index.dtype == torch.int32 and weight.dtype == torch.float32
    assert torch.equal(index.cpu().long(), want_i)  # the logits are far apart; order: best first
    torch.testing.assert_close(weight.cpu().double(), want_w, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(weight.sum(-1).cpu(), torch.ones(9), atol=1e-5, rtol=0)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("experts,top,width,inner,tokens", [(8, 2, 256, 64, 11), (5, 3, 96, 40, 4), (3, 1, 128, 48, 70),
                                                            (4, 4, 64, 32, 1), (6, 2, 128, 96, 300), (16, 2, 128, 64, 3),
                                                            (7, 2, 100, 36, 9)])
def test_experts_weighted_sum(backend, experts, top, width, inner, tokens):
    """The three forms the device has: pair by pair (fewer pairs than experts, or widths without
    16-byte pieces), expert by expert on the device (several pairs an expert), and expert by
    expert through the engine's matrix products (many tokens)."""
    device, dtype = backend
    ops = make_ops(device)
    x = rnd(tokens, width, seed=1).to(DT[dtype])
    w = {}
    for e in range(experts):
        w[f"m.e{e}.gate"], w[f"m.e{e}.up"] = rnd(inner, width, seed=10 + e, scale=0.1), rnd(inner, width, seed=30 + e, scale=0.1)
        w[f"m.e{e}.down"] = rnd(width, inner, seed=50 + e, scale=0.1)
    w = {k: v.to(DT[dtype]) for k, v in w.items()}
    w["m.router"], w["m.router.b"] = rnd(experts, width, seed=2, scale=0.2), rnd(experts, seed=3)
    want = P.moe_ff(x.double(), {k: v.double() for k, v in w.items()}, "m.", experts, top)
    gate_up = torch.stack([torch.cat([w[f"m.e{e}.gate"], w[f"m.e{e}.up"]]) for e in range(experts)]).to(device)
    down = torch.stack([w[f"m.e{e}.down"] for e in range(experts)]).to(device)
    index, weight = ops.route_top(x.to(device), w["m.router"].to(device), w["m.router.b"].to(device), top)
    got = ops.moe_swiglu(x.to(device), gate_up, down, index, weight)
    assert got.shape == (tokens, width)
    torch.testing.assert_close(got.double().cpu(), want, **tol(dtype))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sigmoid_gate_on_columns_of_a_wider_matrix(dtype):
    """The gate as a step of its own (the attention kernels apply it themselves; an attention that
    cannot asks for this one)."""
    ops = make_ops("cuda:0")
    out, wide = rnd(7, 96, seed=1).to(DT[dtype]), rnd(7, 96 + 40, seed=2).to(DT[dtype])
    want = out.double() * torch.sigmoid(wide[:, 40:].double())
    got = ops.sigmoid_gate(out.to("cuda:0"), wide.to("cuda:0")[:, 40:])
    torch.testing.assert_close(got.double().cpu(), want, **(tol(dtype) if dtype == "float32" else dict(atol=2e-2, rtol=2e-2)))


def paged(keys, values, page_size, device, dtype, seed=0, spare=3):
    """Put one sequence's keys [n, heads, d] and values [n, heads, dv] into pages in a random
    order among spare ones that are poisoned; returns (view, table)."""
    from qwen3_runtime_amd.parts.base import CacheView, GroupView
    from qwen3_runtime_amd.parts.plan import CacheSpec

    n, heads, d = keys.shape
    dv = values.shape[2]
    need = -(-n // page_size)
    order = torch.randperm(need + spare, generator=torch.Generator().manual_seed(seed))[:need]
    k = torch.full((need + spare, heads, page_size, d), float("nan"))
    v = torch.full((need + spare, heads, dv, page_size), float("inf"))
    for i in range(n):
        k[order[i // page_size], :, i % page_size] = keys[i]
        v[order[i // page_size], :, :, i % page_size] = values[i]
    table = order.to(torch.int32)[None].to(device)
    spec = CacheSpec("paged_kv", heads=heads, head_dim=d, value_dim=None if dv == d else dv)
    group = GroupView(page_size, None, table, torch.zeros(0, dtype=torch.int32, device=device))
    return CacheView(spec, group=group, k=k.to(dtype).to(device), v=v.to(dtype).to(device))


def attention_ctx(ops, device, dtype, q_len, kv_len):
    from qwen3_runtime_amd.parts.base import StepContext

    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)  # noqa: E731
    return StepContext(ops=ops, dtype=dtype, device=torch.device(device), num_tokens=q_len, num_seqs=1,
                       positions=i32(list(range(kv_len - q_len, kv_len))), cu_q=i32([0, q_len]), kv_lens=i32([kv_len]),
                       seq_of_token=i32([0] * q_len), state_slots=i32([0]), first_span=i32([int(kv_len == q_len)]),
                       q_lens_host=[q_len], kv_lens_host=[kv_len], max_q_len=q_len, max_kv_len=kv_len)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("heads,kv_heads,d,dv,chunk,cap,page", [(4, 2, 64, 64, 96, 20.0, 16), (6, 3, 16, 48, 24, 8.0, 8),
                                                                (3, 3, 32, 32, None, None, 16), (8, 1, 32, 32, 40, 30.0, 8),
                                                                (4, 4, 128, 128, 50, None, 16), (2, 1, 64, 64, 7, 5.0, 8),
                                                                (2, 2, 64, 64, 1, 5.0, 8), (17, 1, 32, 32, 300, 12.0, 16)])
@pytest.mark.parametrize("q_len,kv_len", [(1, 1), (1, 97), (1, 250), (5, 5), (33, 130), (200, 200), (2, 98), (70, 333)])
def test_attention_chunks_cap_gate(backend, heads, kv_heads, d, dv, chunk, cap, page, q_len, kv_len):
    """Random queries over a paged sequence, against the plain scores, mask, cap, softmax and gate;
    prompts (many rows) and decoded tokens (one row), keys far back and across chunk edges."""
    device, dtype = backend
    ops = make_ops(device)
    dt = DT[dtype]
    q = rnd(q_len, heads, d, seed=1).to(dt)
    k, v = rnd(kv_len, kv_heads, d, seed=2).to(dt), rnd(kv_len, kv_heads, dv, seed=3).to(dt)
    gate = rnd(q_len, heads * dv + 5, seed=4).to(dt)  # columns of a wider matrix
    scale = 0.7 / math.sqrt(d)
    cache = paged(k, v, page, device, dt, seed=kv_len)
    ctx = attention_ctx(ops, device, dt, q_len, kv_len)
    more = {}
    if chunk:
        more["chunk"] = chunk
    if cap:
        more["softcap"] = cap
    if dv != d:
        more["value_dim"] = dv
    gate_dev = gate.to(device)[:, 5:]
    got = ops.paged_attention(q.reshape(q_len, heads * d).to(device), cache, ctx, heads, kv_heads, d, scale, None,
                              gate=gate_dev, **more)
    # plain: scores, cap, mask of chunks, softmax, values, gate
    rep = heads // kv_heads
    kk, vv = k.double().repeat_interleave(rep, 1), v.double().repeat_interleave(rep, 1)
    s = P.capped(torch.einsum("qhd,khd->hqk", q.double(), kk) * scale, cap)
    s = s.masked_fill(~P.visible(q_len, kv_len, kv_len - q_len, chunk), float("-inf"))
    want = torch.einsum("hqk,khd->qhd", torch.softmax(s, -1), vv).reshape(q_len, heads * dv)
    want = want * torch.sigmoid(gate[:, 5:].double())
    torch.testing.assert_close(got.double().cpu(), want, **(tol(dtype) if dtype == "float32" else dict(atol=2e-2, rtol=2e-2)))


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("q_len", [1, 40])
@pytest.mark.parametrize("chunk,page,d", [(96, 16, 64), (24, 8, 32), (50, 16, 128)])
def test_a_key_that_stands_out_is_seen_inside_the_chunk_only(backend, q_len, chunk, page, d):
    """One key is the query's own direction, scaled so that its score towers over all others; its
    value is a marker. It is placed, in turn, at the first position of the query's chunk, at the
    position just before it (outside), at the query's own position, and far back at a page's
    edge. The output is the marker exactly when the key is visible."""
    device, dtype = backend
    ops = make_ops(device)
    dt = DT[dtype]
    kv_len = 3 * chunk + 7
    pos = kv_len - 1                      # the last query's position
    start = pos - pos % chunk
    places = {start: True, start - 1: False, pos: True, page * (start // page) - 1: False, start + 1: True, 0: False}
    for place, seen in places.items():
        direction = rnd(d, seed=5)
        q = rnd(q_len, 1, d, seed=1, scale=0.05)
        q[-1, 0] = direction
        k, v = rnd(kv_len, 1, d, seed=2, scale=0.05), rnd(kv_len, 1, d, seed=3, scale=0.1)
        k[place, 0] = direction
        v[place, 0] = 7.0
        cache = paged(k.to(dt), v.to(dt), page, device, dt, seed=place)
        ctx = attention_ctx(ops, device, dt, q_len, kv_len)
        got = ops.paged_attention(q.reshape(q_len, d).to(dt).to(device), cache, ctx, 1, 1, d, 1.0, None, chunk=chunk,
                                  softcap=60.0)[-1].float().cpu()
        if seen:
            assert (got - 7.0).abs().max() < 0.1, (place, got[:4])
        else:
            assert got.abs().max() < 1.0, (place, got[:4])


# ------------------------------------------------------------------ whole models
def config_a():
    from qwen3_runtime_amd.models.deginex import PRESETS

    return PRESETS["deginex_tiny_a"].to_dict(), 16


def config_b():
    from qwen3_runtime_amd.models.deginex import PRESETS

    return PRESETS["deginex_tiny_b"].to_dict(), 8


def config_c():
    """Values that other configurations make equal or one: one stream, one key head, one expert
    taken of two, a chunk of one page, a loop over the last layer, no cap."""
    att = {"heads": 2, "kv_heads": 1, "dim": 64, "vdim": 64, "scale": 0.11, "mask": {"size": 16}}
    return {"architecture": "Deginex", "vocab": 97, "width": 64, "norm": {"eps": 1e-5}, "streams": 1,
            "loop": {"start": 1, "stop": 2, "times": 3},
            "layers": [{"type": "attention", "mixer": att, "mlp": {"kind": "moe", "expert": {"ff": 32},
                                                                   "router": {"experts": 2, "top": 1}}},
                       {"type": "attention", "mixer": dict(att, softcap=12.0), "mlp": {"kind": "dense", "ff": 80}}]}, 16


def config_d():
    """No streams at all (the plain residual sum), no loop, a layer without feed-forward."""
    att = {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 32, "scale": 0.2, "softcap": 25.0, "mask": {"size": 33}}
    return {"architecture": "Deginex", "vocab": 150, "width": 128, "norm": {"eps": 1e-5},
            "layers": [{"type": "attention", "mixer": att, "mlp": None},
                       {"type": "attention", "mixer": att, "mlp": {"kind": "dense", "ff": 96}}]}, 8


def config_e():
    """Sizes that fit no kernel's favourite shapes: a width and inner widths that are no multiples
    of 8, keys of 24 and values of 40 elements, 17 query heads to a key head, five streams, a chunk
    of 13 positions, every expert taken, an odd vocabulary."""
    return {"architecture": "Deginex", "vocab": 77, "width": 100, "norm": {"eps": 1e-5}, "streams": 5,
            "loop": {"start": 0, "stop": 1, "times": 2},
            "layers": [{"type": "attention",
                        "mixer": {"heads": 4, "kv_heads": 2, "dim": 24, "vdim": 40, "scale": 0.3, "softcap": 9.0,
                                  "mask": {"size": 13}},
                        "mlp": {"kind": "moe", "expert": {"ff": 20}, "router": {"experts": 3, "top": 3}}},
                       {"type": "attention",
                        "mixer": {"heads": 34, "kv_heads": 2, "dim": 16, "vdim": 16, "scale": 0.2, "mask": {"size": 64}},
                        "mlp": {"kind": "dense", "ff": 52}}]}, 8


CONFIGS = {"a": config_a, "b": config_b, "c": config_c, "d": config_d, "e": config_e}
# share of positions at which a router may choose differently in bfloat16 (three routed runs a
# token in "a", one in "b" and "c", none in "d")
FLIPS = {"a": 0.09, "b": 0.03, "c": 0.03, "d": 0.0, "e": 0.0}
LENGTHS = {"a": [1, 7, 45, 130], "b": [3, 17, 50, 64, 101], "c": [2, 16, 17, 49], "d": [5, 33, 34, 70],
           "e": [1, 13, 14, 66, 90]}
_folders: dict = {}


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    from qwen3_runtime_amd.weights import write_model_folder

    def get(name):
        if name not in _folders:
            raw, _ = CONFIGS[name]()
            _folders[name] = write_model_folder(tmp_path_factory.mktemp("deginex_" + name), raw, seed=31 + len(_folders),
                                                std=0.08, norm_jitter=0.2)
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
    cfg, w = P.read_model(folder)
    out = {}
    for rid, toks in requests.items():
        logits = P.forward(cfg, w, toks).float()
        for p in range(len(toks)):
            out[(rid, p)] = logits[p]
    return out


def check(got, want, dtype, flips=0.03):
    """float32: to rounding of float32 sums, everywhere. bfloat16: as noise relative to the logits'
    own spread; but a router is a hard choice, and where two experts' logits lie within rounding of
    each other bfloat16 may take the other one, which moves that one position's logits by a large
    part of their spread. So up to ``flips`` of the positions may lie over the bound; a wrong mask,
    page or portion shows in float32, where no position may, and in the mechanisms' own tests."""
    if dtype == "float32":
        traces.compare(got, want, atol=1e-4, rtol=1e-4)
        return
    keys = sorted(want)
    assert set(got) == set(want)
    w = torch.stack([want[k].double() for k in keys])
    err = torch.stack([got[k].double() for k in keys]) - w
    std = float(w.std())
    per_pos = err.abs().amax(dim=1)
    good = per_pos < 0.1 * std
    assert int((~good).sum()) <= flips * len(keys), \
        f"{int((~good).sum())} of {len(keys)} positions over the bound, the first {keys[int((~good).nonzero()[0])]}"
    rms = float(err[good].pow(2).mean().sqrt())
    assert rms < 0.02 * std, f"rms error {rms:.4f} against a logit deviation of {std:.3f}"


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("cut", ["whole", "tail_one_by_one", "portions", "mixed"])
def test_cuttings_match_plain(folder, backend, name, cut):
    """Whole prompts; the last tokens one by one (across chunk edges); portions down to two tokens;
    up to four live requests mixed in a pool of the peak's size, so that pages are used again."""
    raw, page = CONFIGS[name]()
    reqs = traces.make_requests(raw["vocab"], LENGTHS[name], seed=5)
    steps = getattr(traces, cut)(reqs)
    loaded = load(folder(name), page, traces.peak_tokens(steps, unit=page) // page, backend)
    got = traces.replay(loaded, steps, poison_freed=True)
    check(got, plain_logits(folder(name), reqs), backend[1], flips=FLIPS[name])


@pytest.mark.parametrize("backend", BACKENDS)
def test_long_decoding_through_many_chunks_in_a_small_pool(folder, backend):
    """A request far longer than the pool, decoded token by token: a chunked cache gives the pages
    of finished chunks back, so the pool of two chunks' pages serves 400 positions."""
    raw, page = config_c()
    reqs = traces.make_requests(raw["vocab"], [400], seed=8)
    steps = traces.tail_one_by_one(reqs, tail=390)
    loaded = load(folder("c"), page, 3, backend)
    got = traces.replay(loaded, steps, poison_freed=True)
    check(got, plain_logits(folder("c"), reqs), backend[1])


@pytest.mark.parametrize("backend", BACKENDS)
def test_batch_mates_do_not_change_a_request(folder, backend):
    """Unequal requests in one batch against each alone: the same logits within rounding."""
    raw, page = config_a()
    reqs = traces.make_requests(raw["vocab"], [9, 60, 121, 33], seed=2)
    together = [{"step": 0, "entries": [{"id": r, "tokens": t, "want": list(range(len(t)))} for r, t in reqs.items()],
                 "end": list(reqs)}]
    loaded = load(folder("a"), page, 32, backend)
    both = traces.replay(loaded, together)
    alone = traces.replay(loaded, traces.whole(reqs))
    if backend[1] == "float32":
        # to rounding: a step of many tokens may take another kernel than a step of few, and the
        # two take a head's sum of squares in another order
        traces.compare(both, alone, atol=1e-5, rtol=1e-5)
    else:
        check(both, alone, "bfloat16", flips=FLIPS["a"])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,graphs", [("float32", False), ("bfloat16", True), ("bfloat16", False)])
@pytest.mark.parametrize("name", ["a", "b", "d"])
def test_greedy_generation_through_the_entry_point(folder, name, dtype, graphs):
    """``LLM.generate`` (scheduler with a small token budget, sampler, graphs where they apply): the
    tokens chosen greedily are, by the plain model given the same context, the best ones or within
    rounding of the best. Requests of unequal lengths, more of them than fit at once."""
    from qwen3_runtime_amd.llm import LLM

    raw, page = CONFIGS[name]()
    llm = LLM(str(folder(name)), dtype=dtype, block_size=page, num_kv_blocks=64, max_num_seqs=3,
              max_num_batched_tokens=48, cuda_graph=graphs)
    prompts = list(traces.make_requests(raw["vocab"], [5, 61, 20, 90], seed=4).values())
    outs = llm.generate(prompts, max_tokens=40)
    cfg, w = P.read_model(folder(name))
    for prompt, tokens in zip(prompts, outs):
        assert len(tokens) == 40
        logits = P.forward(cfg, w, list(prompt) + list(tokens))[len(prompt) - 1: -1]
        below = logits.max(-1).values - logits[range(40), list(tokens)]
        bound = 1e-3 if dtype == "float32" else 0.1 * float(logits.std())
        # in bfloat16 a router may choose differently at a few places (see ``check``)
        allowed = 0 if dtype == "float32" else int(FLIPS[name] * 40)
        assert int((below >= bound).sum()) <= allowed, (float(below.max()), int(below.argmax()))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_command_line_and_trace_replay(folder, tmp_path, dtype):
    """As a user runs them: ``python -m qwen3_runtime_amd.cli --model DIR`` generates greedily, and
    ``bin/trace_run`` replays a mixed schedule from standard input and writes the logits it is
    asked for, with a pool that only holds what is live."""
    import ast
    import json
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np

    root = Path(__file__).resolve().parents[1]
    raw, page = config_d()
    cfg, w = P.read_model(folder("d"))
    prompt = [5, 17, 3, 140, 9, 77, 2]
    proc = subprocess.run([sys.executable, "-m", "qwen3_runtime_amd.cli", "--model", str(folder("d")), "--dtype", dtype,
                           "--prompt-tokens", *map(str, prompt), "--max-tokens", "8"],
                          capture_output=True, text=True, timeout=600, cwd=str(root))
    assert proc.returncode == 0, proc.stderr[-3000:]
    lines = dict(line.split(" ", 1) for line in proc.stdout.splitlines() if " " in line)
    tokens = ast.literal_eval(lines["runtime"])
    assert len(tokens) == 8
    logits = P.forward(cfg, w, prompt + tokens)[len(prompt) - 1: -1]
    below = logits.max(-1).values - logits[range(8), tokens]
    assert float(below.max()) < (1e-3 if dtype == "float32" else 0.1 * float(logits.std()))

    reqs = traces.make_requests(raw["vocab"], [70, 9, 41, 100, 35], seed=6)
    steps = traces.mixed(reqs, seed=1)
    out = tmp_path / "logits"
    proc = subprocess.run([str(root / "bin" / "trace_run"), "--model", str(folder("d")), "--dtype", dtype, "--out", str(out),
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
    check(got, plain_logits(folder("d"), reqs), dtype, flips=FLIPS["d"])


# ------------------------------------------------------------------ host side only
def test_config_reader_and_plan():
    from qwen3_runtime_amd.config.deginex import DeginexConfig
    from qwen3_runtime_amd.config.model import ConfigError
    from qwen3_runtime_amd.engine.factory import build_model

    raw, _ = config_a()
    cfg = DeginexConfig.from_dict(raw)
    assert cfg.to_dict() == raw
    assert cfg.run_order() == P.run_order(raw) == [0, 1, 0, 1, 2]
    _, model = build_model(raw)
    plan = model.plan
    assert [s.layer for s in plan.order] == [0, 1, 0, 1, 2] and [s.cache for s in plan.order] == [0, 1, 2, 3, 4]
    assert all(c.chunk == 40 and c.window is None for c in plan.caches)
    names = {d.file_name for d in model.tensor_decls()}
    assert {"embed", "l0.hc1.mix", "l0.mlp.e5.down", "l0.mlp.router.b", "l1.mlp.gate", "l2.mix.g", "final.norm.b"} <= names
    raw_d, _ = config_d()
    names_d = {d.file_name for d in build_model(raw_d)[1].tensor_decls()}
    assert not any(".hc" in n or n.startswith("l0.mlp") or n.startswith("l0.norm2") for n in names_d)
    for broken, what in [({"vocab": 0}, "vocab"), ({"loop": {"start": 2, "stop": 1, "times": 2}}, "loop"),
                         ({"streams": 0}, "streams")]:
        with pytest.raises(ConfigError, match=what):
            DeginexConfig.from_dict({**raw, **broken})
    bad = {**raw, "layers": [{"type": "recurrence", "mixer": {}, "mlp": None}]}
    with pytest.raises(ConfigError, match="mixer type"):
        DeginexConfig.from_dict(bad)


def test_a_file_may_carry_what_a_layer_without_feed_forward_does_not_read(folder, tmp_path):
    import shutil

    from safetensors.torch import load_file, save_file

    from qwen3_runtime_amd.weights.loader import WeightError

    src = folder("d")   # its first layer is a mixer alone
    tensors = load_file(str(src / "model.safetensors"))
    tensors["l0.norm2"] = torch.ones(128, dtype=torch.bfloat16)
    tensors["l0.norm2.b"] = torch.zeros(128, dtype=torch.bfloat16)
    shutil.copy(src / "config.json", tmp_path / "config.json")
    save_file(tensors, str(tmp_path / "model.safetensors"))
    load(tmp_path, 8, 8, ("cpu", "float32"))
    tensors["l1.surplus"] = torch.ones(3, dtype=torch.bfloat16)
    save_file(tensors, str(tmp_path / "model.safetensors"))
    with pytest.raises(WeightError, match="l1.surplus"):
        load(tmp_path, 8, 8, ("cpu", "float32"))


def test_pages_of_finished_chunks_go_back():
    from qwen3_runtime_amd.cache import CacheManager
    from qwen3_runtime_amd.parts.plan import CacheSpec

    spec = CacheSpec("paged_kv", heads=1, head_dim=8, chunk=20)
    cache = CacheManager([spec, spec], page_size=8, num_pages=6, max_requests=2, allocate=False)
    cache.admit("a")
    cache.reserve("a", 19)
    cache.commit("a", 19)       # positions 0..18: the next query (19) still sees its chunk from 0
    assert cache.block_table(0, "a") == [0, 1, 2]
    cache.reserve("a", 1)
    cache.commit("a", 1)        # 20 stored: the next query is in the chunk that begins at 20
    assert cache.block_table(0, "a") == [-1, -1, 2]   # page 2 holds 16..23
    cache.reserve("a", 30)      # a portion over two chunk edges keeps its pages until it is stored
    assert cache.num_free_pages == 6 - 1 - 4
    cache.commit("a", 30)       # 50 stored: chunk from 40; pages before position 40 are back
    assert [p >= 0 for p in cache.block_table(0, "a")] == [False] * 5 + [True, True]
    cache.check()
    assert cache.bytes_read([50], 2) == 2 * (2 * 8) * 10 * 2   # 10 keys seen (40..49), k and v, two caches
    ok, _ = cache.can_ever_hold(10_000)   # a chunk's pages, not the request's
    assert ok
    assert not CacheManager([spec], page_size=8, num_pages=3, max_requests=1, allocate=False).can_ever_hold(100)[0]
    cache.release("a")
    cache.check()
    assert cache.num_free_pages == 6
    with pytest.raises(ValueError, match="not both"):
        CacheSpec("paged_kv", heads=1, head_dim=8, chunk=20, window=4)
