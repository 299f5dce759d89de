"""Plain, slow Deginex decoder: whole sequences, no cache, one function per mechanism.

It shares no code with the engine: it reads config.json and the safetensors file itself and
works on one whole sequence at a time in ``dtype`` (float64 unless asked otherwise).

The design in short. Several residual streams (hyper-connections) carry the embedding; every
sub-layer reads a weighted sum of them through a layer norm with bias, and its output goes back
into all of them while a small matrix mixes the streams among themselves. Mixers are grouped-query
attention without position encoding: unit-RMS queries and keys, a fixed score scale, a tanh cap
on the scores, a mask that confines each query to the keys of its own chunk of positions, and a
sigmoid gate on the heads' output. Feed-forwards are SwiGLU, either dense or a routed mixture in
which each token takes its best few experts with softmax weights over those few. A span of
layers may run several times in a row. The head is the embedding table.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


def layer_norm(x, weight, bias, eps):
    """(x - mean) / sqrt(var + eps) * w + b with the biased variance, over the last dimension."""
    mu = x.mean(dim=-1, keepdim=True)
    var = (x - mu).pow(2).mean(dim=-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * weight + bias


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last dimension, no weight."""
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def visible(num_q, num_k, q_offset, chunk):
    """[num_q, num_k] bool: key j is seen from query position i = q_offset + row iff j <= i and,
    with a chunk size, both lie in the same chunk of positions counted from 0."""
    qpos = torch.arange(num_q)[:, None] + q_offset
    kpos = torch.arange(num_k)[None, :]
    ok = kpos <= qpos
    if chunk:
        ok = ok & (torch.div(kpos, chunk, rounding_mode="floor") == torch.div(qpos, chunk, rounding_mode="floor"))
    return ok


def capped(scores, cap):
    """cap * tanh(scores / cap); no cap: unchanged."""
    return scores if not cap else cap * torch.tanh(scores / cap)


def attention_mixer(h, w, cfg, eps, q_offset=0, past=None):
    """h [T, width] -> [T, width]. ``w``: dict with q, k, v, g, o. ``past``: (keys, values) of the
    positions before ``q_offset`` (already normed), for checks of pieces; None for a whole sequence."""
    t = h.shape[0]
    nq, nkv, d = cfg["heads"], cfg["kv_heads"], cfg["dim"]
    dv = cfg.get("vdim", d)
    q = unit_rms((h @ w["q"].T).view(t, nq, d), eps)
    k = unit_rms((h @ w["k"].T).view(t, nkv, d), eps)
    v = (h @ w["v"].T).view(t, nkv, dv)
    if past is not None:
        k = torch.cat([past[0], k])
        v = torch.cat([past[1], v])
    rep = nq // nkv
    kk = k.repeat_interleave(rep, dim=1)
    vv = v.repeat_interleave(rep, dim=1)
    scores = torch.einsum("qhd,khd->hqk", q, kk) * cfg["scale"]
    scores = capped(scores, cfg.get("softcap"))
    mask = visible(t, k.shape[0], q_offset, (cfg.get("mask") or {}).get("size"))
    scores = scores.masked_fill(~mask.to(scores.device), float("-inf"))
    probs = torch.softmax(scores, dim=-1)
    heads = torch.einsum("hqk,khd->qhd", probs, vv).reshape(t, nq * dv)
    gate = torch.sigmoid(h @ w["g"].T)
    return (heads * gate) @ w["o"].T, (k, v)


def swiglu_ff(h, gate, up, down):
    a = h @ gate.T
    return (a * torch.sigmoid(a) * (h @ up.T)) @ down.T


def route(h, router, router_bias, top):
    """Logits h W^T + b; the ``top`` largest per token and the softmax over those alone."""
    logits = h @ router.T + router_bias
    best, index = torch.topk(logits, top, dim=-1)
    return index, torch.softmax(best, dim=-1)


def moe_ff(h, w, prefix, num_experts, top):
    index, weight = route(h, w[prefix + "router"], w[prefix + "router.b"], top)
    out = torch.zeros_like(h)
    for e in range(num_experts):
        p = f"{prefix}e{e}."
        y = swiglu_ff(h, w[p + "gate"], w[p + "up"], w[p + "down"])
        share = (weight * (index == e)).sum(dim=-1, keepdim=True)
        out = out + share * y
    return out


def feed_forward(h, w, prefix, cfg):
    if cfg["kind"] == "dense":
        return swiglu_ff(h, w[prefix + "gate"], w[prefix + "up"], w[prefix + "down"])
    if cfg["kind"] == "moe":
        return moe_ff(h, w, prefix, cfg["router"]["experts"], cfg["router"]["top"])
    raise ValueError(cfg["kind"])


def read_streams(streams, weights):
    """streams [S, T, width], weights [S] -> sum_s weights[s] * streams[s]."""
    return torch.einsum("s,stw->tw", weights, streams)


def write_streams(streams, mix, out, y):
    """new[t] = sum_s mix[s, t] * streams[s] + out[t] * y, every new stream from the old ones."""
    return torch.einsum("sr,stw->rtw", mix, streams) + out[:, None, None] * y[None]


def run_order(config):
    """Indices of the layers in the order they run: the looped span repeated in place."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def read_model(folder, dtype=torch.float64):
    from safetensors.torch import load_file

    folder = Path(folder)
    config = json.loads((folder / "config.json").read_text())
    tensors = {k: (v if v.dtype in (torch.int32, torch.int64) else v.to(dtype))
               for k, v in load_file(str(folder / "model.safetensors")).items()}
    return config, tensors


def forward(config, w, ids, keep_layers=False):
    """ids: list of token ids of one sequence -> logits [T, vocab] (and, if asked, the sum of the
    streams after every layer run, [runs, T, width])."""
    eps = config["norm"]["eps"]
    x = w["embed"][torch.as_tensor(ids, dtype=torch.long)]
    s = config.get("streams")
    streams = x[None].repeat(s, 1, 1) if s else None
    after = []
    for i in run_order(config):
        spec, p = config["layers"][i], f"l{i}."
        assert spec["type"] == "attention"
        subs = [(1, lambda h: attention_mixer(h, {n: w[f"{p}mix.{n}"] for n in "qkvgo"}, spec["mixer"], eps)[0])]
        if spec.get("mlp"):
            subs.append((2, lambda h: feed_forward(h, w, p + "mlp.", spec["mlp"])))
        for q, sub in subs:
            nw, nb = w[f"{p}norm{q}"], w[f"{p}norm{q}.b"]
            if streams is None:
                x = x + sub(layer_norm(x, nw, nb, eps))
            else:
                u = read_streams(streams, w[f"{p}hc{q}.in"])
                y = sub(layer_norm(u, nw, nb, eps))
                streams = write_streams(streams, w[f"{p}hc{q}.mix"], w[f"{p}hc{q}.out"], y)
        if keep_layers:
            after.append(x if streams is None else streams.sum(0))
    if streams is not None:
        x = streams.sum(0)
    x = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
    logits = x @ w["embed"].T
    return (logits, torch.stack(after)) if keep_layers else logits
