"""Plain, slow Zisedra decoder: whole sequences, no cache, one function per mechanism.

It shares no code with the engine: it reads config.json and the safetensors file itself and
works on one whole sequence at a time in ``dtype`` (float64 unless asked otherwise).

The design in short. One residual stream; every sub-layer's output is scaled by a constant
before it is added. A layer's mixer is either a gated delta rule (a matrix-valued recurrent
state per head, written with a learned step size and forgotten with a learned decay; queries,
keys and values pass a short causal convolution first) or two mixers side by side, softmax
attention over a sliding window with an interleaved, partial, frequency-scaled rotation next to
a delta rule whose decay has one value per key channel, their outputs normalised and averaged.
Feed-forwards are routed mixtures of clamped gated experts with sigmoid scores, a choice limited
to the best groups of experts, and a shared expert beside them. A span of layers may run several
times in a row; every such pass begins by mixing the embedding back into the stream. The head is
the embedding table.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last dimension."""
    y = x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def unit_vector(x, eps=1e-6):
    """x / sqrt(sum(x^2) + eps) over the last dimension."""
    return x / torch.sqrt(x.pow(2).sum(dim=-1, keepdim=True) + eps)


def causal_conv_silu(x, taps_w):
    """x [T, C], taps_w [C, K] (last column multiplies the current token), zeros before the
    start; then silu."""
    t, c = x.shape
    k = taps_w.shape[1]
    padded = torch.cat([x.new_zeros(k - 1, c), x], dim=0)
    y = x.new_zeros(t, c)
    for j in range(k):
        y = y + padded[j: j + t] * taps_w[:, j]
    return y * torch.sigmoid(y)


def softplus(x):
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


def delta_rule(q, k, v, beta, decay):
    """The recurrence of one head, token by token. q, k [T, D]; v [T, Dv]; beta [T]; decay [T]
    (one value for the head) or [T, D] (one per key channel, acting on the rows of the state).
    S <- decay * S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    t, d = k.shape
    dv = v.shape[1]
    s = q.new_zeros(d, dv)
    out = q.new_zeros(t, dv)
    for i in range(t):
        g = decay[i]
        s = s * (g[:, None] if g.dim() == 1 else g)
        u = beta[i] * (v[i] - s.T @ k[i])
        s = s + torch.outer(k[i], u)
        out[i] = s.T @ q[i]
    return out


def delta_mixer(h, w, sizes, eps, per_channel):
    """h [T, width] -> [T, width]. ``per_channel``: the decay comes from a low-rank pair a1, a2 and has
    one value per head and key channel, and the output gate is sigmoid of a low-rank pair g1, g2;
    otherwise one decay per head from ``a`` and a silu gate from ``g``."""
    t = h.shape[0]
    nh, nk, d, dv = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    q = causal_conv_silu(h @ w["q"].T, w["q.conv"]).view(t, nk, d)
    k = causal_conv_silu(h @ w["k"].T, w["k.conv"]).view(t, nk, d)
    v = causal_conv_silu(h @ w["v"].T, w["v.conv"]).view(t, nh, dv)
    q = unit_vector(q) * d ** -0.5
    k = unit_vector(k)
    beta = torch.sigmoid(h @ w["b"].T)                                   # [T, heads]
    rate = torch.exp(w["A_log"])                                          # [heads]
    if per_channel:
        a = (h @ w["a1"].T) @ w["a2"].T + w["dt_bias"]                    # [T, heads * d]
        decay = torch.exp(-rate[None, :, None] * softplus(a).view(t, nh, d))
        gate = torch.sigmoid((h @ w["g1"].T) @ w["g2"].T)
    else:
        a = h @ w["a"].T + w["dt_bias"]                                   # [T, heads]
        decay = torch.exp(-rate[None, :] * softplus(a))
        z = h @ w["g"].T
        gate = z * torch.sigmoid(z)
    group = nh // nk
    out = h.new_zeros(t, nh, dv)
    for head in range(nh):
        out[:, head] = delta_rule(q[:, head // group], k[:, head // group], v[:, head], beta[:, head], decay[:, head])
    out = rms_norm(out, w["norm"], eps) * gate.view(t, nh, dv)
    return out.reshape(t, nh * dv) @ w["o"].T


def scaled_frequencies(rot, dtype):
    """Angles per position of the rotated pairs: base^(-2i/dims), long wavelengths slowed by
    ``factor``, short ones kept, a linear blend between."""
    dims = rot["dims"]
    i = torch.arange(dims // 2, dtype=dtype)
    f = rot["base"] ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if sc:
        wavelength = 2 * math.pi / f
        smooth = (sc["original"] / wavelength - sc["low"]) / (sc["high"] - sc["low"])
        blended = (1 - smooth) * f / sc["factor"] + smooth * f
        f = torch.where(wavelength < sc["original"] / sc["high"], f,
                        torch.where(wavelength > sc["original"] / sc["low"], f / sc["factor"], blended))
    return f


def rotate_interleaved(x, positions, freqs):
    """x [T, heads, D]: elements 2i, 2i+1 (i < len(freqs)) turn by positions * freqs[i]; the rest pass."""
    n = freqs.shape[0]
    angle = positions.to(x.dtype)[:, None] * freqs[None, :]
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    a, b = x[..., 0: 2 * n: 2], x[..., 1: 2 * n: 2]
    y = x.clone()
    y[..., 0: 2 * n: 2] = a * cos - b * sin
    y[..., 1: 2 * n: 2] = b * cos + a * sin
    return y


def window_attention(h, w, sizes):
    """Softmax attention: position i sees j with 0 <= i - j < window."""
    t = h.shape[0]
    nh, nk, d, dv = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    q = (h @ w["q"].T + w["q.b"]).view(t, nh, d)
    k = (h @ w["k"].T + w["k.b"]).view(t, nk, d)
    v = (h @ w["v"].T + w["v.b"]).view(t, nk, dv)
    pos = torch.arange(t)
    freqs = scaled_frequencies(sizes["rot"], h.dtype)
    q, k = rotate_interleaved(q, pos, freqs), rotate_interleaved(k, pos, freqs)
    gap = pos[:, None] - pos[None, :]
    seen = (gap >= 0) & (gap < sizes["mask"]["size"])
    group = nh // nk
    out = h.new_zeros(t, nh, dv)
    for head in range(nh):
        scores = (q[:, head] @ k[:, head // group].T) * sizes["scale"]
        scores = scores.masked_fill(~seen, float("-inf"))
        out[:, head] = torch.softmax(scores, dim=-1) @ v[:, head // group]
    return out.reshape(t, nh * dv) @ w["o"].T


def parallel_mixer(h, w, sizes, eps):
    left = window_attention(h, {n[5:]: x for n, x in w.items() if n.startswith("left.")}, sizes["left"])
    right = delta_mixer(h, {n[6:]: x for n, x in w.items() if n.startswith("right.")}, sizes["right"], eps, True)
    return 0.5 * (rms_norm(left, w["left.out"], eps) + rms_norm(right, w["right.out"], eps))


def expert(h, gate, up, down, limit):
    g = torch.clamp(h @ gate.T, max=limit)
    u = torch.clamp(h @ up.T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ down.T


def route(h, router, top, groups, keep):
    """Sigmoid scores; experts outside the ``keep`` groups with the largest sums of their two
    best scores cannot be chosen; the ``top`` best of the rest, weighted by their scores."""
    s = torch.sigmoid(h.to(torch.float32) @ router.to(torch.float32).T).to(h.dtype)
    t, e = s.shape
    per = e // groups
    grouped = s.view(t, groups, per)
    group_score = grouped.topk(min(2, per), dim=-1).values.sum(dim=-1)
    kept = group_score.topk(keep, dim=-1).indices
    allowed = torch.zeros(t, groups, dtype=torch.bool)
    allowed.scatter_(1, kept, True)
    masked = torch.where(allowed[:, :, None].expand(t, groups, per).reshape(t, e), s, s.new_full((), -1.0))
    index = masked.topk(top, dim=-1).indices
    return index, s.gather(1, index)


def mixture(h, w, mlp):
    r = mlp["router"]
    index, weight = route(h, w["router"], r["top"], r["groups"]["count"], r["groups"]["keep"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, p in zip(index[t].tolist(), weight[t]):
            out[t] += p * expert(h[t], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], mlp["expert"]["limit"])
    if mlp.get("shared"):
        out = out + expert(h, w["shared.gate"], w["shared.up"], w["shared.down"], mlp["shared"]["limit"])
    return out


def read_safetensors(path, dtype=torch.float64):
    raw = Path(path).read_bytes()
    n = int.from_bytes(raw[:8], "little")
    header = json.loads(raw[8: 8 + n])
    kinds = {"BF16": torch.bfloat16, "F32": torch.float32, "F16": torch.float16, "I32": torch.int32}
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        a, b = meta["data_offsets"]
        t = torch.frombuffer(bytearray(raw[8 + n + a: 8 + n + b]), dtype=kinds[meta["dtype"]]).view(meta["shape"])
        out[name] = t if meta["dtype"] == "I32" else t.to(dtype)
    return out


def sub(weights, prefix):
    return {n[len(prefix):]: x for n, x in weights.items() if n.startswith(prefix)}


def run_order(cfg):
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    first = [(i, False) for i in range(loop["start"])]
    body = [(i, i == loop["start"]) for i in range(loop["start"], loop["stop"])] * loop["times"]
    return first + body + [(i, False) for i in range(loop["stop"], n)]


def forward(cfg, weights, ids, return_layers=False):
    """Logits [T, vocab] of one whole sequence (and the stream after every layer run)."""
    eps, m = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    x0 = weights["embed"][torch.as_tensor(ids, dtype=torch.long)]
    x = x0
    after = []
    for i, enters in run_order(cfg):
        layer = cfg["layers"][i]
        w = sub(weights, f"l{i}.")
        if enters:  # a pass of the looped span begins: the embedding comes back in
            x = torch.cat([x, x0], dim=-1) @ weights["loop.in"].T
        h = rms_norm(x, w["norm1"], eps)
        if layer["type"] == "delta":
            y = delta_mixer(h, sub(w, "mix."), layer["mixer"], eps, False)
        elif layer["type"] == "parallel":
            y = parallel_mixer(h, sub(w, "mix."), layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + m * y
        if layer.get("mlp"):
            x = x + m * mixture(rms_norm(x, w["norm2"], eps), sub(w, "mlp."), layer["mlp"])
        after.append(x)
    logits = rms_norm(x, weights["final.norm"], eps) @ weights["embed"].T
    return (logits, torch.stack(after)) if return_layers else logits


def load(folder, dtype=torch.float64):
    folder = Path(folder)
    cfg = json.loads((folder / "config.json").read_text())
    return cfg, read_safetensors(folder / "model.safetensors", dtype)
