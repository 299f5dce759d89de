"""The Zisedra decoder as a plan of parts.

One residual stream; every sub-layer's output joins it times ``residual_mult``. A layer is a
pre-norm block (RMS norms) whose mixer is a gated delta rule, or windowed softmax attention
beside a delta rule with a decay per key channel (their normalised outputs averaged), and
whose feed-forward is a routed mixture of clamped gated experts with a shared expert, or nothing. A span
of layers may run several times in a row; every pass over it begins with the stream and the
embedding's output going through one matrix, and every run of a layer has caches of its own.
The head is the embedding table. Tensor names are those of the model file: ``embed``,
``loop.in``, ``l<i>.norm1|norm2``, ``l<i>.mix.*`` (under ``.left`` and ``.right`` for a parallel
mixer, with ``l<i>.mix.left.out|right.out`` for the norms on their outputs),
``l<i>.mlp.router``, ``l<i>.mlp.e<j>.gate|up|down``, ``l<i>.mlp.shared.gate|up|down``, ``final.norm``.
"""

from __future__ import annotations

from ..config.zisedra import (DeltaSizes, MixtureSizes, Rotation, WindowAttentionSizes, ZisedraConfig,
                              ZisedraLayer)
from ..parts.plan import LayerSpec, ModelPlan, PartSpec, RunStep
from ..registry import part_class, register_architecture, register_preset


def _norm(cfg: ZisedraConfig, name: str) -> PartSpec:
    return PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps, "delta_scale": cfg.residual_mult}, {"weight": name})


def _delta(cfg: ZisedraConfig, s: DeltaSizes, p: str, per_channel: bool) -> PartSpec:
    names = ["q", "k", "v", "b", "A_log", "dt_bias", "norm", "o"]
    names += ["a1", "a2", "g1", "g2"] if per_channel else ["a", "g"]
    args = {"hidden_size": cfg.width, "num_heads": s.heads, "num_kv_heads": s.kv_heads, "head_dim": s.dim,
            "value_dim": s.vdim, "taps": s.conv, "norm_eps": cfg.eps,
            "decay": "channel" if per_channel else "head", "gate": "sigmoid_low_rank" if per_channel else "silu"}
    if per_channel:
        args.update(decay_rank=s.decay_rank, gate_rank=s.gate_rank)
    return PartSpec("gated_delta", args, {n: f"{p}.{n}" for n in names})


def _window_attention(cfg: ZisedraConfig, s: WindowAttentionSizes, p: str) -> PartSpec:
    tensors = {n: f"{p}.{n}" for n in ("q", "k", "v", "o")}
    tensors.update({f"{n}_bias": f"{p}.{n}.b" for n in ("q", "k", "v")})
    position = PartSpec("rope_pairs", {"head_dim": s.dim, "dims": s.rot.dims, "base": s.rot.base,
                                       "scaling": s.rot.scaling_dict()})
    return PartSpec("gqa_attention", {"hidden_size": cfg.width, "num_heads": s.heads, "num_kv_heads": s.kv_heads,
                                      "head_dim": s.dim, "value_dim": s.vdim, "scale": s.scale, "window": s.window,
                                      "bias": True, "position": position}, tensors)


def _mixer(cfg: ZisedraConfig, layer: ZisedraLayer, p: str) -> PartSpec:
    if layer.kind == "delta":
        return _delta(cfg, layer.mixer, f"{p}.mix", False)
    left, right = layer.mixer
    return PartSpec("side_by_side",
                    {"hidden_size": cfg.width, "eps": cfg.eps,
                     "branches": (_window_attention(cfg, left, f"{p}.mix.left"), _delta(cfg, right, f"{p}.mix.right", True))},
                    {"out0": f"{p}.mix.left.out", "out1": f"{p}.mix.right.out"})


def _feed_forward(cfg: ZisedraConfig, s: MixtureSizes | None, p: str) -> PartSpec | None:
    if s is None:
        return None
    tensors = {n: f"{p}.mlp.e{{e}}.{n}" for n in ("gate", "up", "down")}
    tensors["router"] = f"{p}.mlp.router"
    tensors.update({f"shared_{n}": f"{p}.mlp.shared.{n}" for n in ("gate", "up", "down")})
    return PartSpec("routed_experts",
                    {"hidden_size": cfg.width, "intermediate_size": s.ff, "num_experts": s.experts, "top": s.top,
                     "router_bias": False, "scoring": "sigmoid", "groups": s.groups, "keep": s.keep,
                     "activation": "clamped", "limit": s.limit, "shared_size": s.shared_ff or None,
                     "shared_limit": s.shared_limit}, tensors)


def plan_zisedra(cfg: ZisedraConfig) -> ModelPlan:
    layers, unread = [], []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}"
        ff = _feed_forward(cfg, layer.feed_forward, p)
        norms = {"input": _norm(cfg, f"{p}.norm1")}
        if ff is not None:
            norms["post_mixer"] = _norm(cfg, f"{p}.norm2")
        else:
            unread.append(f"{p}.norm2")  # a file may carry the norm of a feed-forward that is not there
        layers.append(LayerSpec(PartSpec("pre_norm"), _mixer(cfg, layer, p), ff, norms))
    entries = []
    if cfg.loop is not None:
        entries.append(PartSpec("origin_mix", {"hidden_size": cfg.width, "delta_scale": cfg.residual_mult},
                                {"weight": "loop.in"}))
    caches, order = [], []
    for i, enters in cfg.run_order():  # every run of a layer has caches of its own
        mixer = layers[i].mixer
        specs = part_class("mixer", mixer.kind)(**mixer.args, tensors=mixer.tensors).cache_specs()
        ids = tuple(range(len(caches), len(caches) + len(specs)))
        caches.extend(specs)
        order.append(RunStep(layer=i, cache=ids, entry=0 if enters else None))
    sizes = {"vocab_size": cfg.vocab, "hidden_size": cfg.width}
    return ModelPlan(
        hidden_size=cfg.width, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
        embedding=PartSpec("token_embedding", sizes, {"weight": "embed"}),
        layers=layers, caches=caches, order=order, final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("linear_head", sizes, {"weight": "embed"}),
        ignorable=tuple(unread), eos_token_id=cfg.eos_token_id, entries=entries,
    )


def _rot(dims, base, scaling=None):
    return Rotation(dims, base, scaling)


# Small configurations for tests and examples; they differ in every size and option.
_MOE_A = MixtureSizes(ff=48, limit=1.5, experts=12, top=3, groups=3, keep=2, shared_ff=80, shared_limit=2.0)
_MOE_B = MixtureSizes(ff=32, limit=0.8, experts=6, top=2, groups=1, keep=1)
PRESETS: dict[str, ZisedraConfig] = {
    "zisedra_tiny_a": ZisedraConfig(
        vocab=300, width=96, eps=1e-5, residual_mult=0.7, loop=(0, 2, 3),
        layers=(
            ZisedraLayer("delta", DeltaSizes(heads=6, kv_heads=3, dim=16, vdim=24, conv=3), _MOE_A),
            ZisedraLayer("parallel", (WindowAttentionSizes(6, 2, 32, 16, 0.2, 21, _rot(12, 5000.0, (4.0, 1.0, 3.0, 64.0))),
                                      DeltaSizes(heads=3, kv_heads=3, dim=48, vdim=20, conv=2, decay_rank=8, gate_rank=12)),
                         _MOE_B),
            ZisedraLayer("delta", DeltaSizes(heads=2, kv_heads=1, dim=40, vdim=40, conv=5), None),
        ),
    ),
    "zisedra_tiny_b": ZisedraConfig(
        vocab=200, width=64, eps=1e-6, residual_mult=1.0, loop=None,
        layers=(
            ZisedraLayer("parallel", (WindowAttentionSizes(4, 4, 16, 16, 0.25, 9, _rot(16, 100.0)),
                                      DeltaSizes(heads=4, kv_heads=2, dim=16, vdim=16, conv=4, decay_rank=4, gate_rank=4)),
                         _MOE_A),
            ZisedraLayer("delta", DeltaSizes(heads=2, kv_heads=2, dim=72, vdim=8, conv=4), _MOE_B),
        ),
    ),
}
PRESET_PAGE_SIZE = {"zisedra_tiny_a": 16, "zisedra_tiny_b": 8}


def sized(width: int, layers: int, heads: int, kv_heads: int, dim: int, vocab: int, *, expert_ff: int, experts: int = 16,
          top: int = 2, shared_ff: int = 0, window: int = 2048, parallel_every: int = 2) -> ZisedraConfig:
    """A configuration of the sizes of a real model, for measurements: delta layers, every
    ``parallel_every``-th one a parallel mixer, a mixture in each."""
    att = WindowAttentionSizes(heads, kv_heads, dim, dim, dim ** -0.5, window, _rot(dim, 1e6))
    delta = DeltaSizes(heads, kv_heads, dim, dim, 4)
    right = DeltaSizes(heads, kv_heads, dim, dim, 4, decay_rank=64, gate_rank=64)
    moe = MixtureSizes(expert_ff, 7.0, experts, top, 4, 2, shared_ff, 7.0)
    return ZisedraConfig(vocab=vocab, width=width, eps=1e-5, residual_mult=1.0, layers=tuple(
        ZisedraLayer("parallel", (att, right), moe) if i % parallel_every == parallel_every - 1 else
        ZisedraLayer("delta", delta, moe) for i in range(layers)))


register_architecture(ZisedraConfig.architecture, ZisedraConfig.from_dict, plan_zisedra)
for _name, _cfg in PRESETS.items():
    register_preset(_name, _cfg.to_dict(), PRESET_PAGE_SIZE.get(_name, 16))
# layers of the sizes of the 4B and 8B dense presets, and of a smaller width, with a mixture like
# `deginex_4b_moe`'s in every layer, for measurements beside it
register_preset("zisedra_4b", sized(2560, 36, 32, 8, 128, 151936, expert_ff=1536, shared_ff=1536).to_dict(), 16)
register_preset("zisedra_8b", sized(4096, 36, 32, 8, 128, 151936, expert_ff=2048, shared_ff=2048).to_dict(), 16)
register_preset("zisedra_2b", sized(2048, 28, 16, 4, 128, 151936, expert_ff=1024, shared_ff=1024).to_dict(), 16)
