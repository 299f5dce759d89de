"""The Deginex decoder as a plan of parts.

Every layer is a pre-norm block over several residual streams (hyper-connections; over one
stream with the plain residual sum when the file names none): grouped-query attention without
position encoding (unit-RMS queries and keys, fixed scale, tanh cap, a mask of chunks, an output
gate), then a dense SwiGLU, a routed mixture of SwiGLU experts, or nothing. All norms are layer
norms with bias. A span of layers may run several times in a row, each run with a cache of its
own. The head is the embedding table. Tensor names are those of the model file:
``embed``, ``l<i>.norm1|norm2[.b]``, ``l<i>.mix.q|k|v|g|o``, ``l<i>.mlp.gate|up|down`` or
``l<i>.mlp.e<j>.gate|up|down`` with ``l<i>.mlp.router[.b]``, ``l<i>.hc1|hc2.in|out|mix``,
``final.norm[.b]``.
"""

from __future__ import annotations

from ..config.deginex import AttentionSizes, DeginexConfig, DeginexLayer, FeedForwardSizes
from ..parts.plan import CacheSpec, LayerSpec, ModelPlan, PartSpec, RunStep
from ..registry import register_architecture, register_preset


def _norm(cfg: DeginexConfig, name: str, streams: int = 1) -> PartSpec:
    args = {"size": cfg.width, "eps": cfg.eps}
    if streams > 1:
        args["streams"] = streams
    return PartSpec("layernorm", args, {"weight": name, "bias": name + ".b"})


def _mixer(cfg: DeginexConfig, sizes: AttentionSizes, p: str) -> PartSpec:
    return PartSpec(
        "gqa_attention",
        {
            "hidden_size": cfg.width, "num_heads": sizes.heads, "num_kv_heads": sizes.kv_heads,
            "head_dim": sizes.dim, "value_dim": sizes.vdim,
            "qk_norm_eps": cfg.eps, "qk_norm_weight": False, "position": None,
            "scale": sizes.scale, "softcap": sizes.softcap, "chunk": sizes.chunk, "output_gate": True,
        },
        {name: f"{p}.mix.{name}" for name in ("q", "k", "v", "g", "o")},
    )


def _feed_forward(cfg: DeginexConfig, sizes: FeedForwardSizes | None, p: str) -> PartSpec | None:
    if sizes is None:
        return None
    if sizes.kind == "dense":
        return PartSpec("swiglu", {"hidden_size": cfg.width, "intermediate_size": sizes.ff},
                        {name: f"{p}.mlp.{name}" for name in ("gate", "up", "down")})
    tensors = {name: f"{p}.mlp.e{{e}}.{name}" for name in ("gate", "up", "down")}
    tensors.update(router=f"{p}.mlp.router", router_bias=f"{p}.mlp.router.b")
    return PartSpec("moe_swiglu", {"hidden_size": cfg.width, "intermediate_size": sizes.ff,
                                   "num_experts": sizes.experts, "top": sizes.top, "router_bias": True}, tensors)


def plan_deginex(cfg: DeginexConfig) -> ModelPlan:
    layers, unread = [], []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}"
        ff = _feed_forward(cfg, layer.feed_forward, p)
        norms = {"input": _norm(cfg, f"{p}.norm1")}
        if ff is not None:
            norms["post_mixer"] = _norm(cfg, f"{p}.norm2")
        else:
            # a layer without feed-forward has no second sub-layer: a file may still carry the norm
            # and the stream coefficients that would have gone with it; they are not read
            unread += [f"{p}.norm2", f"{p}.norm2.b"] + [f"{p}.hc2.{kind}" for kind in ("in", "out", "mix")]
        if cfg.streams is None:
            block = PartSpec("pre_norm")
        else:
            names = {f"{kind}{q}": f"{p}.hc{q}.{kind}" for q in ("1", "2") for kind in ("in", "out", "mix")}
            block = PartSpec("hyper_connections", {"streams": cfg.streams}, names)
        layers.append(LayerSpec(block, _mixer(cfg, layer.mixer, p), ff, norms))
    caches, order = [], []
    for i in cfg.run_order():  # a layer that runs again has a cache of its own for that run
        m = cfg.layers[i].mixer
        caches.append(CacheSpec("paged_kv", heads=m.kv_heads, head_dim=m.dim, chunk=m.chunk,
                                value_dim=None if m.vdim == m.dim else m.vdim))
        order.append(RunStep(layer=i, cache=len(caches) - 1))
    sizes = {"vocab_size": cfg.vocab, "hidden_size": cfg.width}
    return ModelPlan(
        hidden_size=cfg.width, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
        embedding=PartSpec("token_embedding", sizes, {"weight": "embed"}),
        layers=layers, caches=caches, order=order,
        final_norm=_norm(cfg, "final.norm", cfg.streams or 1),
        head=PartSpec("linear_head", sizes, {"weight": "embed"}),
        ignorable=tuple(unread),
        eos_token_id=cfg.eos_token_id,
    )


def _attention(heads, kv_heads, dim, vdim, scale, softcap, chunk):
    return AttentionSizes(heads, kv_heads, dim, vdim, scale, softcap, chunk)


# Small configurations for tests and examples; they differ in every size and option.
PRESETS: dict[str, DeginexConfig] = {
    "deginex_tiny_a": DeginexConfig(
        vocab=320, width=128, eps=1e-5, streams=3, loop=(0, 2, 2),
        layers=(
            DeginexLayer(_attention(4, 2, 32, 32, 0.2, 15.0, 40), FeedForwardSizes("moe", 48, 6, 2)),
            DeginexLayer(_attention(4, 1, 32, 32, 0.2, 15.0, 40), FeedForwardSizes("dense", 160)),
            DeginexLayer(_attention(4, 2, 32, 32, 0.2, 15.0, 40), FeedForwardSizes("moe", 48, 6, 2)),
        ),
    ),
    "deginex_tiny_b": DeginexConfig(
        vocab=200, width=96, eps=1e-6, streams=2, loop=None,
        layers=(
            DeginexLayer(_attention(6, 3, 16, 48, 0.3, 8.0, 24), FeedForwardSizes("dense", 112)),
            DeginexLayer(_attention(3, 3, 32, 16, 0.15, None, None), None),
            DeginexLayer(_attention(6, 1, 16, 16, 0.25, 30.0, 56), FeedForwardSizes("moe", 32, 5, 3)),
        ),
    ),
}
PRESET_PAGE_SIZE = {"deginex_tiny_a": 16, "deginex_tiny_b": 8}


def sized(width: int, layers: int, heads: int, kv_heads: int, dim: int, ff: int, vocab: int, *,
          experts: int = 0, top: int = 0, expert_ff: int = 0, chunk: int | None = 2048, streams: int | None = 4,
          softcap: float | None = 30.0) -> DeginexConfig:
    """A configuration of the sizes of a real model, for measurements: every layer alike, dense
    feed-forwards, or, with ``experts``, every other one a mixture."""
    att = _attention(heads, kv_heads, dim, dim, dim ** -0.5, softcap, chunk)
    dense, moe = FeedForwardSizes("dense", ff), FeedForwardSizes("moe", expert_ff or ff, experts, top)
    return DeginexConfig(vocab=vocab, width=width, eps=1e-5, streams=streams,
                         layers=tuple(DeginexLayer(att, moe if experts and i % 2 else dense) for i in range(layers)))


register_architecture(DeginexConfig.architecture, DeginexConfig.from_dict, plan_deginex)
for _name, _cfg in PRESETS.items():
    register_preset(_name, _cfg.to_dict(), PRESET_PAGE_SIZE.get(_name, 16))
# the sizes of the 4B dense preset, for measurements beside it
register_preset("deginex_4b", sized(2560, 36, 32, 8, 128, 9728, 151936).to_dict(), 16)
register_preset("deginex_4b_moe", sized(2560, 36, 32, 8, 128, 9728, 151936, experts=16, top=2, expert_ff=1536).to_dict(), 16)
register_preset("deginex_8b_moe", sized(4096, 36, 32, 8, 128, 12288, 151936, experts=16, top=2, expert_ff=2048).to_dict(), 16)
