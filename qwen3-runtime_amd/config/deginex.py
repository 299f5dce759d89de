"""Typed configuration of a Deginex decoder, read from a model folder's ``config.json``.

The file names the design under ``architecture`` and gives ``vocab``, ``width``, the norm's
``eps`` (``norm.eps``), optionally the number of residual ``streams`` (hyper-connections) and a
``loop`` (``start``, ``stop``, ``times``: the layers ``start .. stop-1`` run ``times`` times in a
row), and ``layers``: per layer its ``type`` (the mixer), the mixer's sizes (``mixer``) and its
feed-forward (``mlp``, null for none). Every size and every constant that may differ between two
models of the design is read here; nothing else in the package knows one.
"""

from __future__ import annotations

import sys
from dataclasses import dataclass
from typing import Any, Mapping

from .model import ConfigError


def _positive(where: str, key: str, value) -> int:
    if isinstance(value, bool) or not isinstance(value, int) or value < 1:
        raise ConfigError(f"{where}: {key} must be a positive integer, got {value!r}")
    return value


def _unknown(where: str, raw: Mapping[str, Any], known: set) -> None:
    """Keys the design does not define change nothing; they are named, once, on standard error."""
    extra = sorted(set(raw) - known)
    if extra:
        print(f"[qwen3_runtime_amd] {where}: keys without a meaning here are ignored: {extra}", file=sys.stderr)


@dataclass(frozen=True)
class AttentionSizes:
    """Grouped-query attention without position encoding: ``heads`` query heads on ``kv_heads``
    key/value heads, keys and queries of ``dim`` elements, values of ``vdim``; scores times
    ``scale``, then capped at ``softcap`` (None: no cap); a query sees the earlier keys of its own
    chunk of ``chunk`` positions (None: all earlier keys)."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float | None
    chunk: int | None

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "AttentionSizes":
        for key in ("heads", "dim"):
            if key not in raw:
                raise ConfigError(f"{where}: the mixer lacks {key!r}")
        heads = _positive(where, "heads", raw["heads"])
        kv_heads = _positive(where, "kv_heads", raw.get("kv_heads", heads))  # absent: a key head per query head
        if heads % kv_heads:
            raise ConfigError(f"{where}: {heads} query heads do not divide into {kv_heads} key/value heads")
        dim = _positive(where, "dim", raw["dim"])
        vdim = _positive(where, "vdim", raw.get("vdim", dim))
        scale = float(raw.get("scale", dim ** -0.5))  # absent: the usual 1 / sqrt(dim)
        if not scale > 0.0:
            raise ConfigError(f"{where}: scale must be positive, got {scale!r}")
        softcap = raw.get("softcap")
        if softcap is not None and not float(softcap) > 0.0:
            raise ConfigError(f"{where}: softcap must be positive, got {softcap!r}")
        mask = raw.get("mask")
        chunk = None
        if mask is not None:
            if "size" not in mask:
                raise ConfigError(f"{where}: a mask gives its chunk 'size', got {dict(mask)!r}")
            _unknown(where + " mask", mask, {"size"})
            chunk = _positive(where, "mask.size", mask["size"])
        _unknown(where + " mixer", raw, {"heads", "kv_heads", "dim", "vdim", "scale", "softcap", "mask"})
        return cls(heads, kv_heads, dim, vdim, scale, None if softcap is None else float(softcap), chunk)

    def to_dict(self) -> dict[str, Any]:
        raw: dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                               "scale": self.scale}
        if self.softcap is not None:
            raw["softcap"] = self.softcap
        if self.chunk is not None:
            raw["mask"] = {"size": self.chunk}
        return raw


@dataclass(frozen=True)
class FeedForwardSizes:
    """``kind`` "dense": one SwiGLU of inner width ``ff``. ``kind`` "moe": ``experts`` SwiGLUs of
    inner width ``ff`` of which each token takes its ``top`` best by the router's logits."""

    kind: str
    ff: int
    experts: int = 0
    top: int = 0

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "FeedForwardSizes":
        kind = raw.get("kind")
        if kind == "dense":
            return cls("dense", _positive(where, "mlp.ff", raw.get("ff")))
        if kind == "moe":
            router, expert = raw.get("router") or {}, raw.get("expert") or {}
            experts = _positive(where, "mlp.router.experts", router.get("experts"))
            top = _positive(where, "mlp.router.top", router.get("top"))
            if top > experts:
                raise ConfigError(f"{where}: each token takes {top} experts of {experts}")
            return cls("moe", _positive(where, "mlp.expert.ff", expert.get("ff")), experts, top)
        raise ConfigError(f"{where}: unknown feed-forward kind {kind!r} (dense, moe)")

    def to_dict(self) -> dict[str, Any]:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}


@dataclass(frozen=True)
class DeginexLayer:
    mixer: AttentionSizes
    feed_forward: FeedForwardSizes | None


@dataclass(frozen=True)
class DeginexConfig:
    vocab: int
    width: int
    eps: float
    layers: tuple[DeginexLayer, ...]
    streams: int | None = None             # None: one residual stream and the plain residual sum
    loop: tuple[int, int, int] | None = None  # (start, stop, times)
    # the design has no position encoding, hence no limit of its own; a file may still give one
    max_positions: int = 1 << 20
    eos_token_id: int | None = None

    architecture = "Deginex"

    def __post_init__(self) -> None:
        _positive("config", "vocab", self.vocab)
        _positive("config", "width", self.width)
        if not self.eps > 0.0:
            raise ConfigError(f"norm.eps must be positive, got {self.eps!r}")
        if not self.layers:
            raise ConfigError("the model has no layers")
        if self.streams is not None:
            _positive("config", "streams", self.streams)
            if self.streams > 8:
                raise ConfigError(f"at most 8 residual streams are supported, got {self.streams}")
        if self.loop is not None:
            start, stop, times = self.loop
            if not (0 <= start < stop <= len(self.layers)) or times < 1:
                raise ConfigError(f"loop {self.loop} does not fit {len(self.layers)} layers")

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "DeginexConfig":
        if raw.get("architecture") != cls.architecture and cls.architecture not in (raw.get("architectures") or []):
            raise ConfigError(f"unsupported architecture: {raw.get('architecture')!r}")
        for key in ("vocab", "width", "layers", "norm"):
            if key not in raw:
                raise ConfigError(f"config.json lacks {key!r}")
        layers = []
        for i, spec in enumerate(raw["layers"]):
            where = f"layer {i}"
            if spec.get("type") != "attention":
                raise ConfigError(f"{where}: unknown mixer type {spec.get('type')!r} (attention)")
            mlp = spec.get("mlp")
            layers.append(DeginexLayer(AttentionSizes.from_dict(spec.get("mixer") or {}, where),
                                       None if mlp is None else FeedForwardSizes.from_dict(mlp, where)))
        loop = raw.get("loop")
        if loop is not None:
            loop = (int(loop["start"]), int(loop["stop"]), int(loop["times"]))
        eos = raw.get("eos_token_id")
        return cls(
            vocab=raw["vocab"], width=raw["width"], eps=float((raw["norm"] or {}).get("eps", 0.0)),
            layers=tuple(layers), streams=raw.get("streams"), loop=loop,
            max_positions=int(raw.get("max_positions", 1 << 20)),
            eos_token_id=None if eos is None else int(eos),
        )

    def to_dict(self) -> dict[str, Any]:
        """The config.json a model folder of this configuration carries."""
        raw: dict[str, Any] = {
            "architecture": self.architecture,
            "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
            "layers": [{"type": "attention", "mixer": layer.mixer.to_dict(),
                        "mlp": None if layer.feed_forward is None else layer.feed_forward.to_dict()}
                       for layer in self.layers],
        }
        if self.streams is not None:
            raw["streams"] = self.streams
        if self.loop is not None:
            raw["loop"] = {"start": self.loop[0], "stop": self.loop[1], "times": self.loop[2]}
        if self.max_positions != 1 << 20:
            raw["max_positions"] = self.max_positions
        if self.eos_token_id is not None:
            raw["eos_token_id"] = self.eos_token_id
        return raw

    def run_order(self) -> list[int]:
        """Indices of the layers in the order a pass runs them, the looped span repeated in place."""
        n = len(self.layers)
        if self.loop is None:
            return list(range(n))
        start, stop, times = self.loop
        return list(range(start)) + list(range(start, stop)) * times + list(range(stop, n))
