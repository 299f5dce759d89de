"""Typed configuration of a Zisedra decoder, read from a model folder's ``config.json``.

The file names the design under ``architecture`` and gives ``vocab``, ``width``, the norms'
``eps`` (``norm.eps``), ``residual_mult`` (what every sub-layer's output is multiplied by before it
joins the stream), optionally a ``loop`` (``start``, ``stop``, ``times``: the layers
``start .. stop-1`` run ``times`` times in a row, each pass entered through the matrix ``loop.in``),
and ``layers``: per layer its ``type`` (``delta``: a gated delta rule; ``parallel``: windowed softmax
attention, ``left``, beside a delta rule with a decay per key channel, ``right``), the mixer's
sizes (``mixer``) and its feed-forward (``mlp``: a routed mixture, or null). Every size and every
constant that may differ between two models of the design is read here. The inner sizes of the
low-rank pairs of a ``right`` mixer are the model file's (its tensors' shapes); a configuration
made here for random weights names them (``decay_rank``, ``gate_rank``).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .deginex import _positive, _unknown
from .model import ConfigError


def _number(where: str, key: str, raw: Mapping[str, Any], positive: bool = True) -> float:
    if key not in raw or isinstance(raw[key], bool) or not isinstance(raw[key], (int, float)):
        raise ConfigError(f"{where}: {key} must be a number, got {raw.get(key)!r}")
    value = float(raw[key])
    if positive and not value > 0.0:
        raise ConfigError(f"{where}: {key} must be positive, got {value!r}")
    return value


@dataclass(frozen=True)
class DeltaSizes:
    """A gated delta rule: ``heads`` value heads of ``vdim`` on ``kv_heads`` query/key heads of
    ``dim``, convolutions of ``conv`` taps."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    decay_rank: int | None = None
    gate_rank: int | None = None

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "DeltaSizes":
        for key in ("heads", "dim", "conv"):
            if key not in raw:
                raise ConfigError(f"{where}: the mixer lacks {key!r}")
        heads = _positive(where, "heads", raw["heads"])
        kv_heads = _positive(where, "kv_heads", raw.get("kv_heads", heads))
        if heads % kv_heads:
            raise ConfigError(f"{where}: {heads} heads do not divide into {kv_heads} query/key heads")
        dim = _positive(where, "dim", raw["dim"])
        _unknown(where + " mixer", raw, {"heads", "kv_heads", "dim", "vdim", "conv", "decay_rank", "gate_rank"})
        ranks = [None if raw.get(k) is None else _positive(where, k, raw[k]) for k in ("decay_rank", "gate_rank")]
        return cls(heads, kv_heads, dim, _positive(where, "vdim", raw.get("vdim", dim)),
                   _positive(where, "conv", raw["conv"]), *ranks)

    def to_dict(self) -> dict[str, Any]:
        raw = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}
        for key in ("decay_rank", "gate_rank"):
            if getattr(self, key) is not None:
                raw[key] = getattr(self, key)
        return raw


@dataclass(frozen=True)
class Rotation:
    """The first ``dims`` elements of a head turn, in interleaved pairs, with frequencies
    ``base^(-2i/dims)`` that ``scaling`` (factor, low, high, original; None: none) slows down
    for long wavelengths."""

    dims: int
    base: float
    scaling: tuple[float, float, float, float] | None = None

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "Rotation":
        dims = raw.get("dims")
        if isinstance(dims, bool) or not isinstance(dims, int) or dims < 0 or dims % 2:
            raise ConfigError(f"{where}: rot.dims must be an even number of elements, got {dims!r}")
        base = _number(where, "base", raw)
        scaling = raw.get("scaling")
        if scaling is not None:
            scaling = tuple(_number(where + " rot.scaling", k, scaling) for k in ("factor", "low", "high", "original"))
            if scaling[1] == scaling[2]:
                raise ConfigError(f"{where}: rot.scaling.low and .high must differ")
        _unknown(where + " rot", raw, {"dims", "base", "scaling"})
        return cls(dims, base, scaling)

    def to_dict(self) -> dict[str, Any]:
        raw: dict[str, Any] = {"dims": self.dims, "base": self.base}
        if self.scaling is not None:
            raw["scaling"] = dict(zip(("factor", "low", "high", "original"), self.scaling))
        return raw

    def scaling_dict(self):
        return None if self.scaling is None else dict(zip(("factor", "low", "high", "original"), self.scaling))


@dataclass(frozen=True)
class WindowAttentionSizes:
    """Softmax attention with biased projections: ``heads`` query heads on ``kv_heads`` key/value
    heads, keys of ``dim`` and values of ``vdim`` elements, scores times ``scale``, a query sees itself
    and the ``window - 1`` tokens before it."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    rot: Rotation

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "WindowAttentionSizes":
        for key in ("heads", "dim", "scale", "mask", "rot"):
            if key not in raw:
                raise ConfigError(f"{where}: the mixer lacks {key!r}")
        heads = _positive(where, "heads", raw["heads"])
        kv_heads = _positive(where, "kv_heads", raw.get("kv_heads", heads))
        if heads % kv_heads:
            raise ConfigError(f"{where}: {heads} query heads do not divide into {kv_heads} key/value heads")
        dim = _positive(where, "dim", raw["dim"])
        if dim % 2:
            raise ConfigError(f"{where}: rotated heads have an even size, got {dim}")
        rot = Rotation.from_dict(raw["rot"], where)
        if rot.dims > dim:
            raise ConfigError(f"{where}: {rot.dims} rotated elements in heads of {dim}")
        _unknown(where + " mask", raw["mask"], {"size"})
        _unknown(where + " mixer", raw, {"heads", "kv_heads", "dim", "vdim", "scale", "mask", "rot"})
        return cls(heads, kv_heads, dim, _positive(where, "vdim", raw.get("vdim", dim)), _number(where, "scale", raw),
                   _positive(where, "mask.size", raw["mask"].get("size")), rot)

    def to_dict(self) -> dict[str, Any]:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
                "mask": {"size": self.window}, "rot": self.rot.to_dict()}


@dataclass(frozen=True)
class MixtureSizes:
    """``experts`` experts of inner width ``ff`` clamped at ``limit``, ``top`` a token by sigmoid scores
    from the ``keep`` best of ``groups`` groups; a shared expert of ``shared_ff`` (0: none)."""

    ff: int
    limit: float
    experts: int
    top: int
    groups: int = 1
    keep: int = 1
    shared_ff: int = 0
    shared_limit: float = 0.0

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "MixtureSizes":
        if raw.get("kind") != "moe":
            raise ConfigError(f"{where}: unknown feed-forward kind {raw.get('kind')!r} (moe)")
        router, expert, shared = raw.get("router") or {}, raw.get("expert") or {}, raw.get("shared")
        experts = _positive(where, "mlp.router.experts", router.get("experts"))
        top = _positive(where, "mlp.router.top", router.get("top"))
        groups_raw = router.get("groups")
        groups, keep = 1, 1
        if groups_raw is not None:
            groups = _positive(where, "mlp.router.groups.count", groups_raw.get("count"))
            keep = _positive(where, "mlp.router.groups.keep", groups_raw.get("keep"))
        if experts % groups or keep > groups or keep * (experts // groups) < top or groups > 64:
            raise ConfigError(f"{where}: {experts} experts in {groups} groups (64 at most) of which {keep} stay, {top} chosen")
        _unknown(where + " mlp", raw, {"kind", "router", "expert", "shared"})
        _unknown(where + " mlp.router", router, {"experts", "top", "groups"})
        return cls(_positive(where, "mlp.expert.ff", expert.get("ff")), _number(where + " mlp.expert", "limit", expert),
                   experts, top, groups, keep,
                   0 if shared is None else _positive(where, "mlp.shared.ff", shared.get("ff")),
                   0.0 if shared is None else _number(where + " mlp.shared", "limit", shared))

    def to_dict(self) -> dict[str, Any]:
        raw: dict[str, Any] = {"kind": "moe", "expert": {"ff": self.ff, "limit": self.limit},
                               "router": {"experts": self.experts, "top": self.top,
                                          "groups": {"count": self.groups, "keep": self.keep}}}
        if self.shared_ff:
            raw["shared"] = {"ff": self.shared_ff, "limit": self.shared_limit}
        return raw


@dataclass(frozen=True)
class ZisedraLayer:
    """``kind`` "delta": ``mixer`` is a ``DeltaSizes``. ``kind`` "parallel": ``mixer`` is the pair
    (``WindowAttentionSizes``, ``DeltaSizes``), left and right."""

    kind: str
    mixer: Any
    feed_forward: MixtureSizes | None


@dataclass(frozen=True)
class ZisedraConfig:
    vocab: int
    width: int
    eps: float
    layers: tuple[ZisedraLayer, ...]
    residual_mult: float = 1.0
    loop: tuple[int, int, int] | None = None  # (start, stop, times)
    max_positions: int = 1 << 20
    eos_token_id: int | None = None

    architecture = "Zisedra"

    def __post_init__(self) -> None:
        _positive("config", "vocab", self.vocab)
        _positive("config", "width", self.width)
        if not self.eps > 0.0:
            raise ConfigError(f"norm.eps must be positive, got {self.eps!r}")
        if not self.layers:
            raise ConfigError("the model has no layers")
        if self.loop is not None:
            start, stop, times = self.loop
            if not (0 <= start < stop <= len(self.layers)) or times < 1:
                raise ConfigError(f"loop {self.loop} does not fit {len(self.layers)} layers")

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "ZisedraConfig":
        if raw.get("architecture") != cls.architecture and cls.architecture not in (raw.get("architectures") or []):
            raise ConfigError(f"unsupported architecture: {raw.get('architecture')!r}")
        for key in ("vocab", "width", "layers", "norm"):
            if key not in raw:
                raise ConfigError(f"config.json lacks {key!r}")
        layers = []
        for i, spec in enumerate(raw["layers"]):
            where = f"layer {i}"
            kind, sizes = spec.get("type"), spec.get("mixer") or {}
            if kind == "delta":
                mixer = DeltaSizes.from_dict(sizes, where)
            elif kind == "parallel":
                if "left" not in sizes or "right" not in sizes:
                    raise ConfigError(f"{where}: a parallel mixer has a 'left' and a 'right'")
                mixer = (WindowAttentionSizes.from_dict(sizes["left"], where + " left"),
                         DeltaSizes.from_dict(sizes["right"], where + " right"))
            else:
                raise ConfigError(f"{where}: unknown mixer type {kind!r} (delta, parallel)")
            mlp = spec.get("mlp")
            layers.append(ZisedraLayer(kind, mixer, None if mlp is None else MixtureSizes.from_dict(mlp, where)))
        loop = raw.get("loop")
        if loop is not None:
            loop = (int(loop["start"]), int(loop["stop"]), int(loop["times"]))
        eos = raw.get("eos_token_id")
        _unknown("config", raw, {"architecture", "architectures", "vocab", "width", "layers", "norm", "loop",
                                 "residual_mult", "max_positions", "eos_token_id"})
        return cls(vocab=raw["vocab"], width=raw["width"], eps=float((raw["norm"] or {}).get("eps", 0.0)),
                   layers=tuple(layers), residual_mult=float(raw.get("residual_mult", 1.0)), loop=loop,
                   max_positions=int(raw.get("max_positions", 1 << 20)), eos_token_id=None if eos is None else int(eos))

    def to_dict(self) -> dict[str, Any]:
        """The config.json a model folder of this configuration carries."""
        layers = []
        for layer in self.layers:
            mixer = layer.mixer.to_dict() if layer.kind == "delta" else \
                {"left": layer.mixer[0].to_dict(), "right": layer.mixer[1].to_dict()}
            layers.append({"type": layer.kind, "mixer": mixer,
                           "mlp": None if layer.feed_forward is None else layer.feed_forward.to_dict()})
        raw: dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                               "norm": {"eps": self.eps}, "residual_mult": self.residual_mult, "layers": layers}
        if self.loop is not None:
            raw["loop"] = {"start": self.loop[0], "stop": self.loop[1], "times": self.loop[2]}
        if self.max_positions != 1 << 20:
            raw["max_positions"] = self.max_positions
        if self.eos_token_id is not None:
            raw["eos_token_id"] = self.eos_token_id
        return raw

    def run_order(self) -> list[tuple[int, bool]]:
        """(layer, whether a pass over the looped span begins with it), in the order a pass over
        the model runs them."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        start, stop, times = self.loop
        body = [(i, i == start) for i in range(start, stop)] * times
        return [(i, False) for i in range(start)] + body + [(i, False) for i in range(stop, n)]
