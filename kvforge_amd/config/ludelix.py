"""Typed configuration of the Ludelix decoder, read from its own ``config.json`` keys.

A Ludelix ``config.json`` names its model with ``"architecture": "Ludelix"`` and describes every
layer by itself under ``"layers"``: ``type`` (``"gla"``, ``"attention"`` or ``"parallel"``),
``mixer`` (that mixer's sizes and constants; a ``parallel`` mixer holds ``left``, ``right``,
``left_scale`` and ``right_scale``) and ``mlp`` (``kind`` ``"dense"`` with ``ff``, or ``"moe"``
with ``expert.ff``, ``router.experts``, ``router.top`` and ``shared.ff``; ``null`` for none).
Top-level keys: ``vocab``, ``width``, ``norm.eps``.  The design has no position limit of its
own; ``max_positions`` may be given, and is otherwise ``DEFAULT_MAX_POSITIONS``.  The rank of a
``gla`` mixer's gate matrices is the checkpoint's; ``rank`` may name it (a model with random
weights needs it).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any

from kvforge_amd.config.fogorax import _positive
from kvforge_amd.config.model import ConfigError, ModelConfig, _require
from kvforge_amd.config.rudorax import DEFAULT_MAX_POSITIONS, YarnScaling, _number


@dataclass(frozen=True)
class WavelengthScaling:
    """Frequencies slowed by ``factor`` where a pair's wavelength exceeds ``original / low``,
    kept where it is below ``original / high``, blended between."""

    factor: float
    low: float
    high: float
    original: int

    @classmethod
    def from_dict(cls, d: dict[str, Any], where: str) -> "WavelengthScaling":
        low, high = _number(d, "low", where), _number(d, "high", where)
        if not high > low:
            raise ConfigError(f"{where}: rot.scaling.high ({high}) must exceed rot.scaling.low ({low})")
        return cls(_number(d, "factor", where), low, high, _positive(d, "original", where))

    def to_dict(self) -> dict[str, Any]:
        return {"factor": self.factor, "high": self.high, "low": self.low, "original": self.original}


@dataclass(frozen=True)
class LudelixRotary:
    """Rotation over the first ``dims`` elements of a head.  ``pairs``: ``"neighbours"`` (element
    ``2i`` with ``2i + 1``) or ``"halves"`` (element ``i`` with ``i + dims / 2``); which of the two
    a mixer uses is the design's, not the file's."""

    base: float
    dims: int
    pairs: str
    scaling: "WavelengthScaling | YarnScaling | None" = None

    @classmethod
    def from_dict(cls, d: dict[str, Any], where: str, pairs: str, scaling_cls) -> "LudelixRotary":
        dims = _positive(d, "dims", where)
        if dims % 2:
            raise ConfigError(f"{where}: rot.dims must be even, got {dims}")
        sc = d.get("scaling")
        if sc and scaling_cls is None:
            raise ConfigError(f"{where}: this mixer's rotation takes no scaling")
        return cls(_number(d, "base", where), dims, pairs, scaling_cls.from_dict(sc, where) if sc else None)

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            out["scaling"] = self.scaling.to_dict()
        return out


def _heads(d: dict[str, Any], where: str) -> tuple[int, int, int, int]:
    heads = _positive(d, "heads", where)
    kv_heads = _positive(d, "kv_heads", where) if d.get("kv_heads") is not None else heads
    if heads % kv_heads:
        raise ConfigError(f"{where}: heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
    dim = _positive(d, "dim", where)
    vdim = _positive(d, "vdim", where) if d.get("vdim") is not None else dim
    return heads, kv_heads, dim, vdim


def _rot(d: dict[str, Any], where: str, dim: int, pairs: str, scaling_cls) -> LudelixRotary | None:
    rot = d.get("rot")
    rot = LudelixRotary.from_dict(rot, where, pairs, scaling_cls) if rot else None
    if rot is not None and rot.dims > dim:
        raise ConfigError(f"{where}: rot.dims ({rot.dims}) exceeds the head size ({dim})")
    return rot


@dataclass(frozen=True)
class GlaConfig:
    """Gated linear attention: ``heads`` memories of ``dim x vdim``, decays
    ``sigmoid(.)^(1 / tau)``.  ``rank``: rows of the gates' first matrix (``None``: the
    checkpoint's)."""

    heads: int
    dim: int
    vdim: int
    tau: float
    rank: int | None = None

    @classmethod
    def from_dict(cls, d: dict[str, Any], where: str) -> "GlaConfig":
        dim = _positive(d, "dim", where)
        return cls(_positive(d, "heads", where), dim,
                   _positive(d, "vdim", where) if d.get("vdim") is not None else dim,
                   _number(d, "tau", where), _positive(d, "rank", where) if d.get("rank") is not None else None)

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"dim": self.dim, "heads": self.heads, "tau": self.tau, "vdim": self.vdim}
        if self.rank is not None:
            out["rank"] = self.rank
        return out


@dataclass(frozen=True)
class KeyValueAttentionConfig:
    """Attention whose values are its keys: biases on q and k, a norm over the whole of q and of
    k, neighbouring pairs rotated with wavelength scaling, a sliding window (``None``: none), a
    sink per head.  ``vdim`` is ``dim`` by the design."""

    heads: int
    kv_heads: int
    dim: int
    scale: float
    window: int | None
    rot: LudelixRotary | None

    @classmethod
    def from_dict(cls, d: dict[str, Any], where: str) -> "KeyValueAttentionConfig":
        heads, kv_heads, dim, vdim = _heads(d, where)
        if vdim != dim:
            raise ConfigError(f"{where}: the values are the keys, so vdim ({vdim}) must equal dim ({dim})")
        mask = d.get("mask")
        return cls(heads, kv_heads, dim, _number(d, "scale", where),
                   _positive(mask, "size", where) if mask else None,
                   _rot(d, where, dim, "neighbours", WavelengthScaling))

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
                               "scale": self.scale, "vdim": self.dim}
        if self.window:
            out["mask"] = {"size": self.window}
        if self.rot:
            out["rot"] = self.rot.to_dict()
        return out


@dataclass(frozen=True)
class ChunkAttentionConfig:
    """Attention within chunks of ``chunk`` positions (``None``: every earlier key), halves
    rotated against each other with YaRN scaling, one sigmoid gate per head."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int | None
    rot: LudelixRotary | None

    @classmethod
    def from_dict(cls, d: dict[str, Any], where: str) -> "ChunkAttentionConfig":
        heads, kv_heads, dim, vdim = _heads(d, where)
        mask = d.get("mask")
        return cls(heads, kv_heads, dim, vdim, _number(d, "scale", where),
                   _positive(mask, "size", where) if mask else None, _rot(d, where, dim, "halves", YarnScaling))

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
                               "scale": self.scale, "vdim": self.vdim}
        if self.chunk:
            out["mask"] = {"size": self.chunk}
        if self.rot:
            out["rot"] = self.rot.to_dict()
        return out


@dataclass(frozen=True)
class RetentionConfig:
    """Linear attention with one constant decay per head (``decay``), halves rotated against
    each other without scaling."""

    heads: int
    dim: int
    vdim: int
    decay: tuple[float, ...]
    rot: LudelixRotary | None

    @classmethod
    def from_dict(cls, d: dict[str, Any], where: str) -> "RetentionConfig":
        heads, dim = _positive(d, "heads", where), _positive(d, "dim", where)
        decay = _require(d, "decay")
        if (not isinstance(decay, (list, tuple)) or len(decay) != heads
                or any(isinstance(x, bool) or not isinstance(x, (int, float)) for x in decay)):
            raise ConfigError(f"{where}: 'decay' must list one number per head ({heads}), got {decay!r}")
        return cls(heads, dim, _positive(d, "vdim", where) if d.get("vdim") is not None else dim,
                   tuple(float(x) for x in decay), _rot(d, where, dim, "halves", None))

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"decay": list(self.decay), "dim": self.dim, "heads": self.heads, "vdim": self.vdim}
        if self.rot:
            out["rot"] = self.rot.to_dict()
        return out


@dataclass(frozen=True)
class SideBySideConfig:
    """``left_scale * left(h) + right_scale * right(h)``."""

    left: ChunkAttentionConfig
    right: RetentionConfig
    left_scale: float
    right_scale: float

    @classmethod
    def from_dict(cls, d: dict[str, Any], where: str) -> "SideBySideConfig":
        return cls(ChunkAttentionConfig.from_dict(_require(d, "left"), where + " (left)"),
                   RetentionConfig.from_dict(_require(d, "right"), where + " (right)"),
                   _number(d, "left_scale", where, positive=False), _number(d, "right_scale", where, positive=False))

    def to_dict(self) -> dict[str, Any]:
        return {"left": self.left.to_dict(), "left_scale": self.left_scale, "right": self.right.to_dict(),
                "right_scale": self.right_scale}


@dataclass(frozen=True)
class LudelixMlpConfig:
    """``kind`` ``"dense"``: ``down(relu(up h)^2)`` of width ``ff``.  ``"moe"``: ``experts`` gated
    feed-forwards of width ``ff`` of which a token uses the ``top`` that a table names for its
    id, plus a shared one of width ``shared_ff`` (0: none) behind a sigmoid gate per token."""

    kind: str
    ff: int
    experts: int = 0
    top: int = 0
    shared_ff: int = 0

    @classmethod
    def from_dict(cls, d: dict[str, Any], where: str) -> "LudelixMlpConfig":
        kind = _require(d, "kind")
        if kind == "dense":
            return cls("dense", _positive(d, "ff", where))
        if kind != "moe":
            raise ConfigError(f"{where}: feed-forward kind {kind!r} is not supported (known: ('dense', 'moe'))")
        r = _require(d, "router")
        experts, top = _positive(r, "experts", where), _positive(r, "top", where)
        if top > experts:
            raise ConfigError(f"{where}: router.top ({top}) exceeds the {experts} experts")
        shared = d.get("shared")
        return cls("moe", _positive(_require(d, "expert"), "ff", where), experts, top,
                   _positive(shared, "ff", where) if shared else 0)

    def to_dict(self) -> dict[str, Any]:
        if self.kind == "dense":
            return {"ff": self.ff, "kind": "dense"}
        out: dict[str, Any] = {"expert": {"ff": self.ff}, "kind": "moe",
                               "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff:
            out["shared"] = {"ff": self.shared_ff}
        return out


@dataclass(frozen=True)
class LudelixLayerConfig:
    type: str
    mixer: "GlaConfig | KeyValueAttentionConfig | SideBySideConfig"
    mlp: LudelixMlpConfig | None

    MIXERS = {"gla": GlaConfig, "attention": KeyValueAttentionConfig, "parallel": SideBySideConfig}

    @classmethod
    def from_dict(cls, d: dict[str, Any], index: int) -> "LudelixLayerConfig":
        where = f"layer {index}"
        kind = _require(d, "type")
        if kind not in cls.MIXERS:
            raise ConfigError(f"{where}: mixer type {kind!r} is not supported (known: {tuple(cls.MIXERS)})")
        mlp = d.get("mlp")
        return cls(kind, cls.MIXERS[kind].from_dict(_require(d, "mixer"), where),
                   LudelixMlpConfig.from_dict(mlp, where) if mlp is not None else None)

    def to_dict(self) -> dict[str, Any]:
        return {"mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None, "type": self.type}


@dataclass
class LudelixConfig(ModelConfig):
    """``vocab_size`` of the base class is the file's ``vocab``."""

    width: int = 0
    norm_eps: float = 0.0
    layers: list[LudelixLayerConfig] = field(default_factory=list)

    NAME = "Ludelix"

    def __post_init__(self) -> None:
        if self.width <= 0 or self.vocab_size <= 0 or self.max_position_embeddings <= 0:
            raise ConfigError("vocab, width and max_positions must be positive")
        if not self.layers:
            raise ConfigError("a model needs at least one layer")

    @classmethod
    def from_dict(cls, d: dict[str, Any]) -> "LudelixConfig":
        layers = _require(d, "layers")
        if not isinstance(layers, list):
            raise ConfigError("'layers' must be a list")
        return cls(
            architecture=cls.NAME,
            vocab_size=_positive(d, "vocab", "config.json"),
            max_position_embeddings=(_positive(d, "max_positions", "config.json")
                                     if d.get("max_positions") is not None else DEFAULT_MAX_POSITIONS),
            bos_token_id=d.get("bos_token_id"), eos_token_id=d.get("eos_token_id"),
            width=_positive(d, "width", "config.json"),
            norm_eps=_number(_require(d, "norm"), "eps", "norm", positive=False),
            layers=[LudelixLayerConfig.from_dict(x, i) for i, x in enumerate(layers)])

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "architecture": self.NAME,
            "layers": [x.to_dict() for x in self.layers],
            "max_positions": self.max_position_embeddings,
            "norm": {"eps": self.norm_eps},
            "vocab": self.vocab_size,
            "width": self.width,
        }
        for key in ("bos_token_id", "eos_token_id"):
            if getattr(self, key) is not None:
                out[key] = getattr(self, key)
        return out

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)
