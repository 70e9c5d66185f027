"""Typed configuration of the Buzinex decoder, read from its own ``config.json`` keys.

A Buzinex ``config.json`` names its model with ``"architecture": "Buzinex"`` and describes every
layer by itself under ``"layers"``: ``type`` (``"attention"``, ``"latent_attention"`` or
``"wkv"``), ``mixer`` (that mixer's sizes and constants) and ``mlp`` (``{"kind": "dense", "ff":
n}``, or ``null`` for none).  Top-level keys: ``vocab``, ``width``, ``norm.eps``,
``embedding.scale``, ``logit_scale`` and ``logit_softcap`` (absent or ``null``: none).  The
design has no position limit of its own; ``max_positions`` may be given, and is otherwise
``DEFAULT_MAX_POSITIONS``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any

from kvforge_amd.config.fogorax import _positive
from kvforge_amd.config.model import ConfigError, ModelConfig, _require
from kvforge_amd.config.rudorax import DEFAULT_MAX_POSITIONS, RotaryConfig, _number


def _window(d: dict[str, Any], where: str) -> int | None:
    mask = d.get("mask")
    return _positive(mask, "size", where) if mask else None


@dataclass(frozen=True)
class QueryTemperature:
    """The query of position ``p`` is multiplied by ``1 + coef * ln(floor((p + 1) / every) + 1)``."""

    coef: float
    every: int

    def to_dict(self) -> dict[str, Any]:
        return {"coef": self.coef, "every": self.every}


@dataclass(frozen=True)
class CappedAttentionConfig:
    """Grouped-query attention without rotation: q and k normalised per head, a query
    temperature, scores under a soft cap.  A file may leave out ``kv_heads`` (then as many as
    ``heads``), ``vdim`` (then ``dim``), ``q_temp``, ``softcap`` and ``mask`` (no window)."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float | None
    q_temp: QueryTemperature | None
    window: int | None = None

    @classmethod
    def from_dict(cls, d: dict[str, Any], where: str) -> "CappedAttentionConfig":
        heads = _positive(d, "heads", where)
        kv_heads = _positive(d, "kv_heads", where) if d.get("kv_heads") is not None else heads
        if heads % kv_heads:
            raise ConfigError(f"{where}: heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
        dim = _positive(d, "dim", where)
        qt = d.get("q_temp")
        if qt:
            qt = QueryTemperature(_number(qt, "coef", where, positive=False), _positive(qt, "every", where))
        cap = d.get("softcap")
        return cls(heads, kv_heads, dim, _positive(d, "vdim", where) if d.get("vdim") is not None else dim,
                   _number(d, "scale", where), _number(d, "softcap", where) if cap is not None else None,
                   qt or None, _window(d, where))

    def to_dict(self) -> dict[str, Any]:
        out = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
               "q_temp": self.q_temp.to_dict() if self.q_temp else None, "scale": self.scale,
               "softcap": self.softcap, "vdim": self.vdim}
        if self.window:
            out["mask"] = {"size": self.window}
        return out


@dataclass(frozen=True)
class LatentAttentionConfig:
    """Per head ``dim`` plain and ``rot_dim`` rotated query/key elements and ``vdim`` value
    elements, all keys and values read out of a latent of ``kv_rank`` elements.  ``window``:
    keys a query sees, itself included (``None``: all)."""

    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    window: int | None
    rot: RotaryConfig | None

    @classmethod
    def from_dict(cls, d: dict[str, Any], where: str) -> "LatentAttentionConfig":
        rot_dim = d.get("rot_dim") or 0
        if not isinstance(rot_dim, int) or isinstance(rot_dim, bool) or rot_dim < 0:
            raise ConfigError(f"{where}: 'rot_dim' must be a non-negative integer, got {rot_dim!r}")
        dim = d.get("dim") or 0
        if not isinstance(dim, int) or isinstance(dim, bool) or dim < 0 or dim + rot_dim <= 0:
            raise ConfigError(f"{where}: 'dim' and 'rot_dim' must be non-negative integers with a positive sum")
        rot = d.get("rot")
        rot = RotaryConfig.from_dict(rot, where) if rot else None
        if rot is not None and rot.dims > rot_dim:
            raise ConfigError(f"{where}: rot.dims ({rot.dims}) exceeds rot_dim ({rot_dim})")
        if rot_dim + _positive(d, "kv_rank", where) > 256:
            raise ConfigError(f"{where}: rot_dim + kv_rank must not exceed 256 (the attention kernels' head size)")
        return cls(_positive(d, "heads", where), dim, rot_dim, _positive(d, "vdim", where),
                   _positive(d, "kv_rank", where), _number(d, "scale", where), _window(d, where), rot)

    def to_dict(self) -> dict[str, Any]:
        return {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank,
                "mask": {"size": self.window} if self.window else None,
                "rot": ({"base": self.rot.base, "dims": self.rot.dims} if self.rot else None),
                "rot_dim": self.rot_dim, "scale": self.scale, "vdim": self.vdim}


@dataclass(frozen=True)
class DecayMemoryConfig:
    """``decay_rank``: rows of the first of the two small matrices behind the decay; a file may
    leave it out, and the checkpoint's tensor then decides it."""

    heads: int
    dim: int
    decay_rank: int | None = None

    @classmethod
    def from_dict(cls, d: dict[str, Any], where: str) -> "DecayMemoryConfig":
        dim = _positive(d, "dim", where)
        if dim > 256:
            raise ConfigError(f"{where}: wkv heads of more than 256 elements are not supported, got {dim}")
        rank = d.get("decay_rank")
        return cls(_positive(d, "heads", where), dim, _positive(d, "decay_rank", where) if rank is not None else None)

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"dim": self.dim, "heads": self.heads}
        if self.decay_rank is not None:
            out["decay_rank"] = self.decay_rank
        return out


@dataclass(frozen=True)
class DenseFfConfig:
    ff: int
    kind: str = "dense"

    @classmethod
    def from_dict(cls, d: dict[str, Any], where: str) -> "DenseFfConfig":
        kind = _require(d, "kind")
        if kind != "dense":
            raise ConfigError(f"{where}: feed-forward kind {kind!r} is not supported (known: ('dense',))")
        return cls(_positive(d, "ff", where))

    def to_dict(self) -> dict[str, Any]:
        return {"ff": self.ff, "kind": self.kind}


@dataclass(frozen=True)
class BuzinexLayerConfig:
    type: str
    mixer: "CappedAttentionConfig | LatentAttentionConfig | DecayMemoryConfig"
    mlp: DenseFfConfig | None

    MIXERS = {"attention": CappedAttentionConfig, "latent_attention": LatentAttentionConfig,
              "wkv": DecayMemoryConfig}

    @classmethod
    def from_dict(cls, d: dict[str, Any], index: int) -> "BuzinexLayerConfig":
        where = f"layer {index}"
        kind = _require(d, "type")
        if kind not in cls.MIXERS:
            raise ConfigError(f"{where}: mixer type {kind!r} is not supported (known: {tuple(cls.MIXERS)})")
        mlp = d.get("mlp")
        return cls(kind, cls.MIXERS[kind].from_dict(_require(d, "mixer"), where),
                   DenseFfConfig.from_dict(mlp, where) if mlp is not None else None)

    def to_dict(self) -> dict[str, Any]:
        return {"mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None,
                "type": self.type}


@dataclass
class BuzinexConfig(ModelConfig):
    """``vocab_size`` of the base class is the file's ``vocab``."""

    width: int = 0
    norm_eps: float = 0.0
    embedding_scale: float = 1.0
    logit_scale: float = 1.0
    logit_softcap: float | None = None
    layers: list[BuzinexLayerConfig] = field(default_factory=list)

    NAME = "Buzinex"

    def __post_init__(self) -> None:
        if self.width <= 0 or self.vocab_size <= 0 or self.max_position_embeddings <= 0:
            raise ConfigError("vocab, width and max_positions must be positive")
        if not self.layers:
            raise ConfigError("a model needs at least one layer")

    @classmethod
    def from_dict(cls, d: dict[str, Any]) -> "BuzinexConfig":
        layers = _require(d, "layers")
        if not isinstance(layers, list):
            raise ConfigError("'layers' must be a list")
        emb, cap = d.get("embedding") or {}, d.get("logit_softcap")
        return cls(
            architecture=cls.NAME,
            vocab_size=_positive(d, "vocab", "config.json"),
            max_position_embeddings=(_positive(d, "max_positions", "config.json")
                                     if d.get("max_positions") is not None else DEFAULT_MAX_POSITIONS),
            bos_token_id=d.get("bos_token_id"), eos_token_id=d.get("eos_token_id"),
            width=_positive(d, "width", "config.json"),
            norm_eps=_number(_require(d, "norm"), "eps", "norm", positive=False),
            embedding_scale=_number(emb, "scale", "embedding", positive=False) if "scale" in emb else 1.0,
            logit_scale=_number(d, "logit_scale", "config.json") if d.get("logit_scale") is not None else 1.0,
            logit_softcap=_number(d, "logit_softcap", "config.json") if cap is not None else None,
            layers=[BuzinexLayerConfig.from_dict(x, i) for i, x in enumerate(layers)])

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "architecture": self.NAME,
            "embedding": {"scale": self.embedding_scale},
            "layers": [x.to_dict() for x in self.layers],
            "logit_scale": self.logit_scale,
            "logit_softcap": self.logit_softcap,
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
