"""Typed configuration of the Fogorax decoder, read from its own ``config.json`` keys.

A Fogorax ``config.json`` names its model with ``"architecture": "Fogorax"`` and describes every
layer by itself under ``"layers"``: ``type`` (which mixer), ``mixer`` (the mixer's sizes and
constants) and ``mlp`` (the feed-forward, or ``null`` for none).  Nothing is inherited from one
layer to the next, so layers may differ in head counts, head sizes, windows and feed-forward
widths.  Top-level keys: ``vocab``, ``width``, ``max_positions`` (rows of the learned position
table), ``norm.eps`` and ``token_side.dim`` (columns of the per-token side table that each layer
owns; absent or ``null``: no per-layer token input).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any

from kvforge_amd.config.model import ConfigError, ModelConfig, _require


def _positive(d: dict[str, Any], key: str, where: str) -> int:
    v = _require(d, key)
    if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
        raise ConfigError(f"{where}: {key!r} must be a positive integer, got {v!r}")
    return v


@dataclass(frozen=True)
class WindowMask:
    """Causal mask with a sliding window and kept first tokens: query ``i`` sees key ``j`` iff
    ``j <= i`` and (``i - j < size`` or ``j < keep_first``)."""

    size: int
    keep_first: int = 0

    @classmethod
    def from_dict(cls, d: dict[str, Any], where: str) -> "WindowMask":
        keep = d.get("keep_first", 0)
        if not isinstance(keep, int) or keep < 0:
            raise ConfigError(f"{where}: 'keep_first' must be a non-negative integer, got {keep!r}")
        return cls(_positive(d, "size", where), keep)

    def to_dict(self) -> dict[str, Any]:
        return {"keep_first": self.keep_first, "size": self.size}


@dataclass(frozen=True)
class AttentionMixerConfig:
    """``kv_from``: the layer whose keys and values this layer reads instead of projecting its
    own (``None``: its own).  A file may leave out ``kv_heads`` (then as many as ``heads``) and
    ``vdim`` (then ``dim``)."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    mask: WindowMask
    kv_from: int | None = None

    @classmethod
    def from_dict(cls, d: dict[str, Any], where: str) -> "AttentionMixerConfig":
        heads = _positive(d, "heads", where)
        kv_heads = _positive(d, "kv_heads", where) if d.get("kv_heads") is not None else heads
        if heads % kv_heads:
            raise ConfigError(f"{where}: heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
        scale = float(_require(d, "scale"))
        if not scale > 0.0:
            raise ConfigError(f"{where}: 'scale' must be positive, got {scale!r}")
        kv_from = d.get("kv_from")
        if kv_from is not None and (not isinstance(kv_from, int) or kv_from < 0):
            raise ConfigError(f"{where}: 'kv_from' must name a layer, got {kv_from!r}")
        dim = _positive(d, "dim", where)
        vdim = _positive(d, "vdim", where) if d.get("vdim") is not None else dim
        return cls(heads, kv_heads, dim, vdim, scale, WindowMask.from_dict(_require(d, "mask"), where), kv_from)

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"dim": self.dim, "heads": self.heads}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        out.update(kv_heads=self.kv_heads, mask=self.mask.to_dict(), scale=self.scale, vdim=self.vdim)
        return out


@dataclass(frozen=True)
class DenseMlpConfig:
    ff: int
    kind: str = "dense"

    def to_dict(self) -> dict[str, Any]:
        return {"ff": self.ff, "kind": self.kind}


@dataclass(frozen=True)
class FogoraxLayerConfig:
    type: str
    mixer: AttentionMixerConfig
    mlp: DenseMlpConfig | None

    MIXERS = ("attention",)
    MLPS = ("dense",)

    @classmethod
    def from_dict(cls, d: dict[str, Any], index: int) -> "FogoraxLayerConfig":
        where = f"layer {index}"
        kind = _require(d, "type")
        if kind not in cls.MIXERS:
            raise ConfigError(f"{where}: mixer type {kind!r} is not supported (known: {cls.MIXERS})")
        mixer = AttentionMixerConfig.from_dict(_require(d, "mixer"), where)
        mlp = d.get("mlp")
        if mlp is not None:
            mk = _require(mlp, "kind")
            if mk not in cls.MLPS:
                raise ConfigError(f"{where}: feed-forward kind {mk!r} is not supported (known: {cls.MLPS})")
            mlp = DenseMlpConfig(_positive(mlp, "ff", where), mk)
        return cls(kind, mixer, mlp)

    def to_dict(self) -> dict[str, Any]:
        return {"mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None,
                "type": self.type}


@dataclass
class FogoraxConfig(ModelConfig):
    """``vocab_size`` and ``max_position_embeddings`` of the base class are the file's ``vocab``
    and ``max_positions``."""

    width: int = 0
    norm_eps: float = 0.0
    side_dim: int = 0          # 0: no per-layer token input
    layers: list[FogoraxLayerConfig] = field(default_factory=list)

    NAME = "Fogorax"

    def __post_init__(self) -> None:
        if self.width <= 0 or self.vocab_size <= 0 or self.max_position_embeddings <= 0:
            raise ConfigError("vocab, width and max_positions must be positive")
        if not self.layers:
            raise ConfigError("a model needs at least one layer")
        for i, layer in enumerate(self.layers):
            j = layer.mixer.kv_from
            if j is None:
                continue
            if not 0 <= j < len(self.layers) or j == i:
                raise ConfigError(f"layer {i}: kv_from names layer {j}, which is not another layer")
            if j > i:
                raise ConfigError(f"layer {i}: kv_from names a later layer ({j}), whose keys do not "
                                  "exist yet when this layer runs")
            src = self.layers[j].mixer
            if src.kv_from is not None:
                raise ConfigError(f"layer {i}: kv_from names layer {j}, which has no keys of its own")
            if (src.kv_heads, src.dim, src.vdim) != (layer.mixer.kv_heads, layer.mixer.dim, layer.mixer.vdim):
                raise ConfigError(f"layer {i} and layer {j} share keys and values but differ in "
                                  "kv_heads, dim or vdim")

    @classmethod
    def from_dict(cls, d: dict[str, Any]) -> "FogoraxConfig":
        norm = _require(d, "norm")
        side = d.get("token_side")
        layers = _require(d, "layers")
        if not isinstance(layers, list):
            raise ConfigError("'layers' must be a list")
        return cls(
            architecture=cls.NAME,
            vocab_size=_positive(d, "vocab", "config.json"),
            max_position_embeddings=_positive(d, "max_positions", "config.json"),
            bos_token_id=d.get("bos_token_id"), eos_token_id=d.get("eos_token_id"),
            width=_positive(d, "width", "config.json"),
            norm_eps=float(_require(norm, "eps")),
            side_dim=_positive(side, "dim", "token_side") if side else 0,
            layers=[FogoraxLayerConfig.from_dict(x, i) for i, x in enumerate(layers)])

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "architecture": self.NAME,
            "layers": [x.to_dict() for x in self.layers],
            "max_positions": self.max_position_embeddings,
            "norm": {"eps": self.norm_eps},
            "token_side": {"dim": self.side_dim} if self.side_dim else None,
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
