"""Typed configuration of the Rudorax decoder, read from its own ``config.json`` keys.

A Rudorax ``config.json`` names its model with ``"architecture": "Rudorax"`` and describes every
layer by itself under ``"layers"``: ``type`` (``"attention"`` or ``"mlstm"``), ``mixer`` (that
mixer's sizes and constants) and ``mlp`` (a feed-forward of routed experts, or ``null`` for
none).  Top-level keys: ``vocab``, ``width``, ``norm.eps``, ``embedding.scale``,
``logit_softcap`` (absent or ``null``: none) and ``loop`` (``start``, ``stop``, ``times``: the
layers ``start..stop-1`` are gone through ``times`` times in a row with the same weights;
absent: every layer once).  The design has no position limit of its own; ``max_positions`` may
be given, and is otherwise ``DEFAULT_MAX_POSITIONS``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any

from kvforge_amd.config.fogorax import _positive
from kvforge_amd.config.model import ConfigError, ModelConfig, _require

DEFAULT_MAX_POSITIONS = 131072


def _number(d: dict[str, Any], key: str, where: str, positive: bool = True) -> float:
    v = _require(d, key)
    if isinstance(v, bool) or not isinstance(v, (int, float)) or (positive and not v > 0):
        raise ConfigError(f"{where}: {key!r} must be a {'positive ' if positive else ''}number, got {v!r}")
    return float(v)


@dataclass(frozen=True)
class YarnScaling:
    """Frequencies stretched by ``factor`` where a pair turns fewer than ``slow`` times over
    ``original`` positions, kept where it turns more than ``fast`` times, blended between."""

    factor: float
    original: int
    fast: float
    slow: float

    @classmethod
    def from_dict(cls, d: dict[str, Any], where: str) -> "YarnScaling":
        return cls(_number(d, "factor", where), _positive(d, "original", where),
                   _number(d, "fast", where), _number(d, "slow", where))

    def to_dict(self) -> dict[str, Any]:
        return {"factor": self.factor, "fast": self.fast, "original": self.original, "slow": self.slow}


@dataclass(frozen=True)
class RotaryConfig:
    """Rotation of neighbouring pairs over the first ``dims`` elements of a head."""

    base: float
    dims: int
    scaling: YarnScaling | None = None

    @classmethod
    def from_dict(cls, d: dict[str, Any], where: str) -> "RotaryConfig":
        dims = _positive(d, "dims", where)
        if dims % 2:
            raise ConfigError(f"{where}: rot.dims must be even, got {dims}")
        sc = d.get("scaling")
        return cls(_number(d, "base", where), dims, YarnScaling.from_dict(sc, where) if sc else None)

    def to_dict(self) -> dict[str, Any]:
        return {"base": self.base, "dims": self.dims,
                "scaling": self.scaling.to_dict() if self.scaling else None}


@dataclass(frozen=True)
class SinkAttentionConfig:
    """``window``: keys a query sees, itself included (``None``: all).  A file may leave out
    ``kv_heads`` (then as many as ``heads``), ``vdim`` (then ``dim``), ``rot`` (no rotation) and
    ``mask`` (no window)."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int | None
    rot: RotaryConfig | None

    @classmethod
    def from_dict(cls, d: dict[str, Any], where: str) -> "SinkAttentionConfig":
        heads = _positive(d, "heads", where)
        kv_heads = _positive(d, "kv_heads", where) if d.get("kv_heads") is not None else heads
        if heads % kv_heads:
            raise ConfigError(f"{where}: heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
        dim = _positive(d, "dim", where)
        vdim = _positive(d, "vdim", where) if d.get("vdim") is not None else dim
        mask, rot = d.get("mask"), d.get("rot")
        rot = RotaryConfig.from_dict(rot, where) if rot else None
        if rot is not None and rot.dims > dim:
            raise ConfigError(f"{where}: rot.dims ({rot.dims}) exceeds the head size ({dim})")
        return cls(heads, kv_heads, dim, vdim, _number(d, "scale", where),
                   _positive(mask, "size", where) if mask else None, rot)

    def to_dict(self) -> dict[str, Any]:
        return {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
                "mask": {"size": self.window} if self.window else None,
                "rot": self.rot.to_dict() if self.rot else None, "scale": self.scale, "vdim": self.vdim}


@dataclass(frozen=True)
class MatrixLstmConfig:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @classmethod
    def from_dict(cls, d: dict[str, Any], where: str) -> "MatrixLstmConfig":
        dim = _positive(d, "dim", where)
        return cls(_positive(d, "heads", where), dim,
                   _positive(d, "vdim", where) if d.get("vdim") is not None else dim,
                   _number(d, "gate_cap", where))

    def to_dict(self) -> dict[str, Any]:
        return {"dim": self.dim, "gate_cap": self.gate_cap, "heads": self.heads, "vdim": self.vdim}


@dataclass(frozen=True)
class RoutedMlpConfig:
    """``experts`` feed-forwards of width ``ff`` of which a token uses ``top``; the router has
    ``experts + identity`` outputs, the last ``identity`` of which pass the input on;
    ``shared_ff``: width of an expert that every token uses (0: none)."""

    ff: int
    experts: int
    top: int
    identity: int = 0
    shared_ff: int = 0
    kind: str = "moe"

    @classmethod
    def from_dict(cls, d: dict[str, Any], where: str) -> "RoutedMlpConfig":
        kind = _require(d, "kind")
        if kind != "moe":
            raise ConfigError(f"{where}: feed-forward kind {kind!r} is not supported (known: ('moe',))")
        r = _require(d, "router")
        experts, top = _positive(r, "experts", where), _positive(r, "top", where)
        identity = r.get("identity") or 0
        if not isinstance(identity, int) or identity < 0:
            raise ConfigError(f"{where}: router.identity must be a non-negative integer, got {identity!r}")
        if top > experts + identity:
            raise ConfigError(f"{where}: router.top ({top}) exceeds the router's {experts + identity} outputs")
        shared = d.get("shared")
        return cls(_positive(_require(d, "expert"), "ff", where), experts, top, identity,
                   _positive(shared, "ff", where) if shared else 0)

    def to_dict(self) -> dict[str, Any]:
        return {"expert": {"ff": self.ff}, "kind": self.kind,
                "router": {"experts": self.experts, "identity": self.identity, "top": self.top},
                "shared": {"ff": self.shared_ff} if self.shared_ff else None}


@dataclass(frozen=True)
class RudoraxLayerConfig:
    type: str
    mixer: "SinkAttentionConfig | MatrixLstmConfig"
    mlp: RoutedMlpConfig | None

    MIXERS = {"attention": SinkAttentionConfig, "mlstm": MatrixLstmConfig}

    @classmethod
    def from_dict(cls, d: dict[str, Any], index: int) -> "RudoraxLayerConfig":
        where = f"layer {index}"
        kind = _require(d, "type")
        if kind not in cls.MIXERS:
            raise ConfigError(f"{where}: mixer type {kind!r} is not supported (known: {tuple(cls.MIXERS)})")
        mlp = d.get("mlp")
        return cls(kind, cls.MIXERS[kind].from_dict(_require(d, "mixer"), where),
                   RoutedMlpConfig.from_dict(mlp, where) if mlp is not None else None)

    def to_dict(self) -> dict[str, Any]:
        return {"mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None,
                "type": self.type}


@dataclass(frozen=True)
class LayerLoop:
    start: int
    stop: int
    times: int

    def to_dict(self) -> dict[str, Any]:
        return {"start": self.start, "stop": self.stop, "times": self.times}


@dataclass
class RudoraxConfig(ModelConfig):
    """``vocab_size`` of the base class is the file's ``vocab``."""

    width: int = 0
    norm_eps: float = 0.0
    embedding_scale: float = 1.0
    logit_softcap: float | None = None
    loop: LayerLoop | None = None
    layers: list[RudoraxLayerConfig] = field(default_factory=list)

    NAME = "Rudorax"

    def __post_init__(self) -> None:
        if self.width <= 0 or self.vocab_size <= 0 or self.max_position_embeddings <= 0:
            raise ConfigError("vocab, width and max_positions must be positive")
        if not self.layers:
            raise ConfigError("a model needs at least one layer")
        if self.loop is not None:
            lp = self.loop
            if not 0 <= lp.start <= lp.stop <= len(self.layers) or lp.times < 1:
                raise ConfigError(f"loop {lp} does not fit {len(self.layers)} layers")

    def run_order(self) -> list[int]:
        """The layers in the order they run, a looped stretch as often as it is gone through."""
        n = len(self.layers)
        if self.loop is None:
            return list(range(n))
        lp = self.loop
        return list(range(lp.start)) + list(range(lp.start, lp.stop)) * lp.times + list(range(lp.stop, n))

    @classmethod
    def from_dict(cls, d: dict[str, Any]) -> "RudoraxConfig":
        layers = _require(d, "layers")
        if not isinstance(layers, list):
            raise ConfigError("'layers' must be a list")
        emb, loop, cap = d.get("embedding") or {}, d.get("loop"), d.get("logit_softcap")
        if loop:
            for key in ("start", "stop", "times"):
                if not isinstance(loop.get(key), int) or isinstance(loop.get(key), bool):
                    raise ConfigError(f"loop.{key} must be an integer, got {loop.get(key)!r}")
            loop = LayerLoop(loop["start"], loop["stop"], loop["times"])
        return cls(
            architecture=cls.NAME,
            vocab_size=_positive(d, "vocab", "config.json"),
            max_position_embeddings=(_positive(d, "max_positions", "config.json")
                                     if d.get("max_positions") is not None else DEFAULT_MAX_POSITIONS),
            bos_token_id=d.get("bos_token_id"), eos_token_id=d.get("eos_token_id"),
            width=_positive(d, "width", "config.json"),
            norm_eps=_number(_require(d, "norm"), "eps", "norm", positive=False),
            embedding_scale=_number(emb, "scale", "embedding", positive=False) if "scale" in emb else 1.0,
            logit_softcap=_number(d, "logit_softcap", "config.json") if cap is not None else None,
            loop=loop or None,
            layers=[RudoraxLayerConfig.from_dict(x, i) for i, x in enumerate(layers)])

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "architecture": self.NAME,
            "embedding": {"scale": self.embedding_scale},
            "layers": [x.to_dict() for x in self.layers],
            "logit_softcap": self.logit_softcap,
            "loop": self.loop.to_dict() if self.loop else None,
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
