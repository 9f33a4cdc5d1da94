"""Configuration of the Mafosun decoder (config.json ``"architecture": "Mafosun"``): a normed token embedding and a list
of layers whose sublayers read the stream itself and whose outputs alone are normed.  A layer's mixer is either
grouped-query attention over a sliding window with pooled blocks of older positions, or two mixers side by side:
chunked attention and retention (linear attention with a fixed decay a head).  Its feed-forward is dense or a set of
routed experts whose choice is limited to the best groups."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from .base import ConfigError, ModelConfig, checked_float, checked_int, end_token_of, required_int

ATTENTION, PARALLEL = "attention", "parallel"
DENSE, MOE = "dense", "moe"


def _int(m: Any, key: str, where: str, minimum: int = 1) -> int:
    if not isinstance(m, Mapping) or key not in m:
        raise ConfigError(f"config.json: {where} has no '{key}'")
    return checked_int(m[key], f"{where}.{key}", minimum)


def _float(m: Any, key: str, where: str, positive: bool = True) -> float:
    if not isinstance(m, Mapping) or key not in m:
        raise ConfigError(f"config.json: {where} has no '{key}'")
    return checked_float(m[key], f"{where}.{key}", positive)


@dataclass(frozen=True)
class RotationConfig:
    """The first ``dims`` values of a head turn at base^(-2i/dims) a position; ``scaling`` = (factor, low, high,
    original) rescales the frequencies by their wavelength, or None."""

    base: float
    dims: int
    scaling: Optional[Tuple[float, float, float, float]] = None

    @classmethod
    def read(cls, raw: Any, where: str, dim: int) -> Optional["RotationConfig"]:
        if raw is None:
            return None
        if not isinstance(raw, Mapping):
            raise ConfigError(f"config.json: {where} must be an object")
        dims = _int(raw, "dims", where, 0)
        if dims == 0:
            return None
        if dims % 2 or dims > dim:
            raise ConfigError(f"config.json: {where}.dims {dims} must be even and at most {dim}")
        scaling, s = None, raw.get("scaling")
        if s is not None:
            scaling = (_float(s, "factor", where + ".scaling"), _float(s, "low", where + ".scaling"),
                       _float(s, "high", where + ".scaling"), _float(s, "original", where + ".scaling"))
            if not scaling[1] < scaling[2]:
                raise ConfigError(f"config.json: {where}.scaling: low {scaling[1]} must be below high {scaling[2]}")
        return cls(_float(raw, "base", where), dims, scaling)

    def to_dict(self) -> dict:
        d: dict = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            d["scaling"] = dict(zip(("factor", "low", "high", "original"), self.scaling))
        return d


@dataclass(frozen=True)
class AttentionConfig:
    """``heads`` query and ``kv_heads`` key/value heads, keys of ``dim`` and values of ``vdim``, scores times ``scale``,
    capped at ``softcap`` (None: not capped).  ``mask_size`` is the window (``windowed``) or the chunk; ``pool`` the
    positions of a pooled block (None: no pooled blocks)."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    mask_size: int
    pool: Optional[int] = None
    softcap: Optional[float] = None
    rot: Optional[RotationConfig] = None

    @classmethod
    def read(cls, m: Any, where: str) -> "AttentionConfig":
        if not isinstance(m, Mapping):
            raise ConfigError(f"config.json: {where} must be an object")
        dim = _int(m, "dim", where)
        mask = m.get("mask")
        pool = mask.get("pool") if isinstance(mask, Mapping) else None
        cap = m.get("softcap")
        cfg = cls(heads=_int(m, "heads", where), kv_heads=_int(m, "kv_heads", where), dim=dim, vdim=_int(m, "vdim", where),
                  scale=_float(m, "scale", where), mask_size=_int(mask, "size", where + ".mask"),
                  pool=None if pool is None else checked_int(pool, f"{where}.mask.pool", 1),
                  softcap=None if cap is None else checked_float(cap, f"{where}.softcap"),
                  rot=RotationConfig.read(m.get("rot"), where + ".rot", dim))
        if cfg.heads % cfg.kv_heads:
            raise ConfigError(f"config.json: {where}: heads {cfg.heads} must be a multiple of kv_heads {cfg.kv_heads}")
        return cfg

    def to_dict(self) -> dict:
        d: dict = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
                   "mask": {"size": self.mask_size}}
        if self.pool is not None:
            d["mask"]["pool"] = self.pool
        if self.softcap is not None:
            d["softcap"] = self.softcap
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        return d


@dataclass(frozen=True)
class RetentionConfig:
    """``heads`` heads with a state of ``dim`` x ``vdim`` and a fixed ``decay`` each."""

    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    rot: Optional[RotationConfig] = None

    @classmethod
    def read(cls, m: Any, where: str) -> "RetentionConfig":
        if not isinstance(m, Mapping):
            raise ConfigError(f"config.json: {where} must be an object")
        heads, dim = _int(m, "heads", where), _int(m, "dim", where)
        decay = m.get("decay")
        if not isinstance(decay, list) or len(decay) != heads:
            raise ConfigError(f"config.json: {where}.decay must list one decay for each of the {heads} heads")
        decay = tuple(checked_float(d, f"{where}.decay[{i}]") for i, d in enumerate(decay))
        if any(d > 1.0 for d in decay):
            raise ConfigError(f"config.json: {where}.decay: a decay is at most 1")
        return cls(heads, dim, _int(m, "vdim", where), decay, RotationConfig.read(m.get("rot"), where + ".rot", dim))

    def to_dict(self) -> dict:
        d: dict = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay)}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        return d


@dataclass(frozen=True)
class ParallelConfig:
    """Chunked attention (``left``) and retention (``right``) side by side; the result is their weighted sum."""

    left: AttentionConfig
    right: RetentionConfig
    left_scale: float
    right_scale: float

    def to_dict(self) -> dict:
        return {"left": self.left.to_dict(), "right": self.right.to_dict(), "left_scale": self.left_scale,
                "right_scale": self.right_scale}


@dataclass(frozen=True)
class FeedForwardConfig:
    """``kind`` dense: one gated feed-forward of width ``ff``.  moe: ``experts`` of width ``ff`` of which a token uses
    ``top``, chosen among the experts of the ``keep`` best of ``groups`` equal groups of neighbours."""

    kind: str
    ff: int
    experts: int = 0
    top: int = 0
    groups: int = 1
    keep: int = 1

    @classmethod
    def read(cls, m: Any, where: str) -> Optional["FeedForwardConfig"]:
        if m is None:
            return None
        if not isinstance(m, Mapping) or m.get("kind") not in (DENSE, MOE):
            raise ConfigError(f"config.json: {where} must be null or a feed-forward of kind '{DENSE}' or '{MOE}'")
        if m["kind"] == DENSE:
            return cls(DENSE, _int(m, "ff", where))
        router = m.get("router")
        experts, top = _int(router, "experts", where + ".router"), _int(router, "top", where + ".router")
        g = router.get("groups")
        groups, keep = (1, 1) if g is None else (_int(g, "count", where + ".router.groups"), _int(g, "keep", where + ".router.groups"))
        if experts % groups or keep > groups or top > keep * (experts // groups):
            raise ConfigError(f"config.json: {where}.router: {experts} experts in {groups} groups of which {keep} are kept "
                              f"do not give {top} choices")
        return cls(MOE, _int(m.get("expert"), "ff", where + ".expert"), experts, top, groups, keep)

    def to_dict(self) -> dict:
        if self.kind == DENSE:
            return {"kind": DENSE, "ff": self.ff}
        return {"kind": MOE, "expert": {"ff": self.ff},
                "router": {"experts": self.experts, "top": self.top, "groups": {"count": self.groups, "keep": self.keep}}}


@dataclass(frozen=True)
class LayerConfig:
    kind: str                           # ATTENTION or PARALLEL
    mixer: object                       # AttentionConfig or ParallelConfig
    mlp: Optional[FeedForwardConfig]    # None: the layer has no feed-forward

    def to_dict(self) -> dict:
        return {"type": self.kind, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class MafosunConfig(ModelConfig):
    width: int = 0
    vocab: int = 0
    norm_eps: float = 1e-5
    layers: Tuple[LayerConfig, ...] = ()
    eos_token_id: int = -1

    @property
    def end_token(self) -> int:
        return self.eos_token_id

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "MafosunConfig":
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers = []
        for i, entry in enumerate(layers_raw):
            where = f"layers[{i}]"
            if not isinstance(entry, dict) or not isinstance(entry.get("mixer"), dict):
                raise ConfigError(f"config.json: {where} must be an object with a 'mixer'")
            kind, m = entry.get("type"), entry["mixer"]
            if kind == ATTENTION:
                mixer = AttentionConfig.read(m, where + ".mixer")
            elif kind == PARALLEL:
                mixer = ParallelConfig(AttentionConfig.read(m.get("left"), where + ".mixer.left"),
                                       RetentionConfig.read(m.get("right"), where + ".mixer.right"),
                                       _float(m, "left_scale", where + ".mixer", positive=False),
                                       _float(m, "right_scale", where + ".mixer", positive=False))
                if mixer.left.pool is not None or mixer.left.rot is not None or mixer.left.softcap is not None:
                    raise ConfigError(f"config.json: {where}.mixer.left is chunked attention: no pooled blocks, rotation or cap")
            else:
                raise ConfigError(f"config.json: {where}.type '{kind}' is not a mixer of this architecture "
                                  f"({ATTENTION}, {PARALLEL})")
            layers.append(LayerConfig(kind, mixer, FeedForwardConfig.read(entry.get("mlp"), where + ".mlp")))
        norm = raw.get("norm") or {}
        return cls(architecture="Mafosun", width=required_int(raw, "width"), vocab=required_int(raw, "vocab"),
                   norm_eps=checked_float(norm.get("eps", 1e-5), "norm.eps", positive=False),
                   layers=tuple(layers), eos_token_id=end_token_of(raw))

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "width": self.width, "vocab": self.vocab, "norm": {"eps": self.norm_eps},
             "layers": [layer.to_dict() for layer in self.layers]}
        if self.eos_token_id >= 0:
            d["eos_token_id"] = self.eos_token_id
        return d
