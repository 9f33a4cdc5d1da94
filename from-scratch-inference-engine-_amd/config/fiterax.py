"""Configuration of the Fiterax decoder (config.json ``"architecture": "Fiterax"``): a scaled token embedding, a list
of layers whose mixer (grouped-query attention with capped scores, or an mLSTM matrix memory) and feed-forward of
routed experts read the same stream side by side, each through an RMS norm in groups and a short causal convolution;
the sublayers' sum is added with a constant factor."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from .base import ConfigError, ModelConfig, checked_float, checked_int, end_token_of, required_int

ATTENTION, MLSTM = "attention", "mlstm"


def _int(m: Mapping, key: str, where: str, minimum: int = 1) -> int:
    if not isinstance(m, Mapping) or key not in m:
        raise ConfigError(f"config.json: {where} has no '{key}'")
    return checked_int(m[key], f"{where}.{key}", minimum)


@dataclass(frozen=True)
class AttentionConfig:
    """``heads`` query and ``kv_heads`` key/value heads, keys of ``dim`` and values of ``vdim``; the first ``rot_dims``
    values of a head turn (value i with value i + rot_dims / 2) at rot_base^(-2i/rot_dims) a position; scores times
    ``scale`` (and the head's temperature), capped at ``softcap`` (None: not capped)."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: Optional[float]
    rot_base: float
    rot_dims: int

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
             "rot": {"base": self.rot_base, "dims": self.rot_dims}}
        if self.softcap is not None:
            d["softcap"] = self.softcap
        return d


@dataclass(frozen=True)
class MLSTMConfig:
    """``heads`` heads with a memory of ``dim`` x ``vdim``; gate logits capped at ``gate_cap``."""

    heads: int
    dim: int
    vdim: int
    gate_cap: float

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


@dataclass(frozen=True)
class ExpertsConfig:
    """``experts`` feed-forward layers of width ``ff`` of which a token uses ``top``; routing weights times ``scale``."""

    ff: int
    experts: int
    top: int
    scale: float

    def to_dict(self) -> dict:
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top, "scale": self.scale}}


@dataclass(frozen=True)
class LayerConfig:
    kind: str                      # ATTENTION or MLSTM
    mixer: object
    mlp: Optional[ExpertsConfig]   # None: the layer has no feed-forward

    def to_dict(self) -> dict:
        return {"type": self.kind, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class FiteraxConfig(ModelConfig):
    width: int = 0
    vocab: int = 0
    norm_eps: float = 1e-5
    norm_groups: int = 1
    embedding_scale: float = 1.0
    residual_mult: float = 1.0
    canon_taps: int = 1
    layers: Tuple[LayerConfig, ...] = ()
    eos_token_id: int = -1

    @property
    def end_token(self) -> int:
        return self.eos_token_id

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "FiteraxConfig":
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        width = required_int(raw, "width")
        layers = []
        for i, entry in enumerate(layers_raw):
            where = f"layers[{i}]"
            if not isinstance(entry, dict) or not isinstance(entry.get("mixer"), dict):
                raise ConfigError(f"config.json: {where} must be an object with a 'mixer'")
            kind, m = entry.get("type"), entry["mixer"]
            if kind == ATTENTION:
                dim = _int(m, "dim", where)
                rot = m.get("rot") or {}
                if not isinstance(rot, dict):
                    raise ConfigError(f"config.json: {where}.rot must be an object")
                rot_dims = checked_int(rot.get("dims", 0), f"{where}.rot.dims", 0)
                if rot_dims % 2 or rot_dims > dim:
                    raise ConfigError(f"config.json: {where}.rot.dims {rot_dims} must be even and at most {dim}")
                cap = m.get("softcap")
                mixer = AttentionConfig(
                    heads=_int(m, "heads", where), kv_heads=_int(m, "kv_heads", where), dim=dim, vdim=_int(m, "vdim", where),
                    scale=checked_float(m.get("scale"), f"{where}.scale"),
                    softcap=None if cap is None else checked_float(cap, f"{where}.softcap"),
                    rot_base=checked_float(rot.get("base", 10000.0), f"{where}.rot.base") if rot_dims else 10000.0,
                    rot_dims=rot_dims)
                if mixer.heads % mixer.kv_heads:
                    raise ConfigError(f"config.json: {where}: heads {mixer.heads} must be a multiple of kv_heads {mixer.kv_heads}")
            elif kind == MLSTM:
                mixer = MLSTMConfig(heads=_int(m, "heads", where), dim=_int(m, "dim", where), vdim=_int(m, "vdim", where),
                                    gate_cap=checked_float(m.get("gate_cap"), f"{where}.gate_cap"))
            else:
                raise ConfigError(f"config.json: {where}.type '{kind}' is not a mixer of this architecture "
                                  f"({ATTENTION}, {MLSTM})")
            mlp_raw, mlp = entry.get("mlp"), None
            if mlp_raw is not None:
                if not isinstance(mlp_raw, dict) or mlp_raw.get("kind") != "moe":
                    raise ConfigError(f"config.json: {where}.mlp must be null or a feed-forward of kind 'moe'")
                router = mlp_raw.get("router")
                if not isinstance(router, dict):
                    raise ConfigError(f"config.json: {where}.mlp has no 'router'")
                mlp = ExpertsConfig(ff=_int(mlp_raw.get("expert"), "ff", where + ".mlp.expert"),
                                    experts=_int(router, "experts", where + ".mlp.router"),
                                    top=_int(router, "top", where + ".mlp.router"),
                                    scale=checked_float(router.get("scale", 1.0), f"{where}.mlp.router.scale"))
                if mlp.top > mlp.experts:
                    raise ConfigError(f"config.json: {where}.mlp.router: top {mlp.top} of {mlp.experts} experts")
            layers.append(LayerConfig(kind, mixer, mlp))
        norm = raw.get("norm") or {}
        groups = checked_int(norm.get("groups", 1), "norm.groups", 1)
        if width % groups:
            raise ConfigError(f"config.json: norm.groups {groups} does not divide width {width}")
        return cls(architecture="Fiterax", width=width, vocab=required_int(raw, "vocab"),
                   norm_eps=checked_float(norm.get("eps", 1e-5), "norm.eps", positive=False), norm_groups=groups,
                   embedding_scale=checked_float((raw.get("embedding") or {}).get("scale", 1.0), "embedding.scale"),
                   residual_mult=checked_float(raw.get("residual_mult", 1.0), "residual_mult"),
                   canon_taps=checked_int((raw.get("canon") or {}).get("taps", 1), "canon.taps", 1),
                   layers=tuple(layers), eos_token_id=end_token_of(raw))

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "width": self.width, "vocab": self.vocab,
             "norm": {"eps": self.norm_eps, "groups": self.norm_groups}, "embedding": {"scale": self.embedding_scale},
             "residual_mult": self.residual_mult, "canon": {"taps": self.canon_taps},
             "layers": [layer.to_dict() for layer in self.layers]}
        if self.eos_token_id >= 0:
            d["eos_token_id"] = self.eos_token_id
        return d
