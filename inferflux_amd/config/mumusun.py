"""Configuration of the Mumusun decoder, from its config.json.

The file is nested: the model's own sizes at the top (``vocab``, ``width``, ``norm.eps``) and a list
``layers`` whose entries each give the layer's ``type`` (its mixer), the mixer's sizes and constants
(``mixer``) and its feed-forward (``mlp``, or null for a layer without one).  Layers need not be alike:
every layer carries its own sizes, window and constants, and the plan is built layer by layer.

    mixer   heads, dim (unrotated query/key size per head), rot_dim (rotated size per head), vdim, q_rank,
            kv_rank, scale (the factor on the scores), rot.base / rot.dims (the rotation's base and how many of
            the rot_dim dimensions turn), mask.size (how many positions, its own included, a query sees; absent
            or null: all before it)
    mlp     kind "moe": expert.ff, router.experts / top / groups.count / groups.keep

A missing or mistyped key is an error that names it by its path.
"""
from __future__ import annotations

import dataclasses
from typing import Any, ClassVar, Dict, Mapping, Optional, Tuple

from .base import ConfigError, ModelConfig, read_key

MIXER_TYPES = ("latent_attention",)
MLP_KINDS = ("moe",)


def _section(d: Mapping[str, Any], key: str, where: str, optional: bool = False) -> Optional[Mapping[str, Any]]:
    v = d.get(key)
    if v is None:
        if optional:
            return None
        raise ConfigError(f"config.json: required section '{where}{key}' is missing")
    if not isinstance(v, dict):
        raise ConfigError(f"config.json: '{where}{key}' must be an object, got {v!r}")
    return v


def _read(d: Mapping[str, Any], key: str, kind, where: str, *default):
    try:
        return read_key(d, key, kind, *default)
    except ConfigError as e:
        raise ConfigError(str(e).replace(f"'{key}'", f"'{where}{key}'")) from None


@dataclasses.dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int
    window: Optional[int]

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "LatentAttentionConfig":
        rot = _section(d, "rot", where)
        mask = _section(d, "mask", where, optional=True)
        rot_dim = _read(d, "rot_dim", int, where)
        return cls(
            heads=_read(d, "heads", int, where), dim=_read(d, "dim", int, where), rot_dim=rot_dim,
            vdim=_read(d, "vdim", int, where), q_rank=_read(d, "q_rank", int, where),
            kv_rank=_read(d, "kv_rank", int, where), scale=_read(d, "scale", float, where),
            rot_base=_read(rot, "base", float, where + "rot."), rot_dims=_read(rot, "dims", int, where + "rot.", rot_dim),
            window=_read(mask, "size", int, where + "mask.", None) if mask is not None else None)

    def to_dict(self) -> Dict[str, Any]:
        out = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "q_rank": self.q_rank,
               "kv_rank": self.kv_rank, "scale": self.scale, "rot": {"base": self.rot_base, "dims": self.rot_dims}}
        if self.window is not None:
            out["mask"] = {"size": self.window}
        return out

    def validate(self, where: str) -> None:
        for name in ("heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"config.json: '{where}{name}' must be positive, got {getattr(self, name)}")
        if self.rot_dims <= 0 or self.rot_dims % 2 or self.rot_dims > self.rot_dim:
            raise ConfigError(f"config.json: '{where}rot.dims' = {self.rot_dims} must be even and within rot_dim {self.rot_dim}")
        if not self.rot_base > 0:
            raise ConfigError(f"config.json: '{where}rot.base' must be positive, got {self.rot_base}")
        if self.window is not None and self.window <= 0:
            raise ConfigError(f"config.json: '{where}mask.size' must be positive, got {self.window}")


@dataclasses.dataclass(frozen=True)
class MoEConfig:
    ff: int
    experts: int
    top: int
    groups: int
    keep_groups: int

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "MoEConfig":
        kind = _read(d, "kind", str, where, "moe")
        if kind not in MLP_KINDS:
            raise ConfigError(f"config.json: '{where}kind' = '{kind}' is not supported (one of {MLP_KINDS})")
        expert, router = _section(d, "expert", where), _section(d, "router", where)
        groups = _section(router, "groups", where + "router.", optional=True) or {}
        return cls(ff=_read(expert, "ff", int, where + "expert."), experts=_read(router, "experts", int, where + "router."),
                   top=_read(router, "top", int, where + "router."),
                   groups=_read(groups, "count", int, where + "router.groups.", 1),
                   keep_groups=_read(groups, "keep", int, where + "router.groups.", 1))

    def to_dict(self) -> Dict[str, Any]:
        return {"kind": "moe", "expert": {"ff": self.ff},
                "router": {"experts": self.experts, "top": self.top, "groups": {"count": self.groups, "keep": self.keep_groups}}}

    def validate(self, where: str) -> None:
        for name in ("ff", "experts", "top", "groups", "keep_groups"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"config.json: '{where}{name}' must be positive, got {getattr(self, name)}")
        if self.experts % self.groups:
            raise ConfigError(f"config.json: '{where}router.experts' = {self.experts} is not a multiple of groups.count {self.groups}")
        if self.keep_groups > self.groups:
            raise ConfigError(f"config.json: '{where}router.groups.keep' = {self.keep_groups} exceeds groups.count {self.groups}")
        if self.top > self.keep_groups * (self.experts // self.groups):
            raise ConfigError(f"config.json: '{where}router.top' = {self.top} exceeds the {self.keep_groups} x "
                              f"{self.experts // self.groups} experts of the groups that are kept")


@dataclasses.dataclass(frozen=True)
class MumusunLayer:
    type: str
    mixer: LatentAttentionConfig
    mlp: Optional[MoEConfig]

    def to_dict(self) -> Dict[str, Any]:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp is not None else None}


@dataclasses.dataclass(frozen=True)
class MumusunConfig(ModelConfig):
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[MumusunLayer, ...]
    # The file names no longest sequence: positions are formed in 32-bit floats like every other angle of the
    # engine, which counts integers exactly up to 2^24.
    max_positions: int = 1 << 24

    model_type: ClassVar[str] = "mumusun"
    architectures: ClassVar[Tuple[str, ...]] = ("Mumusun",)

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "MumusunConfig":
        layers_in = d.get("layers")
        if not isinstance(layers_in, list) or not layers_in:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for i, L in enumerate(layers_in):
            where = f"layers[{i}]."
            if not isinstance(L, dict):
                raise ConfigError(f"config.json: 'layers[{i}]' must be an object")
            kind = _read(L, "type", str, where)
            if kind not in MIXER_TYPES:
                raise ConfigError(f"config.json: '{where}type' = '{kind}' is not a known mixer (one of {MIXER_TYPES})")
            mixer = LatentAttentionConfig.from_dict(_section(L, "mixer", where), where + "mixer.")
            mlp = _section(L, "mlp", where, optional=True)
            layers.append(MumusunLayer(kind, mixer, MoEConfig.from_dict(mlp, where + "mlp.") if mlp is not None else None))
        norm = _section(d, "norm", "")
        cfg = cls(vocab=read_key(d, "vocab", int), width=read_key(d, "width", int), norm_eps=_read(norm, "eps", float, "norm."),
                  layers=tuple(layers), max_positions=read_key(d, "max_positions", int, 1 << 24))
        cfg.validate()
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        out = {"architecture": self.architectures[0], "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "layers": [L.to_dict() for L in self.layers]}
        if self.max_positions != 1 << 24:
            out["max_positions"] = self.max_positions
        return out

    def validate(self) -> None:
        for name in ("vocab", "width", "max_positions"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"config.json: '{name}' must be positive, got {getattr(self, name)}")
        if not self.norm_eps >= 0:
            raise ConfigError(f"config.json: 'norm.eps' must be >= 0, got {self.norm_eps}")
        for i, L in enumerate(self.layers):
            L.mixer.validate(f"layers[{i}].mixer.")
            if L.mlp is not None:
                L.mlp.validate(f"layers[{i}].mlp.")
