"""Configuration of the Podurax decoder, from its config.json.

The file is nested: the model's own sizes and constants at the top (``vocab``, ``width``, ``norm.eps``,
``embedding.scale``, ``residual_mult``) and a list ``layers`` whose entries each give the layer's ``type`` (its
mixer: "attention" or "mamba1"), the mixer's sizes and constants (``mixer``) and its feed-forward (``mlp``, or null
for a layer without one).  Layers need not be alike: the plan is built layer by layer.

    attention   heads, kv_heads, dim (query/key size per head), vdim (value size per head), scale (the factor on the
                scores), rot.base / rot.dims (the rotation's base and how many of a head's dimensions turn),
                rot.scaling {factor, original, fast, slow} (frequencies stretched for long contexts; absent: none),
                mask.size (how many positions, its own included, a query sees; absent or null: all before it),
                mask.keep_first (the first positions every query goes on seeing), v_mix (whether the layer takes
                part in the mixing of values across layers)
    mamba1      inner (channels), state (states per channel), dt_rank, conv (taps of the short convolution)
    mlp         kind "dense": ff (the gated feed-forward's inner size)

A missing or mistyped key is an error that names it by its path.
"""
from __future__ import annotations

import dataclasses
from typing import Any, ClassVar, Dict, Mapping, Optional, Tuple, Union

from .base import ConfigError, ModelConfig, read_key
from .mumusun import _read, _section

MIXER_TYPES = ("attention", "mamba1")
MLP_KINDS = ("dense",)


@dataclasses.dataclass(frozen=True)
class RotaryScaling:
    factor: float
    original: float
    fast: float
    slow: float

    def to_dict(self) -> Dict[str, Any]:
        return {"factor": self.factor, "original": self.original, "fast": self.fast, "slow": self.slow}


@dataclasses.dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: float
    rot_dims: int
    rot_scaling: Optional[RotaryScaling]
    window: Optional[int]
    keep_first: int
    v_mix: bool

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "AttentionConfig":
        rot = _section(d, "rot", where)
        mask = _section(d, "mask", where, optional=True) or {}
        sc = _section(rot, "scaling", where + "rot.", optional=True)
        scaling = None
        if sc is not None:
            w = where + "rot.scaling."
            scaling = RotaryScaling(_read(sc, "factor", float, w), _read(sc, "original", float, w), _read(sc, "fast", float, w),
                                    _read(sc, "slow", float, w))
        dim = _read(d, "dim", int, where)
        heads = _read(d, "heads", int, where)
        return cls(heads=heads, kv_heads=_read(d, "kv_heads", int, where, heads), dim=dim, vdim=_read(d, "vdim", int, where, dim),
                   scale=_read(d, "scale", float, where), rot_base=_read(rot, "base", float, where + "rot."),
                   rot_dims=_read(rot, "dims", int, where + "rot.", dim), rot_scaling=scaling,
                   window=_read(mask, "size", int, where + "mask.", None),
                   keep_first=_read(mask, "keep_first", int, where + "mask.", 0), v_mix=_read(d, "v_mix", bool, where, False))

    def to_dict(self) -> Dict[str, Any]:
        rot: Dict[str, Any] = {"base": self.rot_base, "dims": self.rot_dims}
        if self.rot_scaling is not None:
            rot["scaling"] = self.rot_scaling.to_dict()
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
               "rot": rot, "v_mix": self.v_mix}
        if self.window is not None or self.keep_first:
            out["mask"] = {"size": self.window, "keep_first": self.keep_first}
        return out

    def validate(self, where: str) -> None:
        for name in ("heads", "kv_heads", "dim", "vdim"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"config.json: '{where}{name}' must be positive, got {getattr(self, name)}")
        if self.heads % self.kv_heads:
            raise ConfigError(f"config.json: '{where}heads' = {self.heads} is not a multiple of kv_heads {self.kv_heads}")
        if self.dim % 2:
            raise ConfigError(f"config.json: '{where}dim' = {self.dim} must be even")
        if self.rot_dims <= 0 or self.rot_dims % 2 or self.rot_dims > self.dim:
            raise ConfigError(f"config.json: '{where}rot.dims' = {self.rot_dims} must be even and within dim {self.dim}")
        if not self.rot_base > 1:
            raise ConfigError(f"config.json: '{where}rot.base' must be above 1, got {self.rot_base}")
        if self.rot_scaling is not None and min(dataclasses.astuple(self.rot_scaling)) <= 0:
            raise ConfigError(f"config.json: '{where}rot.scaling' needs positive factor, original, fast and slow")
        if self.window is not None and self.window <= 0:
            raise ConfigError(f"config.json: '{where}mask.size' must be positive, got {self.window}")
        if self.keep_first < 0:
            raise ConfigError(f"config.json: '{where}mask.keep_first' must not be negative, got {self.keep_first}")


@dataclasses.dataclass(frozen=True)
class Mamba1Config:
    inner: int
    state: int
    dt_rank: int
    conv: int

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "Mamba1Config":
        return cls(inner=_read(d, "inner", int, where), state=_read(d, "state", int, where),
                   dt_rank=_read(d, "dt_rank", int, where), conv=_read(d, "conv", int, where))

    def to_dict(self) -> Dict[str, Any]:
        return {"inner": self.inner, "state": self.state, "dt_rank": self.dt_rank, "conv": self.conv}

    def validate(self, where: str) -> None:
        for name in ("inner", "state", "dt_rank", "conv"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"config.json: '{where}{name}' must be positive, got {getattr(self, name)}")
        if self.conv > 16:
            raise ConfigError(f"config.json: '{where}conv' = {self.conv}: at most 16 taps")
        if self.state > 128:
            raise ConfigError(f"config.json: '{where}state' = {self.state}: at most 128 states per channel")


@dataclasses.dataclass(frozen=True)
class DenseMlpConfig:
    ff: int

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "DenseMlpConfig":
        kind = _read(d, "kind", str, where, "dense")
        if kind not in MLP_KINDS:
            raise ConfigError(f"config.json: '{where}kind' = '{kind}' is not supported (one of {MLP_KINDS})")
        return cls(ff=_read(d, "ff", int, where))

    def to_dict(self) -> Dict[str, Any]:
        return {"kind": "dense", "ff": self.ff}

    def validate(self, where: str) -> None:
        if self.ff <= 0:
            raise ConfigError(f"config.json: '{where}ff' must be positive, got {self.ff}")


@dataclasses.dataclass(frozen=True)
class PoduraxLayer:
    type: str
    mixer: Union[AttentionConfig, Mamba1Config]
    mlp: Optional[DenseMlpConfig]

    def to_dict(self) -> Dict[str, Any]:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp is not None else None}


@dataclasses.dataclass(frozen=True)
class PoduraxConfig(ModelConfig):
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    residual_mult: float
    layers: Tuple[PoduraxLayer, ...]
    # The file names no longest sequence: positions are formed in 32-bit floats like every other angle of the
    # engine, which counts integers exactly up to 2^24.
    max_positions: int = 1 << 24

    model_type: ClassVar[str] = "podurax"
    architectures: ClassVar[Tuple[str, ...]] = ("Podurax",)

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "PoduraxConfig":
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
            mixer_cls = AttentionConfig if kind == "attention" else Mamba1Config
            mixer = mixer_cls.from_dict(_section(L, "mixer", where), where + "mixer.")
            mlp = _section(L, "mlp", where, optional=True)
            layers.append(PoduraxLayer(kind, mixer, DenseMlpConfig.from_dict(mlp, where + "mlp.") if mlp is not None else None))
        norm = _section(d, "norm", "")
        emb = _section(d, "embedding", "", optional=True) or {}
        cfg = cls(vocab=read_key(d, "vocab", int), width=read_key(d, "width", int), norm_eps=_read(norm, "eps", float, "norm."),
                  embedding_scale=_read(emb, "scale", float, "embedding.", 1.0),
                  residual_mult=read_key(d, "residual_mult", float, 1.0), layers=tuple(layers),
                  max_positions=read_key(d, "max_positions", int, 1 << 24))
        cfg.validate()
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        out = {"architecture": self.architectures[0], "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "embedding": {"scale": self.embedding_scale}, "residual_mult": self.residual_mult,
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
        mixing = None
        for i, L in enumerate(self.layers):
            L.mixer.validate(f"layers[{i}].mixer.")
            if L.mlp is not None:
                L.mlp.validate(f"layers[{i}].mlp.")
            if L.type == "attention" and L.mixer.v_mix:
                shape = (L.mixer.kv_heads, L.mixer.vdim)
                if mixing is not None and shape != mixing:
                    raise ConfigError(f"config.json: 'layers[{i}].mixer' mixes values of {shape[0]} kv heads x {shape[1]} with "
                                      f"an earlier layer's {mixing[0]} x {mixing[1]}: layers with v_mix must agree in both")
                mixing = shape
