"""Typed Rezelix configuration, read from the keys of its ``config.json``.

A Rezelix model lists its layers one by one: each names its mixer (``rglru``, ``attention`` or
``latent_attention``) with the mixer's own sizes and constants, and its feed-forward (``dense``
or none).  Rotary positions are described per mixer (``rot``: rotated dimensions, base and an
optional YaRN ``scaling``).  Every size and constant comes from the file.
"""

from dataclasses import dataclass
from typing import Optional, Tuple

from .base import ConfigError, require_int

MIXERS = ("rglru", "attention", "latent_attention")


def _number(raw, key, where, positive=True):
    value = raw.get(key) if isinstance(raw, dict) else None
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ConfigError(f"config.json {where} '{key}' must be a number, got {value!r}")
    if positive and not value > 0:
        raise ConfigError(f"config.json {where} '{key}' must be positive, got {value!r}")
    return float(value)


@dataclass(frozen=True)
class RezelixScaling:
    """YaRN: how the rotation's frequencies are stretched beyond the ``original`` length."""

    factor: float
    original: float
    fast: float
    slow: float

    def to_dict(self):
        return {"factor": self.factor, "original": self.original, "fast": self.fast, "slow": self.slow}


@dataclass(frozen=True)
class RezelixRotation:
    dims: int
    base: float
    scaling: Optional[RezelixScaling] = None

    def to_dict(self):
        out = {"dims": self.dims, "base": self.base}
        if self.scaling is not None:
            out["scaling"] = self.scaling.to_dict()
        return out


@dataclass(frozen=True)
class RezelixRecurrent:
    width: int
    blocks: int
    conv: int

    def to_dict(self):
        return {"width": self.width, "blocks": self.blocks, "conv": self.conv}


@dataclass(frozen=True)
class RezelixAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float            # 0: none
    rot: Optional[RezelixRotation]

    def to_dict(self):
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
               "scale": self.scale}
        if self.softcap:
            out["softcap"] = self.softcap
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        return out


@dataclass(frozen=True)
class RezelixLatent:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    softcap: float
    rot: Optional[RezelixRotation]

    def to_dict(self):
        out = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim,
               "kv_rank": self.kv_rank, "scale": self.scale}
        if self.softcap:
            out["softcap"] = self.softcap
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        return out


@dataclass(frozen=True)
class RezelixFeedForward:
    kind: str
    ff: int

    def to_dict(self):
        return {"kind": self.kind, "ff": self.ff}


@dataclass(frozen=True)
class RezelixLayer:
    type: str
    mixer: object
    mlp: Optional[RezelixFeedForward]

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(),
                "mlp": None if self.mlp is None else self.mlp.to_dict()}


def _read_rotation(raw, where, most):
    if raw is None:
        return None
    if not isinstance(raw, dict):
        raise ConfigError(f"config.json {where} 'rot' must be an object")
    dims = require_int(raw, "dims", minimum=0)
    if dims == 0:
        return None
    if dims % 2 or dims > most:
        raise ConfigError(f"config.json {where} 'rot.dims' {dims} must be even and at most {most}")
    scaling = raw.get("scaling")
    if scaling is not None:
        if not isinstance(scaling, dict):
            raise ConfigError(f"config.json {where} 'rot.scaling' must be an object")
        inner = where + ".rot.scaling"
        scaling = RezelixScaling(factor=_number(scaling, "factor", inner),
                                 original=_number(scaling, "original", inner),
                                 fast=_number(scaling, "fast", inner),
                                 slow=_number(scaling, "slow", inner))
    return RezelixRotation(dims=dims, base=_number(raw, "base", where + ".rot"), scaling=scaling)


def _cap(mixer, where):
    if mixer.get("softcap") in (None, 0, 0.0):
        return 0.0
    return _number(mixer, "softcap", where)


def _read_mixer(kind, mixer, where):
    if kind == "rglru":
        width = require_int(mixer, "width")
        blocks = require_int(mixer, "blocks")
        if width % blocks:
            raise ConfigError(f"'width' {width} must be a multiple of 'blocks' {blocks}")
        return RezelixRecurrent(width=width, blocks=blocks, conv=require_int(mixer, "conv"))
    heads = require_int(mixer, "heads")
    dim = require_int(mixer, "dim")
    if kind == "attention":
        kv_heads = require_int(mixer, "kv_heads", default=heads)
        if heads % kv_heads:
            raise ConfigError(f"heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
        vdim = require_int(mixer, "vdim", default=dim)
        if vdim != dim:
            raise ConfigError(f"the values are the keys as projected: 'vdim' {vdim} must equal 'dim' {dim}")
        return RezelixAttention(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim,
                                scale=_number(mixer, "scale", where + ".mixer"),
                                softcap=_cap(mixer, where + ".mixer"),
                                rot=_read_rotation(mixer.get("rot"), where + ".mixer", dim))
    rot_dim = require_int(mixer, "rot_dim", minimum=0)
    rot = _read_rotation(mixer.get("rot"), where + ".mixer", rot_dim) if rot_dim else None
    if rot is not None and rot.dims != rot_dim:
        raise ConfigError(f"'rot.dims' {rot.dims} must equal 'rot_dim' {rot_dim}: the rotated part is rotated whole")
    return RezelixLatent(heads=heads, dim=dim, rot_dim=rot_dim, vdim=require_int(mixer, "vdim"),
                         kv_rank=require_int(mixer, "kv_rank"),
                         scale=_number(mixer, "scale", where + ".mixer"),
                         softcap=_cap(mixer, where + ".mixer"), rot=rot)


def _read_feed_forward(mlp, where):
    if mlp is None:
        return None
    if not isinstance(mlp, dict) or mlp.get("kind", "dense") != "dense":
        raise ConfigError(f"config.json {where} 'mlp.kind' must be 'dense', got {mlp!r}")
    return RezelixFeedForward("dense", require_int(mlp, "ff"))


@dataclass(frozen=True)
class RezelixConfig:
    vocab: int
    width: int
    layers: Tuple[RezelixLayer, ...]
    norm_eps: float
    max_positions: int

    architecture = "Rezelix"
    eos_token_id = None        # the configuration names no token that ends a request
    # where the file names no bound, requests may grow to this many tokens (an engine's pool or
    # its own bound may be smaller)
    DEFAULT_MAX_POSITIONS = 32768

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @classmethod
    def from_dict(cls, raw) -> "RezelixConfig":
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json 'layers' must be a non-empty list")
        layers = []
        for index, entry in enumerate(listed):
            where = f"layers[{index}]"
            if not isinstance(entry, dict) or entry.get("type") not in MIXERS:
                raise ConfigError(f"config.json {where} 'type' must be one of {', '.join(MIXERS)}, "
                                  f"got {entry.get('type') if isinstance(entry, dict) else entry!r}")
            if not isinstance(entry.get("mixer"), dict):
                raise ConfigError(f"config.json {where} lacks 'mixer'")
            try:
                mixer = _read_mixer(entry["type"], entry["mixer"], where)
                mlp = _read_feed_forward(entry.get("mlp"), where)
            except ConfigError as error:
                raise ConfigError(f"{where}: {error}") from None
            layers.append(RezelixLayer(entry["type"], mixer, mlp))
        norm = raw.get("norm") or {}
        return cls(
            vocab=require_int(raw, "vocab"),
            width=require_int(raw, "width"),
            layers=tuple(layers),
            norm_eps=_number(norm, "eps", "norm"),
            max_positions=require_int(raw, "max_positions", default=cls.DEFAULT_MAX_POSITIONS),
        )

    def to_dict(self) -> dict:
        out = {
            "architecture": self.architecture,
            "vocab": self.vocab,
            "width": self.width,
            "layers": [layer.to_dict() for layer in self.layers],
            "norm": {"eps": self.norm_eps},
        }
        if self.max_positions != self.DEFAULT_MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        return out
