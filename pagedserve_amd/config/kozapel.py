"""Typed Kozapel configuration, read from the keys of its ``config.json``.

A Kozapel model lists its layers one by one: each names its mixer (``attention``: differential
attention under a sliding window, with its own key and value projections or those of an earlier
layer; ``latent_attention``: attention over a cached latent, queries through a latent of their
own) with the mixer's sizes and constants, and its feed-forward (``dense``, ``moe`` or none).
The residual stream is kept in ``streams`` copies.  Every size and constant comes from the file.
"""

from dataclasses import dataclass
from typing import Optional, Tuple

from .base import ConfigError, require_int

MIXERS = ("attention", "latent_attention")


def _number(raw, key, where, positive=True):
    value = raw.get(key) if isinstance(raw, dict) else None
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ConfigError(f"config.json {where} '{key}' must be a number, got {value!r}")
    if positive and not value > 0:
        raise ConfigError(f"config.json {where} '{key}' must be positive, got {value!r}")
    return float(value)


@dataclass(frozen=True)
class KozapelAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    window: int                  # 0: every earlier token is seen
    kv_from: Optional[int]       # the layer whose keys and values this one reads (None: its own)

    def to_dict(self):
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
               "scale": self.scale, "diff": self.diff}
        if self.window:
            out["mask"] = {"size": self.window}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


@dataclass(frozen=True)
class KozapelLatent:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot_base: float

    def to_dict(self):
        out = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim,
               "kv_rank": self.kv_rank, "q_rank": self.q_rank, "scale": self.scale}
        if self.rot_dim:
            out["rot"] = {"dims": self.rot_dim, "base": self.rot_base}
        return out


@dataclass(frozen=True)
class KozapelFeedForward:
    kind: str                    # "dense" or "moe"
    ff: int                      # inner width (of one expert for "moe")
    experts: int = 0
    top: int = 0
    groups: int = 1
    keep: int = 1
    scale: float = 1.0
    shared_ff: int = 0           # 0: no shared expert

    def to_dict(self):
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        out = {"kind": "moe", "expert": {"ff": self.ff},
               "router": {"experts": self.experts, "top": self.top, "scale": self.scale,
                          "groups": {"count": self.groups, "keep": self.keep}}}
        if self.shared_ff:
            out["shared"] = {"ff": self.shared_ff}
        return out


@dataclass(frozen=True)
class KozapelLayer:
    type: str
    mixer: object
    mlp: Optional[KozapelFeedForward]

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(),
                "mlp": None if self.mlp is None else self.mlp.to_dict()}


def _read_mixer(kind, mixer, where, index):
    heads = require_int(mixer, "heads")
    dim = require_int(mixer, "dim")
    vdim = require_int(mixer, "vdim", default=dim)
    scale = _number(mixer, "scale", where + ".mixer")
    if kind == "attention":
        kv_heads = require_int(mixer, "kv_heads", default=heads)
        if heads % kv_heads:
            raise ConfigError(f"heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
        mask = mixer.get("mask")
        if mask is not None and not isinstance(mask, dict):
            raise ConfigError(f"config.json {where} 'mask' must be an object")
        window = require_int(mask, "size") if mask else 0
        kv_from = mixer.get("kv_from")
        if kv_from is not None:
            kv_from = require_int(mixer, "kv_from", minimum=0)
            if kv_from >= index:
                raise ConfigError(f"'kv_from' {kv_from} must name an earlier layer")
        return KozapelAttention(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale,
                                diff=_number(mixer, "diff", where + ".mixer", positive=False),
                                window=window, kv_from=kv_from)
    rot_dim = require_int(mixer, "rot_dim", minimum=0)
    rot = mixer.get("rot") or {}
    if not isinstance(rot, dict):
        raise ConfigError(f"config.json {where} 'rot' must be an object")
    if rot_dim % 2:
        raise ConfigError(f"'rot_dim' {rot_dim} must be even")
    if rot_dim and require_int(rot, "dims", default=rot_dim) != rot_dim:
        raise ConfigError(f"'rot.dims' {rot.get('dims')} must equal 'rot_dim' {rot_dim}: the rotated part "
                          "is rotated whole")
    return KozapelLatent(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim,
                         kv_rank=require_int(mixer, "kv_rank"), q_rank=require_int(mixer, "q_rank"),
                         scale=scale,
                         rot_base=_number(rot, "base", where + ".mixer.rot") if rot_dim else 10000.0)


def _read_feed_forward(mlp, where):
    if mlp is None:
        return None
    if not isinstance(mlp, dict) or mlp.get("kind", "dense") not in ("dense", "moe"):
        raise ConfigError(f"config.json {where} 'mlp.kind' must be 'dense' or 'moe', got {mlp!r}")
    if mlp.get("kind", "dense") == "dense":
        return KozapelFeedForward("dense", require_int(mlp, "ff"))
    expert, router = mlp.get("expert"), mlp.get("router")
    if not isinstance(expert, dict) or not isinstance(router, dict):
        raise ConfigError(f"config.json {where} 'mlp' of kind 'moe' needs 'expert' and 'router'")
    experts = require_int(router, "experts")
    top = require_int(router, "top")
    groups = router.get("groups") or {}
    count = require_int(groups, "count", default=1)
    keep = require_int(groups, "keep", default=count)
    if experts % count or not 1 <= keep <= count:
        raise ConfigError(f"'router.groups' {groups!r} must divide {experts} experts and keep 1..count groups")
    if top > (experts // count) * keep:
        raise ConfigError(f"'router.top' {top} exceeds the experts of the {keep} groups that are kept")
    shared = mlp.get("shared")
    return KozapelFeedForward("moe", require_int(expert, "ff"), experts=experts, top=top, groups=count,
                              keep=keep, scale=_number(router, "scale", where + ".mlp.router")
                              if "scale" in router else 1.0,
                              shared_ff=require_int(shared, "ff") if shared else 0)


@dataclass(frozen=True)
class KozapelConfig:
    vocab: int
    width: int
    layers: Tuple[KozapelLayer, ...]
    norm_eps: float
    embedding_scale: float
    streams: int                 # 0: one plain residual stream
    max_positions: int

    architecture = "Kozapel"
    eos_token_id = None        # the configuration names no token that ends a request
    # where the file names no bound, requests may grow to this many tokens (an engine's pool or
    # its own bound may be smaller)
    DEFAULT_MAX_POSITIONS = 32768

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @classmethod
    def from_dict(cls, raw) -> "KozapelConfig":
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
                mixer = _read_mixer(entry["type"], entry["mixer"], where, index)
                mlp = _read_feed_forward(entry.get("mlp"), where)
            except ConfigError as error:
                raise ConfigError(f"{where}: {error}") from None
            layers.append(KozapelLayer(entry["type"], mixer, mlp))
        for index, layer in enumerate(layers):
            source = getattr(layer.mixer, "kv_from", None)
            if source is None:
                continue
            other = layers[source]
            if other.type != "attention" or other.mixer.kv_from is not None:
                raise ConfigError(f"layers[{index}]: 'kv_from' {source} must name an attention layer with "
                                  "key and value projections of its own")
            mine = layer.mixer
            if (mine.kv_heads, mine.dim, mine.vdim) != (other.mixer.kv_heads, other.mixer.dim, other.mixer.vdim):
                raise ConfigError(f"layers[{index}]: kv_heads, dim and vdim must equal those of layer {source}, "
                                  "whose keys and values it reads")
        norm = raw.get("norm") or {}
        embedding = raw.get("embedding") or {}
        return cls(
            vocab=require_int(raw, "vocab"),
            width=require_int(raw, "width"),
            layers=tuple(layers),
            norm_eps=_number(norm, "eps", "norm"),
            embedding_scale=_number(embedding, "scale", "embedding") if "scale" in embedding else 1.0,
            streams=require_int(raw, "streams", default=0, minimum=0),
            max_positions=require_int(raw, "max_positions", default=cls.DEFAULT_MAX_POSITIONS),
        )

    def to_dict(self) -> dict:
        out = {
            "architecture": self.architecture,
            "vocab": self.vocab,
            "width": self.width,
            "layers": [layer.to_dict() for layer in self.layers],
            "norm": {"eps": self.norm_eps},
            "embedding": {"scale": self.embedding_scale},
        }
        if self.streams:
            out["streams"] = self.streams
        if self.max_positions != self.DEFAULT_MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        return out

    def cache_window(self, index: int) -> int:
        """The window of the cache entry that layer ``index`` writes: its own, or the widest of
        the layers that read the entry (0, everything, if one of them sees everything)."""
        windows = [self.layers[index].mixer.window]
        windows += [layer.mixer.window for layer in self.layers
                    if layer.type == "attention" and layer.mixer.kv_from == index]
        return 0 if 0 in windows else max(windows)
