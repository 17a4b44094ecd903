"""Typed configuration of the Repolix decoder, read from config.json's own keys.

    {"architecture": "Repolix", "vocab": V, "width": W, "norm": {"eps": e}, "embedding": {"scale": s},
     "layers": [{"type": "mamba2" | "channel_delta" | "attention", "mixer": {...}, "mlp": {...} | null}, ...]}

    mixer of "mamba2":         heads, vdim, state, groups, norm_groups, conv
    mixer of "channel_delta":  heads, kv_heads, dim, vdim, conv
    mixer of "attention":      heads, kv_heads, dim, vdim, conv, scale, diff, mask: {size},
                               rot: {base, dims, scaling: {factor, original, fast, slow}}
    mlp:  {"kind": "moe", "expert": {ff, limit}, "router": {experts, top, identity, groups: {count, keep}},
           "shared": {ff, limit}}

Every layer carries its own sizes; the list's order is the order in which the layers run.  Keys that a layer may do
without: mask (every earlier key is seen), rot.scaling (the plain rates), router.identity (none), router.groups (one
group), shared (no such expert), embedding (scale 1).
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Optional

import numpy as np

from .errors import ConfigError
from .fields import obj as _obj, integer as _int, number as _num

LAYER_TYPES = ("mamba2", "channel_delta", "attention")


@dataclass(frozen=True)
class StateSpaceConfig:
    heads: int
    vdim: int
    state: int
    groups: int
    norm_groups: int
    conv: int

    @classmethod
    def from_dict(cls, d, where):
        c = cls(_int(d, "heads", where), _int(d, "vdim", where), _int(d, "state", where), _int(d, "groups", where),
                _int(d, "norm_groups", where) if d.get("norm_groups") is not None else 1, _int(d, "conv", where))
        if c.heads % c.groups:
            raise ConfigError(f"{where}: {c.heads} heads do not divide into {c.groups} groups")
        if (c.heads * c.vdim) % c.norm_groups:
            raise ConfigError(f"{where}: {c.heads * c.vdim} values do not divide into {c.norm_groups} normed parts")
        return c

    def to_dict(self):
        return {"heads": self.heads, "vdim": self.vdim, "state": self.state, "groups": self.groups,
                "norm_groups": self.norm_groups, "conv": self.conv}


@dataclass(frozen=True)
class ChannelDeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @classmethod
    def from_dict(cls, d, where):
        c = cls(_int(d, "heads", where), _int(d, "kv_heads", where), _int(d, "dim", where), _int(d, "vdim", where),
                _int(d, "conv", where))
        if c.heads % c.kv_heads:
            raise ConfigError(f"{where}: {c.heads} heads do not divide into {c.kv_heads} kv heads")
        return c

    def to_dict(self):
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}


@dataclass(frozen=True)
class RotationScaling:
    factor: float
    original: float
    fast: float
    slow: float

    @classmethod
    def from_dict(cls, d, where):
        c = cls(_num(d, "factor", where), _num(d, "original", where), _num(d, "fast", where), _num(d, "slow", where))
        if not (c.factor > 0.0 and c.original > 0.0 and c.fast > 0.0 and c.slow > 0.0):
            raise ConfigError(f"{where}: factor, original, fast and slow must be positive")
        return c

    def to_dict(self):
        return {"factor": self.factor, "original": self.original, "fast": self.fast, "slow": self.slow}


@dataclass(frozen=True)
class DiffAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    scale: float
    diff: float
    window: Optional[int]          # mask.size; None: every earlier key
    rot_base: float
    rot_dims: int
    rot_scaling: Optional[RotationScaling]

    @classmethod
    def from_dict(cls, d, where):
        rot = _obj(d, "rot", where)
        window = _int(_obj(d, "mask", where), "size", where + ".mask") if d.get("mask") is not None else None
        scaling = (RotationScaling.from_dict(_obj(rot, "scaling", where + ".rot"), where + ".rot.scaling")
                   if rot.get("scaling") is not None else None)
        dim = _int(d, "dim", where)
        c = cls(_int(d, "heads", where), _int(d, "kv_heads", where), dim, _int(d, "vdim", where), _int(d, "conv", where),
                _num(d, "scale", where) if d.get("scale") is not None else float(dim) ** -0.5, _num(d, "diff", where),
                window, _num(rot, "base", where + ".rot"), _int(rot, "dims", where + ".rot", 0), scaling)
        if c.heads % c.kv_heads:
            raise ConfigError(f"{where}: {c.heads} heads do not divide into {c.kv_heads} kv heads")
        if c.rot_dims % 2 or c.rot_dims > c.dim:
            raise ConfigError(f"{where}.rot: dims {c.rot_dims} must be even and at most dim {c.dim}")
        if not c.rot_base > 1.0:
            raise ConfigError(f"{where}.rot: base {c.rot_base} must be larger than 1")
        return c

    def to_dict(self):
        rot = {"base": self.rot_base, "dims": self.rot_dims}
        if self.rot_scaling is not None:
            rot["scaling"] = self.rot_scaling.to_dict()
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv,
             "scale": self.scale, "diff": self.diff, "rot": rot}
        if self.window is not None:
            d["mask"] = {"size": self.window}
        return d


MIXER_CONFIGS = {"mamba2": StateSpaceConfig, "channel_delta": ChannelDeltaConfig, "attention": DiffAttentionConfig}


@dataclass(frozen=True)
class LimitedExpertConfig:
    ff: int
    limit: float

    @classmethod
    def from_dict(cls, d, where):
        c = cls(_int(d, "ff", where), _num(d, "limit", where))
        if not c.limit > 0.0:
            raise ConfigError(f"{where}: limit {c.limit} must be positive")
        return c

    def to_dict(self):
        return {"ff": self.ff, "limit": self.limit}


@dataclass(frozen=True)
class RoutedConfig:
    expert: LimitedExpertConfig
    experts: int                  # experts that have matrices
    top: int
    identity: int                 # further router outputs whose expert is the identity
    groups: int
    keep_groups: int
    shared: Optional[LimitedExpertConfig]

    @classmethod
    def from_dict(cls, d, where):
        if d.get("kind") != "moe":
            raise ConfigError(f"{where}: kind {d.get('kind')!r} (this decoder's feed-forward is 'moe')")
        router = _obj(d, "router", where)
        groups = router.get("groups")
        count = keep = 1
        if groups is not None:
            groups = _obj(router, "groups", where + ".router")
            count, keep = _int(groups, "count", where + ".router.groups"), _int(groups, "keep", where + ".router.groups")
        c = cls(LimitedExpertConfig.from_dict(_obj(d, "expert", where), where + ".expert"),
                _int(router, "experts", where + ".router", 0), _int(router, "top", where + ".router"),
                _int(router, "identity", where + ".router", 0) if router.get("identity") is not None else 0, count, keep,
                LimitedExpertConfig.from_dict(_obj(d, "shared", where), where + ".shared") if d.get("shared") is not None else None)
        total = c.experts + c.identity
        if total <= 0 or total % c.groups or c.keep_groups > c.groups:
            raise ConfigError(f"{where}.router: {total} router outputs in {c.groups} groups of which {c.keep_groups} stay")
        if c.top > c.keep_groups * (total // c.groups):
            raise ConfigError(f"{where}.router: top {c.top} of {c.keep_groups} groups of {total // c.groups}")
        return c

    def to_dict(self):
        d = {"kind": "moe", "expert": self.expert.to_dict(),
             "router": {"experts": self.experts, "top": self.top, "identity": self.identity,
                        "groups": {"count": self.groups, "keep": self.keep_groups}}}
        if self.shared is not None:
            d["shared"] = self.shared.to_dict()
        return d


@dataclass(frozen=True)
class RepolixLayerConfig:
    type: str
    mixer: object
    mlp: Optional[RoutedConfig]

    @classmethod
    def from_dict(cls, d, where):
        kind = d.get("type") if isinstance(d, dict) else None
        if kind not in LAYER_TYPES:
            raise ConfigError(f"{where}: layer type {kind!r} (this decoder has {', '.join(LAYER_TYPES)})")
        mlp = None if d.get("mlp") is None else RoutedConfig.from_dict(_obj(d, "mlp", where), where + ".mlp")
        return cls(kind, MIXER_CONFIGS[kind].from_dict(_obj(d, "mixer", where), where + ".mixer"), mlp)

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class RepolixConfig:
    vocab: int
    width: int
    layers: tuple
    norm_eps: float
    embedding_scale: float = 1.0
    # sizes of the narrow middles of a channel_delta mixer for random weights (stored weights bring their own, and no
    # key of config.json names them); written out only when they were set
    middle_rank: Optional[int] = None

    architecture = "Repolix"
    max_position_embeddings = None    # the rotation's table bounds the positions (the mixers' position parts say how far)
    eos_token_id = None

    @classmethod
    def from_dict(cls, d: dict) -> "RepolixConfig":
        if not isinstance(d.get("layers"), list) or not d["layers"]:
            raise ConfigError("config key 'layers' must be a list with at least one layer")
        scale = 1.0
        if d.get("embedding") is not None:
            scale = _num(_obj(d, "embedding", "config"), "scale", "config.embedding")
        cfg = cls(_int(d, "vocab", "config"), _int(d, "width", "config"),
                  tuple(RepolixLayerConfig.from_dict(l, f"layers[{i}]") for i, l in enumerate(d["layers"])),
                  _num(_obj(d, "norm", "config"), "eps", "config.norm"), scale,
                  _int(d, "middle_rank", "config") if d.get("middle_rank") is not None else None)
        if not cfg.norm_eps > 0.0:
            raise ConfigError(f"norm.eps {cfg.norm_eps} must be positive")
        return cfg

    @classmethod
    def from_json(cls, path: str) -> "RepolixConfig":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        try:
            with open(path) as f:
                d = json.load(f)
        except OSError as e:
            raise ConfigError(f"read {path}: {e}") from None
        except json.JSONDecodeError as e:
            raise ConfigError(f"parse {path}: {e}") from None
        if not isinstance(d, dict):
            raise ConfigError(f"parse {path}: top level is not an object")
        return cls.from_dict(d)

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
             "layers": [l.to_dict() for l in self.layers], "norm": {"eps": self.norm_eps},
             "embedding": {"scale": self.embedding_scale}}
        if self.middle_rank is not None:
            d["middle_rank"] = self.middle_rank
        return d

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def eps_f32(self) -> float:
        return float(np.float32(self.norm_eps))

    @property
    def stop_token_ids(self) -> tuple:
        return ()
