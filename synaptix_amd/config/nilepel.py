"""Typed configuration of the Nilepel decoder, read from config.json's own keys.

    {"architecture": "Nilepel", "vocab": V, "width": W, "norm": {"eps": e}, "embedding": {"scale": s},
     "layers": [{"type": "attention" | "attention_2" | "latent_attention", "mixer": {...}, "mlp": {...} | null}, ...]}

    mixer of "attention":         heads, kv_heads, dim, vdim, scale, mask: {size}, rot: {base, dims}
    mixer of "attention_2":       heads, kv_heads, dim, vdim, scale, mask: {size}, kv_from,
                                  rot: {base, dims, scaling: {factor, low, high, original}}
    mixer of "latent_attention":  heads, dim, rot_dim, vdim, kv_rank, scale, mask: {size}, rot: {base, dims}
    mlp:  {"kind": "dense", "ff", "limit"}
          {"kind": "moe", "expert": {ff}, "router": {experts, top, scale, groups: {count, keep}}, "shared": {ff}}

Every layer carries its own sizes; the list's order is the order in which the layers run.  Keys that a layer may do
without: mask (every earlier key is seen), rot (nothing is turned), rot.scaling (the plain rates), kv_from (keys and
values of its own), router.scale (1), router.groups (one group), shared (no such expert), embedding (scale 1).
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Optional

import numpy as np

from .errors import ConfigError
from .fields import obj as _obj, integer as _int, number as _num

LAYER_TYPES = ("attention", "attention_2", "latent_attention")


def _mask(d, where):
    return _int(_obj(d, "mask", where), "size", where + ".mask") if d.get("mask") is not None else None


def _mask_dict(size):
    return {} if size is None else {"mask": {"size": size}}


@dataclass(frozen=True)
class WavelengthScaling:
    factor: float
    low: float
    high: float
    original: float

    @classmethod
    def from_dict(cls, d, where):
        c = cls(_num(d, "factor", where), _num(d, "low", where), _num(d, "high", where), _num(d, "original", where))
        if not (c.factor > 0.0 and c.original > 0.0 and c.low > 0.0 and c.high > c.low):
            raise ConfigError(f"{where}: factor and original must be positive and 0 < low < high")
        return c

    def to_dict(self):
        return {"factor": self.factor, "low": self.low, "high": self.high, "original": self.original}


@dataclass(frozen=True)
class Rotation:
    base: float
    dims: int                      # 0: nothing is turned
    scaling: Optional[WavelengthScaling] = None

    @classmethod
    def from_dict(cls, d, where, most):
        if d.get("rot") is None:
            return cls(10000.0, 0)
        rot, at = _obj(d, "rot", where), where + ".rot"
        scaling = None
        if rot.get("scaling") is not None:
            scaling = WavelengthScaling.from_dict(_obj(rot, "scaling", at), at + ".scaling")
        c = cls(_num(rot, "base", at), _int(rot, "dims", at, 0), scaling)
        if c.dims % 2 or c.dims > most:
            raise ConfigError(f"{at}: dims {c.dims} must be even and at most {most}")
        if not c.base > 1.0:
            raise ConfigError(f"{at}: base {c.base} must be larger than 1")
        return c

    def to_dict(self):
        d = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            d["scaling"] = self.scaling.to_dict()
        return d


def _heads(d, where):
    heads, kv = _int(d, "heads", where), _int(d, "kv_heads", where)
    if heads % kv:
        raise ConfigError(f"{where}: {heads} heads do not divide into {kv} kv heads")
    return heads, kv


def _scale(d, where, size):
    return _num(d, "scale", where) if d.get("scale") is not None else float(size) ** -0.5


@dataclass(frozen=True)
class ChunkedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: Optional[int]           # mask.size; None: every earlier key
    rot: Rotation

    kv_from: Optional[int] = None  # the layer whose keys and values this one reads; None: its own

    @classmethod
    def from_dict(cls, d, where):
        heads, kv = _heads(d, where)
        dim = _int(d, "dim", where)
        return cls(heads, kv, dim, _int(d, "vdim", where), _scale(d, where, dim), _mask(d, where),
                   Rotation.from_dict(d, where, dim), _int(d, "kv_from", where, 0) if d.get("kv_from") is not None else None)

    def to_dict(self):
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
             "rot": self.rot.to_dict(), **_mask_dict(self.chunk)}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d


@dataclass(frozen=True)
class WindowAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int]          # mask.size; None: every earlier key
    rot: Rotation
    kv_from: Optional[int] = None  # the layer whose keys and values this one reads; None: its own

    @classmethod
    def from_dict(cls, d, where):
        heads, kv = _heads(d, where)
        dim = _int(d, "dim", where)
        return cls(heads, kv, dim, _int(d, "vdim", where), _scale(d, where, dim), _mask(d, where),
                   Rotation.from_dict(d, where, dim),
                   _int(d, "kv_from", where, 0) if d.get("kv_from") is not None else None)

    def to_dict(self):
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
             "rot": self.rot.to_dict(), **_mask_dict(self.window)}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    window: Optional[int]
    rot: Rotation

    kv_from = None

    @classmethod
    def from_dict(cls, d, where):
        dim, rot_dim = _int(d, "dim", where), _int(d, "rot_dim", where, 0)
        return cls(_int(d, "heads", where), dim, rot_dim, _int(d, "vdim", where), _int(d, "kv_rank", where),
                   _scale(d, where, dim + rot_dim), _mask(d, where), Rotation.from_dict(d, where, rot_dim))

    def to_dict(self):
        return {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
                "scale": self.scale, "rot": self.rot.to_dict(), **_mask_dict(self.window)}


MIXER_CONFIGS = {"attention": ChunkedAttentionConfig, "attention_2": WindowAttentionConfig,
                 "latent_attention": LatentAttentionConfig}


@dataclass(frozen=True)
class DenseConfig:
    ff: int
    limit: float

    kind = "dense"

    @classmethod
    def from_dict(cls, d, where):
        c = cls(_int(d, "ff", where), _num(d, "limit", where))
        if not c.limit > 0.0:
            raise ConfigError(f"{where}: limit {c.limit} must be positive")
        return c

    def to_dict(self):
        return {"kind": "dense", "ff": self.ff, "limit": self.limit}


@dataclass(frozen=True)
class MoeConfig:
    ff: int                       # of each routed expert
    experts: int
    top: int
    groups: int
    keep_groups: int
    route_scale: float
    shared_ff: Optional[int]      # None: no expert that every token passes

    kind = "moe"

    @classmethod
    def from_dict(cls, d, where):
        router, at = _obj(d, "router", where), where + ".router"
        count = keep = 1
        if router.get("groups") is not None:
            groups = _obj(router, "groups", at)
            count, keep = _int(groups, "count", at + ".groups"), _int(groups, "keep", at + ".groups")
        c = cls(_int(_obj(d, "expert", where), "ff", where + ".expert"), _int(router, "experts", at), _int(router, "top", at),
                count, keep, _num(router, "scale", at) if router.get("scale") is not None else 1.0,
                _int(_obj(d, "shared", where), "ff", where + ".shared") if d.get("shared") is not None else None)
        if c.experts % c.groups or c.keep_groups > c.groups:
            raise ConfigError(f"{at}: {c.experts} experts in {c.groups} groups of which {c.keep_groups} stay")
        if c.top > c.keep_groups * (c.experts // c.groups):
            raise ConfigError(f"{at}: top {c.top} of {c.keep_groups} groups of {c.experts // c.groups}")
        return c

    def to_dict(self):
        d = {"kind": "moe", "expert": {"ff": self.ff},
             "router": {"experts": self.experts, "top": self.top, "scale": self.route_scale,
                        "groups": {"count": self.groups, "keep": self.keep_groups}}}
        if self.shared_ff is not None:
            d["shared"] = {"ff": self.shared_ff}
        return d


MLP_CONFIGS = {"dense": DenseConfig, "moe": MoeConfig}


@dataclass(frozen=True)
class NilepelLayerConfig:
    type: str
    mixer: object
    mlp: object                    # DenseConfig, MoeConfig or None

    @classmethod
    def from_dict(cls, d, where):
        kind = d.get("type") if isinstance(d, dict) else None
        if kind not in LAYER_TYPES:
            raise ConfigError(f"{where}: layer type {kind!r} (this decoder has {', '.join(LAYER_TYPES)})")
        mlp = None
        if d.get("mlp") is not None:
            m = _obj(d, "mlp", where)
            if m.get("kind") not in MLP_CONFIGS:
                raise ConfigError(f"{where}.mlp: kind {m.get('kind')!r} (one of {', '.join(MLP_CONFIGS)})")
            mlp = MLP_CONFIGS[m["kind"]].from_dict(m, where + ".mlp")
        return cls(kind, MIXER_CONFIGS[kind].from_dict(_obj(d, "mixer", where), where + ".mixer"), mlp)

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class NilepelConfig:
    vocab: int
    width: int
    layers: tuple
    norm_eps: float
    embedding_scale: float = 1.0

    architecture = "Nilepel"
    max_position_embeddings = None    # the rotation's table bounds the positions (the mixers' position parts say how far)
    eos_token_id = None

    @classmethod
    def from_dict(cls, d: dict) -> "NilepelConfig":
        if not isinstance(d.get("layers"), list) or not d["layers"]:
            raise ConfigError("config key 'layers' must be a list with at least one layer")
        scale = 1.0
        if d.get("embedding") is not None:
            scale = _num(_obj(d, "embedding", "config"), "scale", "config.embedding")
        cfg = cls(_int(d, "vocab", "config"), _int(d, "width", "config"),
                  tuple(NilepelLayerConfig.from_dict(l, f"layers[{i}]") for i, l in enumerate(d["layers"])),
                  _num(_obj(d, "norm", "config"), "eps", "config.norm"), scale)
        if not cfg.norm_eps > 0.0:
            raise ConfigError(f"norm.eps {cfg.norm_eps} must be positive")
        for i, layer in enumerate(cfg.layers):
            cfg.kv_source(i)
        return cfg

    def kv_source(self, i: int) -> int:
        """The layer whose cache layer i reads: itself, or where its chain of `kv_from` ends.  The source runs earlier,
        keeps keys and values by head, and has the same head counts and sizes."""
        m, at = self.layers[i].mixer, i
        while self.layers[at].mixer.kv_from is not None:
            src = self.layers[at].mixer.kv_from
            if not 0 <= src < at:
                raise ConfigError(f"layers[{at}].mixer: kv_from {src} must name an earlier layer")
            at = src
        s = self.layers[at].mixer
        if at != i and (self.layers[at].type == "latent_attention"
                        or (s.heads, s.kv_heads, s.dim, s.vdim) != (m.heads, m.kv_heads, m.dim, m.vdim)):
            raise ConfigError(f"layers[{i}].mixer: kv_from {at} names a layer of another kind or other head sizes")
        return at

    @classmethod
    def from_json(cls, path: str) -> "NilepelConfig":
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
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "layers": [l.to_dict() for l in self.layers], "norm": {"eps": self.norm_eps},
                "embedding": {"scale": self.embedding_scale}}

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def eps_f32(self) -> float:
        return float(np.float32(self.norm_eps))

    @property
    def stop_token_ids(self) -> tuple:
        return ()
