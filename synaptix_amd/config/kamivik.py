"""Typed configuration of the Kamivik decoder, read from config.json's own keys.

    {"architecture": "Kamivik", "vocab": V, "width": W, "norm": {"eps": e}, "residual_mult": m,
     "layers": [{"type": "latent_attention" | "latent_attention_2",
                 "mixer": {"heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot": {"base", "dims"},
                           "mask": {"size"}},                       (mask: the second type only)
                 "mlp": {"kind": "moe", "expert": {"ff": F}, "router": {"experts": E, "top": k}} | null}, ...]}

Every layer carries its own sizes; the list's order is the order in which the layers run.  The two types of layer
differ in what a query sees and in how the heads' results are gated:
    latent_attention     every earlier key;                one gate for each head
    latent_attention_2   the last mask.size keys (itself included);  one gate for each value of each head
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Optional

import numpy as np

from .errors import ConfigError
from .fields import obj as _obj, integer as _int, number as _num

LAYER_TYPES = ("latent_attention", "latent_attention_2")


@dataclass(frozen=True)
class LatentMixerConfig:
    heads: int
    dim: int              # unrotated query/key values of a head
    rot_dim: int          # rotated query/key values of a head (the key's are shared by all heads)
    vdim: int
    kv_rank: int          # size of the latent that keys and values are made from
    scale: float
    rot_base: float
    rot_dims: int         # how many of the rot_dim values are turned (pairs 2i, 2i + 1)
    window: Optional[int]  # mask.size; None: every earlier key

    @classmethod
    def from_dict(cls, d, where, windowed: bool):
        rot = _obj(d, "rot", where)
        window = _int(_obj(d, "mask", where), "size", where + ".mask") if windowed else None
        dim, rot_dim = _int(d, "dim", where), _int(d, "rot_dim", where, 0)
        scale = _num(d, "scale", where) if d.get("scale") is not None else float(dim + rot_dim) ** -0.5
        c = cls(_int(d, "heads", where), dim, rot_dim, _int(d, "vdim", where), _int(d, "kv_rank", where), scale,
                _num(rot, "base", where + ".rot"), _int(rot, "dims", where + ".rot", 0), window)
        if c.rot_dims % 2 or c.rot_dims > c.rot_dim:
            raise ConfigError(f"{where}.rot: dims {c.rot_dims} must be even and at most rot_dim {c.rot_dim}")
        if not c.rot_base > 0.0:
            raise ConfigError(f"{where}.rot: base {c.rot_base} must be positive")
        return c

    def to_dict(self):
        d = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
             "scale": self.scale, "rot": {"base": self.rot_base, "dims": self.rot_dims}}
        if self.window is not None:
            d["mask"] = {"size": self.window}
        return d


@dataclass(frozen=True)
class ExpertsConfig:
    ff: int
    experts: int
    top: int

    @classmethod
    def from_dict(cls, d, where):
        if d.get("kind") != "moe":
            raise ConfigError(f"{where}: kind {d.get('kind')!r} (this decoder's feed-forward is 'moe')")
        router = _obj(d, "router", where)
        c = cls(_int(_obj(d, "expert", where), "ff", where + ".expert"), _int(router, "experts", where + ".router"),
                _int(router, "top", where + ".router"))
        if c.top > c.experts:
            raise ConfigError(f"{where}.router: top {c.top} of {c.experts} experts")
        return c

    def to_dict(self):
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}


@dataclass(frozen=True)
class KamivikLayerConfig:
    type: str
    mixer: LatentMixerConfig
    mlp: Optional[ExpertsConfig]

    @classmethod
    def from_dict(cls, d, where):
        kind = d.get("type") if isinstance(d, dict) else None
        if kind not in LAYER_TYPES:
            raise ConfigError(f"{where}: layer type {kind!r} (this decoder has {', '.join(LAYER_TYPES)})")
        mlp = None if d.get("mlp") is None else ExpertsConfig.from_dict(_obj(d, "mlp", where), where + ".mlp")
        return cls(kind, LatentMixerConfig.from_dict(_obj(d, "mixer", where), where + ".mixer",
                                                     windowed=kind == "latent_attention_2"), mlp)

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class KamivikConfig:
    vocab: int
    width: int
    layers: tuple
    norm_eps: float
    residual_mult: float = 1.0

    architecture = "Kamivik"
    max_position_embeddings = None    # the rotation's table bounds the positions (the mixers' position parts say how far)
    eos_token_id = None

    @classmethod
    def from_dict(cls, d: dict) -> "KamivikConfig":
        if not isinstance(d.get("layers"), list) or not d["layers"]:
            raise ConfigError("config key 'layers' must be a list with at least one layer")
        cfg = cls(_int(d, "vocab", "config"), _int(d, "width", "config"),
                  tuple(KamivikLayerConfig.from_dict(l, f"layers[{i}]") for i, l in enumerate(d["layers"])),
                  _num(_obj(d, "norm", "config"), "eps", "config.norm"),
                  _num(d, "residual_mult", "config") if d.get("residual_mult") is not None else 1.0)
        if not cfg.norm_eps > 0.0:
            raise ConfigError(f"norm.eps {cfg.norm_eps} must be positive")
        return cfg

    @classmethod
    def from_json(cls, path: str) -> "KamivikConfig":
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
                "residual_mult": self.residual_mult}

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def eps_f32(self) -> float:
        return float(np.float32(self.norm_eps))

    @property
    def stop_token_ids(self) -> tuple:
        return ()
