"""Typed configuration of the Bizipel decoder, read from config.json's own keys.

    {"architecture": "Bizipel", "vocab": V, "width": W, "streams": S, "norm": {"eps": e},
     "layers": [{"type": "parallel",
                 "mixer": {"left": {"heads", "kv_heads", "dim", "vdim", "scale", "mask": {"size", "keep_first"}},
                           "right": {"heads", "dim", "vdim", "gate_cap"}, "left_scale", "right_scale"},
                 "mlp": {"kind": "dense", "ff": F} | null}, ...]}

Every layer carries its own sizes, so layers may differ from one another; the list's order is the order in which
they run.  `streams` absent: one plain residual.  A key that the model would not honour is an error.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Optional

import numpy as np

from .errors import ConfigError
from .fields import obj as _obj, integer as _int, number as _num


@dataclass(frozen=True)
class WindowAttentionConfig:
    """The left half of a parallel mixer: attention with a kept window."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int           # mask.size
    keep_first: int       # mask.keep_first

    @classmethod
    def from_dict(cls, d, where):
        mask = _obj(d, "mask", where)
        c = cls(_int(d, "heads", where), _int(d, "kv_heads", where), _int(d, "dim", where), _int(d, "vdim", where),
                _num(d, "scale", where), _int(mask, "size", where + ".mask"), _int(mask, "keep_first", where + ".mask", 0))
        if c.heads % c.kv_heads:
            raise ConfigError(f"{where}: heads={c.heads} must be divisible by kv_heads={c.kv_heads}")
        return c

    def to_dict(self):
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
                "mask": {"size": self.window, "keep_first": self.keep_first}}


@dataclass(frozen=True)
class MatrixMemoryConfig:
    """The right half: a matrix memory with exponential gates."""
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @classmethod
    def from_dict(cls, d, where):
        c = cls(_int(d, "heads", where), _int(d, "dim", where), _int(d, "vdim", where), _num(d, "gate_cap", where))
        if not c.gate_cap > 0.0:
            raise ConfigError(f"{where}: gate_cap {c.gate_cap} must be positive")
        return c

    def to_dict(self):
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


@dataclass(frozen=True)
class ParallelLayerConfig:
    left: WindowAttentionConfig
    right: MatrixMemoryConfig
    left_scale: float
    right_scale: float
    ff: Optional[int]     # width of the dense feed-forward; None: the layer has none

    @classmethod
    def from_dict(cls, d, where):
        kind = d.get("type") if isinstance(d, dict) else None
        if kind != "parallel":
            raise ConfigError(f"{where}: layer type {kind!r} (this decoder has 'parallel' layers)")
        m = _obj(d, "mixer", where)
        ff = None
        if d.get("mlp") is not None:
            mlp = _obj(d, "mlp", where)
            if mlp.get("kind") != "dense":
                raise ConfigError(f"{where}.mlp: kind {mlp.get('kind')!r} (this decoder has 'dense' feed-forwards)")
            ff = _int(mlp, "ff", where + ".mlp")
        return cls(WindowAttentionConfig.from_dict(_obj(m, "left", where + ".mixer"), where + ".mixer.left"),
                   MatrixMemoryConfig.from_dict(_obj(m, "right", where + ".mixer"), where + ".mixer.right"),
                   _num(m, "left_scale", where + ".mixer"), _num(m, "right_scale", where + ".mixer"), ff)

    def to_dict(self):
        return {"type": "parallel",
                "mixer": {"left": self.left.to_dict(), "right": self.right.to_dict(), "left_scale": self.left_scale,
                          "right_scale": self.right_scale},
                "mlp": None if self.ff is None else {"kind": "dense", "ff": self.ff}}


@dataclass(frozen=True)
class BizipelConfig:
    vocab: int
    width: int
    layers: tuple
    norm_eps: float
    streams: Optional[int] = None     # copies of the residual (hyper-connections); None: one plain residual

    architecture = "Bizipel"
    max_position_embeddings = None    # positions enter through distances only: no table bounds them
    eos_token_id = None

    @classmethod
    def from_dict(cls, d: dict) -> "BizipelConfig":
        if not isinstance(d.get("layers"), list) or not d["layers"]:
            raise ConfigError("config key 'layers' must be a list with at least one layer")
        streams = None if d.get("streams") is None else _int(d, "streams", "config")
        cfg = cls(_int(d, "vocab", "config"), _int(d, "width", "config"),
                  tuple(ParallelLayerConfig.from_dict(l, f"layers[{i}]") for i, l in enumerate(d["layers"])),
                  _num(_obj(d, "norm", "config"), "eps", "config.norm"), streams)
        if not cfg.norm_eps > 0.0:
            raise ConfigError(f"norm.eps {cfg.norm_eps} must be positive")
        return cfg

    @classmethod
    def from_json(cls, path: str) -> "BizipelConfig":
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
             "layers": [l.to_dict() for l in self.layers], "norm": {"eps": self.norm_eps}}
        if self.streams is not None:
            d["streams"] = self.streams
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
