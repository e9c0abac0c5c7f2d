"""Small Kamivik configurations for the tests, their model folders (random weights), and the plain model's logits."""
from __future__ import annotations

import copy
import os
import tempfile

import torch

from synaptix_amd.config import KamivikConfig
from synaptix_amd import write_random_model
from plain_kamivik import PlainKamivik


def layer(kind, heads, dim, rot_dim, vdim, rank, window=None, ff=None, experts=4, top=2, base=10000.0, dims=None,
          scale=None):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank,
             "scale": scale if scale is not None else 6.0 * (dim + rot_dim) ** -0.5,
             "rot": {"base": base, "dims": rot_dim if dims is None else dims}}
    if kind == "latent_attention_2":
        mixer["mask"] = {"size": window}
    mlp = None if ff is None else {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def config(vocab, width, layers, eps=1e-6, mult=1.0):
    return {"architecture": "Kamivik", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps},
            "residual_mult": mult}


A1, A2 = "latent_attention", "latent_attention_2"
# P: a window shorter than a page before a layer that sees everything, unlike sizes in every layer, part of the
#    rotated values left unturned, one layer without a feed-forward.
# Q: sizes that are multiples of nothing (a width of 72, keys of 12 + 6, a latent of 20, an odd vocabulary), a window
#    of exactly one page and one of a page and a token, all experts of two, no residual factor.
# R: sizes at which the products by group run on the matrix cores and the weights lie in fragment order; a window that
#    no test sequence outgrows; sixteen experts.
# S: one head, a window of one (a query sees itself alone) and of two, a latent smaller than a head, one expert only.
# T: no rotated part at all in one layer, nothing turned in the other.
# U: one expert of four for each token: a choice that the rounding of bfloat16 activations can turn at a near tie of
#    two logits changes that token's result altogether, so this one is run in 32-bit only.
CONFIGS = {
    "P": config(300, 64, [layer(A2, 4, 16, 8, 24, 32, window=20, ff=48, experts=6, top=2, dims=4),
                          layer(A1, 2, 32, 16, 16, 48, ff=None, base=500.0),
                          layer(A1, 3, 8, 4, 40, 24, ff=32, experts=5, top=3)], mult=0.5),
    "Q": config(257, 72, [layer(A2, 3, 12, 6, 10, 20, window=64, ff=40, experts=3, top=2),
                          layer(A2, 2, 20, 2, 12, 36, window=65, ff=24, experts=2, top=2),
                          layer(A1, 5, 6, 10, 14, 12, ff=56, experts=7, top=4)], eps=1e-5),
    "R": config(512, 128, [layer(A1, 4, 32, 32, 32, 64, ff=64, experts=16, top=4),
                           layer(A2, 8, 32, 16, 32, 96, window=4096, ff=96, experts=8, top=2, base=1e6)], mult=0.7),
    "S": config(101, 40, [layer(A2, 1, 8, 4, 8, 6, window=1, ff=16, experts=1, top=1),
                          layer(A2, 1, 4, 8, 12, 10, window=2, ff=None)], mult=1.3),
    "T": config(200, 48, [layer(A1, 2, 16, 0, 16, 24, ff=32, experts=4, top=2, dims=0),
                          layer(A2, 2, 8, 8, 8, 16, window=33, ff=32, experts=4, top=3, dims=0)]),
    "U": config(150, 56, [layer(A1, 2, 8, 8, 12, 16, ff=24, experts=4, top=1),
                          layer(A2, 2, 12, 4, 8, 20, window=7, ff=40, experts=6, top=1)], mult=0.9),
}
SEEDS = {"P": 21, "Q": 22, "R": 23, "S": 24, "T": 25, "U": 26}


def dtypes_of(name: str) -> list:
    return ["float32"] if name == "U" else ["float32", "bfloat16"]


def cases(names) -> list:
    """(configuration, engine type) pairs for pytest.mark.parametrize."""
    return [(n, d) for n in names for d in dtypes_of(n)]
_tmp = None
_folders, _plain, _logits = {}, {}, {}


def model_folder(name: str) -> str:
    """Random bf16 weights, drawn wide enough that every branch carries weight; the configurations' scales make the
    attention peaked, so that a lost or wrong key moves the logits.  The routers' weights are drawn five times wider
    still: their logits then lie several units apart, and where the rounding of bfloat16 activations turns a near tie
    between the last expert chosen and the first one left out, the expert in question carries a weight of a few
    percent (the exact choice is checked in 32-bit, and on equal inputs in the routers' own test)."""
    global _tmp
    if name not in _folders:
        if _tmp is None:
            _tmp = tempfile.TemporaryDirectory(prefix="synaptix_amd_kamivik_")
        cfg = KamivikConfig.from_dict(copy.deepcopy(CONFIGS[name]))
        folder = os.path.join(_tmp.name, name)
        g = torch.Generator().manual_seed(700 + SEEDS[name])
        extra = {}
        for i, l in enumerate(cfg.layers):
            if l.mlp is not None:
                extra[f"l{i}.mlp.router"] = (0.4 * torch.randn(l.mlp.experts, cfg.width, generator=g)).to(torch.bfloat16)
        write_random_model(folder, cfg, SEEDS[name], std=0.08, gain_std=0.3, extra_tensors=extra)
        _folders[name] = folder
    return _folders[name]


def plain_model(name: str) -> PlainKamivik:
    if name not in _plain:
        _plain[name] = PlainKamivik.from_folder(model_folder(name))
    return _plain[name]


def plain_logits(name: str, tokens) -> torch.Tensor:
    key = (name, tuple(tokens))
    if key not in _logits:
        _logits[key] = plain_model(name).forward(list(tokens))
    return _logits[key]


def tokens_for(name: str, n: int, seed: int) -> list:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, CONFIGS[name]["vocab"], (n,), generator=g).tolist()
