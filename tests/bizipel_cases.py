"""Small Bizipel configurations for the tests, their model folders (random weights), and the plain model's logits."""
from __future__ import annotations

import copy
import os
import tempfile

import torch

from synaptix_amd.config import BizipelConfig
from synaptix_amd import write_random_model
from plain_bizipel import PlainBizipel


def layer(heads, kv_heads, dim, vdim, window, keep_first, mem_heads, mem_dim, mem_vdim, ff, cap=8.0, scales=(0.7, 0.6),
          scale=None):
    return {"type": "parallel",
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                               "scale": scale if scale is not None else dim ** -0.5,
                               "mask": {"size": window, "keep_first": keep_first}},
                      "right": {"heads": mem_heads, "dim": mem_dim, "vdim": mem_vdim, "gate_cap": cap},
                      "left_scale": scales[0], "right_scale": scales[1]},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def config(vocab, width, streams, layers, eps=1e-6):
    d = {"architecture": "Bizipel", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps}}
    if streams is not None:
        d["streams"] = streams
    return d


# P: two unlike layers (keys and values of unequal size, grouped heads, a window shorter than a page that keeps three
#    first keys; then a window longer than a page that keeps none and a layer without a feed-forward), two streams.
# Q: one stream, a width that is no multiple of 32, a window of exactly one page, more kept keys than a page holds,
#    a memory whose values span two tiles of columns and whose keys are no multiple of four.
# R: four streams, sizes at which the weights lie in fragment order, as many kv heads as heads, a window that no test
#    sequence outgrows.
# S: three streams and sizes that are multiples of nothing (keys of 20 and 12 values, a memory with keys of 3 and 5
#    values, a width of 72, an odd vocabulary), windows of 10 and of 1.
# T: no `streams` key at all: one plain residual with pre-norm layers.
CONFIGS = {
    "S": config(101, 72, 3, [layer(2, 1, 20, 12, 10, 2, 1, 3, 5, 24), layer(3, 3, 12, 20, 1, 0, 2, 7, 9, 40, cap=20.0)]),
    "U": config(77, 50, 2, [layer(1, 1, 6, 10, 3, 1, 1, 4, 6, 22)]),          # a width that is no multiple of 4
    "T": config(200, 64, None, [layer(2, 2, 16, 16, 30, 1, 1, 8, 8, 48), layer(4, 1, 8, 32, 200, 0, 2, 16, 24, 64)]),
    "P": config(300, 64, 2, [layer(4, 2, 16, 24, 20, 3, 2, 8, 16, 96), layer(2, 1, 32, 16, 70, 0, 1, 24, 40, None)]),
    "Q": config(257, 88, 1, [layer(3, 1, 24, 8, 64, 70, 1, 10, 72, 50, cap=3.0), layer(2, 2, 8, 40, 5, 1, 3, 6, 4, 120),
                             layer(1, 1, 40, 40, 33, 2, 2, 16, 16, 64, scales=(1.0, 1.0))], eps=1e-5),
    "R": config(512, 128, 4, [layer(4, 4, 32, 32, 4096, 0, 2, 32, 64, 256), layer(4, 4, 32, 32, 100, 8, 2, 32, 64, 256)]),
}
SEEDS = {"P": 11, "Q": 12, "R": 13, "S": 14, "T": 15, "U": 16}
_tmp = None
_folders, _plain, _logits = {}, {}, {}


def model_folder(name: str) -> str:
    """Random bf16 weights; the gains of the q/k norms are 3 x larger than one so that attention is peaked and a lost
    or wrong key moves the logits, and the matrices are drawn wide enough that every branch carries weight."""
    global _tmp
    if name not in _folders:
        if _tmp is None:
            _tmp = tempfile.TemporaryDirectory(prefix="synaptix_amd_bizipel_")
        cfg = BizipelConfig.from_dict(copy.deepcopy(CONFIGS[name]))
        g = torch.Generator().manual_seed(500 + SEEDS[name])
        extra = {}
        for i, l in enumerate(cfg.layers):
            for n in ("q.norm", "k.norm"):
                extra[f"l{i}.mix.left.{n}"] = (3.0 + 0.3 * torch.randn(l.left.dim, generator=g)).to(torch.bfloat16)
        folder = os.path.join(_tmp.name, name)
        write_random_model(folder, cfg, SEEDS[name], std=0.08, extra_tensors=extra)
        _folders[name] = folder
    return _folders[name]


def plain_logits(name: str, tokens) -> torch.Tensor:
    key = (name, tuple(tokens))
    if key not in _logits:
        if name not in _plain:
            _plain[name] = PlainBizipel.from_folder(model_folder(name))
        _logits[key] = _plain[name].forward(list(tokens))
    return _logits[key]


def tokens_for(name: str, n: int, seed: int) -> list:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, CONFIGS[name]["vocab"], (n,), generator=g).tolist()
