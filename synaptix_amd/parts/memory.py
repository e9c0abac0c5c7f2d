"""Mixers that keep a state of fixed size for each sequence instead of keys and values.

MatrixMemory: the matrix memory with exponential gates and a running maximum (csrc/matrix_memory.hip has the
equations).  q, k, v, an output gate and the two gates of the cell come from one fused projection; each head's
result is divided by its root mean square, multiplied by a gain over all heads' values and by sigmoid(gate), then
the output product.  Gates, the state and everything between the projections and the output product are 32-bit in
both engine types; the state starts at zero when a slot is taken and is carried from step to step.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.source import TensorSpec
from .base import StateNeed
from .linear import linear, linear_for_sum
from .mixer import Mixer, _projection


class MatrixMemory(Mixer):
    takes_scaled_rows = False
    capturable = True

    NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "i": "i", "f": "f", "bias": ".b"}

    def __init__(self, prefix: str, hidden: int, n_heads: int, dim: int, v_dim: int, *, norm_eps: float,
                 gate_cap: float | None = None, q_scale: float | None = None, names: dict | None = None):
        self.prefix, self.hidden, self.nh, self.dim, self.vdim = prefix, hidden, n_heads, dim, v_dim
        self.norm_eps = float(norm_eps)
        self.gate_cap = float(gate_cap) if gate_cap else 0.0          # 0: the gates' pre-activations are not capped
        self.q_scale = float(q_scale) if q_scale is not None else dim ** -0.5
        self.names = dict(self.NAMES, **(names or {}))
        self.w_in = self.w_o = self.gain = self.i_bias = self.f_bias = None

    def _n(self, key, bias=False):
        return self.prefix + self.names[key] + (self.names["bias"] if bias else "")

    def _widths(self):
        H = self.nh
        return [("q", H * self.dim), ("k", H * self.dim), ("v", H * self.vdim), ("g", H * self.vdim), ("i", H), ("f", H)]

    def tensor_specs(self):
        specs = {self._n(k): TensorSpec((n, self.hidden)) for k, n in self._widths()}
        specs[self._n("o")] = TensorSpec((self.hidden, self.nh * self.vdim))
        specs[self._n("norm")] = TensorSpec((self.nh * self.vdim,), "gain")
        specs[self._n("i", True)] = TensorSpec((self.nh,), "bias")
        specs[self._n("f", True)] = TensorSpec((self.nh,), "bias")
        return specs

    def load(self, get):
        self.w_in = _projection(torch.cat([get(self._n(k)) for k, _ in self._widths()], 0))
        self.w_o = _projection(get(self._n("o")))
        self.gain = get(self._n("norm")).float().contiguous()
        self.i_bias = get(self._n("i", True)).float().contiguous()
        self.f_bias = get(self._n("f", True)).float().contiguous()

    def cache_need(self):
        return StateNeed((self.nh, ops.matrix_memory_state_size(self.dim, self.vdim)))

    def check(self, dtype):
        if self.dim > ops.MATRIX_MEMORY_MAX_DIM:
            raise ValueError(f"{self.prefix}: keys of {self.dim} values (at most {ops.MATRIX_MEMORY_MAX_DIM})")

    def forward(self, h, ctx, cache, owner=True):
        N, H = h.shape[0], self.nh
        proj = linear(h, self.w_in, torch.float32)          # [N, q | k | v | gate | i | f] float
        raw = torch.empty((N, H * self.vdim), dtype=torch.float32, device=h.device)
        ops.matrix_memory_scan(proj, self.i_bias, self.f_bias, self.gate_cap, self.q_scale, cache.state, ctx.seq_start,
                               ctx.seq_slot, raw, H, self.dim, self.vdim, chunked=not ctx.one_token_each,
                               scratch=ctx.scratch)
        o = torch.empty((N, H * self.vdim), dtype=h.dtype, device=h.device)
        ops.head_norm_gate(raw, self.gain, self.norm_eps, proj[:, 2 * H * self.dim + H * self.vdim:], o, H, self.vdim)
        return linear_for_sum(o, self.w_o)
