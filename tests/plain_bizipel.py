"""A plain, slow statement of the Bizipel decoder in float64 on the CPU: one function for each mechanism, whole
sequences only (no cache, no batches, no portions).  The oracle of the GPU tests; it shares no code with the package.

Notation: T tokens, W the width, S residual streams; positions count from 0.
"""
from __future__ import annotations

import json
import math
import os

import torch

F64 = torch.float64


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def unit_rms(x, eps):
    """x over its root mean square along the last axis, eps under the root."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def dynamic_tanh(x, alpha, gain, shift):
    return torch.tanh(alpha * x) * gain + shift


def streams_read(xs, w_in):
    """xs [S, T, W] -> the sublayer's input row, sum_s w_in[s] xs[s]."""
    return torch.einsum("s,stw->tw", w_in, xs)


def streams_write(xs, mix, w_out, y):
    """All streams from the old ones: xs'[t] = sum_s mix[s, t] xs[s] + w_out[t] y."""
    return torch.einsum("sr,stw->rtw", mix, xs) + w_out[:, None, None] * y[None]


def visible(T, window, keep_first):
    """[T, T] bool: query i sees key j iff j <= i and (i - j < window or j < keep_first); window None: all j <= i."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = j <= i
    if window is not None:
        seen = seen & ((i - j < window) | (j < keep_first))
    return seen


def window_attention(q, k, v, scale, window, keep_first, r1=None, r2=None, sink_one=True):
    """q [T, H, D], k [T, G, D], v [T, G, E] -> [T, H, E].  Head h reads kv head h // (H / G).  The score of (i, j) is
    scale q_i.k_j - r1[h] ln(1 + r2[h] (i - j)); the softmax's denominator has one more than the visible keys' sum."""
    T, H, _ = q.shape
    G = k.shape[1]
    dist = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).clamp(min=0).to(F64)
    seen = visible(T, window, keep_first)
    out = []
    for h in range(H):
        g = h // (H // G)
        s = scale * (q[:, h] @ k[:, g].T)
        if r1 is not None:
            s = s - r1[h] * torch.log(1.0 + r2[h] * dist)
        e = torch.where(seen, torch.exp(s), torch.zeros_like(s))
        p = e / ((1.0 if sink_one else 0.0) + e.sum(-1, keepdim=True))
        out.append(p @ v[:, g])
    return torch.stack(out, 1)


def matrix_memory(q, k, v, i_pre, f_pre, cap, state=None):
    """q, k [T, H, D] (q already scaled), v [T, H, E], gate pre-activations [T, H] -> (o [T, H, E], state).
    state = (C [H, D, E], n [H, D], m [H]), zero at the start (m too)."""
    T, H, D = q.shape
    E = v.shape[2]
    if state is None:
        state = (torch.zeros(H, D, E, dtype=F64), torch.zeros(H, D, dtype=F64), torch.zeros(H, dtype=F64))
    C, n, m = state
    log_i = cap * torch.tanh(i_pre / cap)
    log_f = torch.nn.functional.logsigmoid(cap * torch.tanh(f_pre / cap))
    out = torch.zeros(T, H, E, dtype=F64)
    for t in range(T):
        m_new = torch.maximum(log_f[t] + m, log_i[t])
        keep, take = torch.exp(log_f[t] + m - m_new), torch.exp(log_i[t] - m_new)
        C = keep[:, None, None] * C + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        m = m_new
        below = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        out[t] = torch.einsum("hde,hd->he", C, q[t]) / below[:, None]
    return out, (C, n, m)


class PlainBizipel:
    def __init__(self, config: dict, tensors: dict):
        self.cfg = config
        self.w = {n: t.to(F64) for n, t in tensors.items()}

    @classmethod
    def from_folder(cls, folder):
        from safetensors.torch import load_file
        with open(os.path.join(folder, "config.json")) as f:
            cfg = json.load(f)
        return cls(cfg, load_file(os.path.join(folder, "model.safetensors")))

    def norm(self, name, x):
        return dynamic_tanh(x, self.w[name + ".alpha"], self.w[name], self.w[name + ".b"])

    def left(self, p, c, h, eps):
        w, T = self.w, h.shape[0]
        H, G, D, E = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
        q = (h @ w[p + "q"].T + w[p + "q.b"]).view(T, H, D)
        k = (h @ w[p + "k"].T + w[p + "k.b"]).view(T, G, D)
        v = (h @ w[p + "v"].T + w[p + "v.b"]).view(T, G, E)
        q = unit_rms(q, eps) * w[p + "q.norm"]
        k = unit_rms(k, eps) * w[p + "k.norm"]
        o = window_attention(q, k, v, c["scale"], c["mask"]["size"], c["mask"]["keep_first"], w[p + "r1"], w[p + "r2"])
        o = o.reshape(T, H * E) * torch.sigmoid(h @ w[p + "g"].T)
        return o @ w[p + "o"].T + w[p + "o.b"]

    def right(self, p, c, h, eps):
        w, T = self.w, h.shape[0]
        H, D, E = c["heads"], c["dim"], c["vdim"]
        q = (h @ w[p + "q"].T).view(T, H, D) * D ** -0.5
        k = (h @ w[p + "k"].T).view(T, H, D)
        v = (h @ w[p + "v"].T).view(T, H, E)
        o, _ = matrix_memory(q, k, v, h @ w[p + "i"].T + w[p + "i.b"], h @ w[p + "f"].T + w[p + "f.b"], c["gate_cap"])
        o = unit_rms(o, eps).reshape(T, H * E) * w[p + "norm"] * torch.sigmoid(h @ w[p + "g"].T)
        return o @ w[p + "o"].T

    def mixer(self, i, layer, h):
        m, eps = layer["mixer"], self.cfg["norm"]["eps"]
        return (m["left_scale"] * self.left(f"l{i}.mix.left.", m["left"], h, eps)
                + m["right_scale"] * self.right(f"l{i}.mix.right.", m["right"], h, eps))

    def feed_forward(self, i, h):
        w = self.w
        return (gelu_tanh(h @ w[f"l{i}.mlp.gate"].T) * (h @ w[f"l{i}.mlp.up"].T)) @ w[f"l{i}.mlp.down"].T

    def forward(self, tokens, residuals=None) -> torch.Tensor:
        """Logits [T, vocab] (float64) of a whole sequence; residuals: a list that receives the residual (summed
        over its streams) after every layer."""
        w, S = self.w, self.cfg.get("streams")
        x = w["embed"][torch.tensor(list(tokens))]
        xs = torch.stack([x] * S) if S is not None else None
        for i, layer in enumerate(self.cfg["layers"]):
            subs = [(1, lambda h, i=i, layer=layer: self.mixer(i, layer, h))]
            if layer.get("mlp") is not None:
                subs.append((2, lambda h, i=i: self.feed_forward(i, h)))
            for q, fn in subs:
                if xs is None:
                    x = x + fn(self.norm(f"l{i}.norm{q}", x))
                else:
                    hc = f"l{i}.hc{q}."
                    y = fn(self.norm(f"l{i}.norm{q}", streams_read(xs, w[hc + "in"])))
                    xs = streams_write(xs, w[hc + "mix"], w[hc + "out"], y)
            if residuals is not None:
                residuals.append(xs.sum(0) if xs is not None else x)
        x = xs.sum(0) if xs is not None else x
        return self.norm("final.norm", x) @ w["embed"].T
