"""A plain, slow statement of the Kamivik decoder in float64 on the CPU: one function for each mechanism, whole
sequences only (no cache, no batches, no portions).  The oracle of the GPU tests; it shares no code with the package.
Keys and values are made for every head from the latent, the way the design is written down; the package moves those
products to the query's side instead.

Notation: T tokens, W the width, H heads, D unrotated and B rotated query/key values a head, E values a head, C the
latent's size; positions count from 0.
"""
from __future__ import annotations

import json
import math
import os

import torch

F64 = torch.float64


def gelu(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def rms_norm(x, gain, eps):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * gain


def turn_pairs(x, positions, base, dims):
    """x [T, ..., n]: the pairs (2i, 2i + 1), i < dims / 2, turned by positions[t] * base^(-2i / dims); the rest passes."""
    if dims == 0:
        return x.clone()
    i = torch.arange(dims // 2, dtype=F64)
    angle = positions.to(F64)[:, None] * base ** (-2.0 * i / dims)           # [T, dims / 2]
    while angle.dim() < x.dim():
        angle = angle.unsqueeze(1)
    c, s = torch.cos(angle), torch.sin(angle)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    y = x.clone()
    y[..., 0:dims:2] = u * c - v * s
    y[..., 1:dims:2] = v * c + u * s
    return y


def visible(T, window):
    """[T, T] bool: query i sees key j iff 0 <= i - j (< window, if there is one)."""
    d = torch.arange(T)[:, None] - torch.arange(T)[None, :]
    return (d >= 0) if window is None else (d >= 0) & (d < window)


def attention(q, k, v, scale, window):
    """q, k [T, H, n], v [T, H, E] -> [T, H, E]: softmax over the visible keys of scale q_i . k_j."""
    T = q.shape[0]
    s = scale * torch.einsum("ihd,jhd->hij", q, k)
    s = s.masked_fill(~visible(T, window)[None], -math.inf)
    return torch.einsum("hij,jhe->ihe", torch.softmax(s, -1), v)


def shared_row_attention(q, rows, n_values, scale, window):
    """Every head's query against one key row a token whose first n_values values are its value:
    q [T, H, R], rows [T, R] -> [T, H, n_values]."""
    T, H, R = q.shape
    return attention(q, rows[:, None, :].expand(T, H, R), rows[:, None, :n_values].expand(T, H, n_values), scale, window)


def latent_attention(h, w, p, c, eps, per_value_gate, positions=None):
    """h [T, W]; w: the tensors; p: the mixer's prefix; c: its sizes (config.json's mixer entry)."""
    T = h.shape[0]
    H, D, B, E, C = c["heads"], c["dim"], c["rot_dim"], c["vdim"], c["kv_rank"]
    pos = torch.arange(T) if positions is None else positions
    q = (h @ w[p + "q"].T).view(T, H, D + B)
    down = h @ w[p + "dkv"].T
    lat = rms_norm(down[:, :C], w[p + "dkv.norm"], eps)
    k_rot = turn_pairs(down[:, C:], pos, c["rot"]["base"], c["rot"]["dims"])                 # [T, B], one for all heads
    q_rot = turn_pairs(q[..., D:], pos, c["rot"]["base"], c["rot"]["dims"])
    k = torch.cat([(lat @ w[p + "uk"].T).view(T, H, D), k_rot[:, None, :].expand(T, H, B)], -1)
    v = (lat @ w[p + "uv"].T).view(T, H, E)
    o = attention(torch.cat([q[..., :D], q_rot], -1), k, v, c["scale"], c.get("mask", {}).get("size"))
    g = torch.sigmoid(h @ w[p + "g"].T)
    o = o.reshape(T, H * E) * g if per_value_gate else (o * g[:, :, None]).reshape(T, H * E)
    return o @ w[p + "o"].T


def route(h, w_router, bias, top):
    """(experts [T, top], weights [T, top]): the largest logits, softmax over those alone."""
    z = h @ w_router.T + bias
    chosen = torch.topk(z, top, dim=-1)
    return chosen.indices, torch.softmax(chosen.values, -1)


def routed_experts(h, w, p, c):
    ids, weights = route(h, w[p + "router"], w[p + "router.b"], c["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(ids[t].tolist(), weights[t]):
            out[t] += a * (w[p + f"e{e}.down"] @ gelu(w[p + f"e{e}.up"] @ h[t]))
    return out


class PlainKamivik:
    def __init__(self, cfg: dict, tensors: dict):
        self.cfg = cfg
        self.w = {n: t.to(F64) for n, t in tensors.items()}

    @classmethod
    def from_folder(cls, folder):
        from safetensors.torch import load_file
        with open(os.path.join(folder, "config.json")) as f:
            cfg = json.load(f)
        return cls(cfg, load_file(os.path.join(folder, "model.safetensors")))

    def forward(self, tokens, residuals=None) -> torch.Tensor:
        """Logits [T, vocab] of one sequence from its first token."""
        cfg, w = self.cfg, self.w
        eps, m = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
        x = w["embed"][torch.tensor(tokens)]
        for i, layer in enumerate(cfg["layers"]):
            p = f"l{i}."
            h = rms_norm(x, w[p + "norm1"], eps)
            y = latent_attention(h, w, p + "mix.", layer["mixer"], eps, layer["type"] == "latent_attention_2") * w[p + "ls1"]
            if layer["mlp"] is not None:
                y = y + routed_experts(h, w, p + "mlp.", layer["mlp"]) * w[p + "ls2"]
            x = x + m * y
            if residuals is not None:
                residuals.append(x.clone())
        return rms_norm(x, w["final.norm"], eps) @ w["head"].T
