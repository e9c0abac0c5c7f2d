"""The Bizipel decoder put together from parts, and its entry in the registry.

Every layer: a residual in `streams` copies with hyper-connections around two sublayers (parts.HyperConnectionBlock),
dynamic tanh in place of the norms, a mixer that is two mixers side by side reading the same input
(parts.ParallelMixers): on the left gated attention with a kept window, a logarithmic distance bias on the scores
and a sink in the softmax (parts.GatedWindowAttention), on the right a matrix memory (parts.MatrixMemory); then a
dense gated feed-forward with the tanh form of GELU, or none.  The output head is the embedding table.  Layers take
their sizes from their own entry of config.json's `layers`, in its order.
Tensor names: embed; l<i>.norm1|norm2 (+ .alpha, .b); l<i>.mix.left.*, l<i>.mix.right.*; l<i>.mlp.gate|up|down;
l<i>.hc1|hc2.in|out|mix; final.norm (+ .alpha, .b).
"""
from __future__ import annotations

from ..config.bizipel import BizipelConfig
from ..config.registry import register_architecture
from ..parts import (DynamicTanh, RmsNorm, LogDistanceBias, GatedWindowAttention, MatrixMemory, ParallelMixers, GatedMlp,
                     HyperConnectionBlock, PreNormBlock)
from .decoder import DecoderModel, LayerRun, TokenEmbedding, OutputHead


def build_bizipel(cfg: BizipelConfig, max_positions: int | None = None) -> DecoderModel:
    W, eps = cfg.width, cfg.eps_f32
    embedding = TokenEmbedding("embed", cfg.vocab, W)
    blocks = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        a, m = layer.left, layer.right
        left = GatedWindowAttention(p + "mix.left.", W, a.heads, a.kv_heads, a.dim, a.vdim,
                                    position=LogDistanceBias(p + "mix.left.", a.heads), qk_norm_eps=eps, scale=a.scale,
                                    window=a.window, keep_first=a.keep_first, sink_one=True, bias=True, out_bias=True,
                                    gate=True)
        right = MatrixMemory(p + "mix.right.", W, m.heads, m.dim, m.vdim, norm_eps=eps, gate_cap=m.gate_cap)
        mixer = ParallelMixers([left, right], [layer.left_scale, layer.right_scale])
        norm2 = ff = None
        if layer.ff is not None:
            norm2 = DynamicTanh(p + "norm2", W)
            ff = GatedMlp(p + "mlp.", W, layer.ff, "gelu_tanh", names=("gate", "up", "down"))
        if cfg.streams is not None:
            blocks.append(HyperConnectionBlock(p, cfg.streams, DynamicTanh(p + "norm1", W), mixer, norm2, ff))
        else:
            if ff is None:
                raise ValueError(f"layer {i}: a layer without a feed-forward needs the residual streams' block")
            blocks.append(PreNormBlock(DynamicTanh(p + "norm1", W), mixer, norm2, ff))
    schedule = [LayerRun(i, i) for i in range(len(blocks))]
    final_norm = DynamicTanh("final.norm", W)
    head = OutputHead("head", cfg.vocab, W, tied_to=embedding)
    return DecoderModel(cfg, embedding, blocks, schedule, final_norm, head, streams=cfg.streams)


BIZIPEL = register_architecture("Bizipel", BizipelConfig, build_bizipel, model_types=("bizipel",))
