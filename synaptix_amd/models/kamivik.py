"""The Kamivik decoder put together from parts, and its entry in the registry.

Every layer: one RMSNorm whose output both sublayers read (parts.ParallelBlock), x <- x + m (ls1 * mixer(h) +
ls2 * ff(h)) with a scale for every channel of each sublayer's result and one factor m for the model.  The mixer is
latent attention (parts.LatentAttention): keys and values are made from one small latent a token, which is all the
cache holds beside one rotated key part; layers of the first type see every earlier key and gate each head with one
number, layers of the second see a sliding window and gate every value.  The feed-forward is a mixture of small
ungated experts behind a router with a bias (parts.RoutedExperts), or none.  Layers take their sizes from their own
entry of config.json's `layers`, in its order.
Tensor names: embed; l<i>.norm1; l<i>.mix.q|dkv|dkv.norm|uk|uv|g|o; l<i>.mlp.e<j>.up|down, l<i>.mlp.router(.b);
l<i>.ls1|ls2; final.norm; head.
"""
from __future__ import annotations

from ..config.kamivik import KamivikConfig
from ..config.registry import register_architecture
from ..parts import RmsNorm, RotaryInterleaved, LatentAttention, RoutedExperts, ParallelBlock
from .decoder import DecoderModel, LayerRun, TokenEmbedding, OutputHead

DEFAULT_POSITIONS = 1 << 16      # rows of the rotation's tables when the caller names no longest sequence


def build_kamivik(cfg: KamivikConfig, max_positions: int | None = None) -> DecoderModel:
    W, eps = cfg.width, cfg.eps_f32
    embedding = TokenEmbedding("embed", cfg.vocab, W)
    blocks = []
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.", layer.mixer
        position = RotaryInterleaved(m.rot_base, m.rot_dims, max_positions or DEFAULT_POSITIONS)
        mixer = LatentAttention(p + "mix.", W, m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, position=position,
                                norm_eps=eps, scale=m.scale, window=m.window,
                                gate="value" if layer.type == "latent_attention_2" else "head")
        ff = None
        if layer.mlp is not None:
            ff = RoutedExperts(p + "mlp.", W, layer.mlp.ff, layer.mlp.experts, layer.mlp.top, activation="gelu")
        blocks.append(ParallelBlock(p, W, RmsNorm(p + "norm1", W, eps), mixer, ff, mult=cfg.residual_mult))
    schedule = [LayerRun(i, i) for i in range(len(blocks))]
    return DecoderModel(cfg, embedding, blocks, schedule, RmsNorm("final.norm", W, eps), OutputHead("head", cfg.vocab, W))


KAMIVIK = register_architecture("Kamivik", KamivikConfig, build_kamivik, model_types=("kamivik",))
