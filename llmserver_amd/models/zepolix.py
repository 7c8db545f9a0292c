"""Zepolix put together from parts, layer by layer, from its typed configuration.

Token rows are normalised behind the embedding and the stream stays in 32-bit.  Every layer is a
:class:`~llmserver_amd.parts.block.PostNormBlock`: a short convolution and attention over a shared latent
(:class:`~llmserver_amd.parts.latent_attention.LatentAttention`, with a sink in the softmax and gated heads), then
routed experts, each normalised on its way out, scaled per channel, and the layer's result averaged with the results
before it.  The norms' weights are stored around zero.  Tensor names: ``embed``, ``embed.norm``, ``l<i>.<...>``,
``final.norm``, ``head``; every name is the tensor's whole name (no ``.weight`` behind it).
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.zepolix import ZepolixConfig
from ..parts import (DepthAverage, LatentAttention, LatentAttentionNames, Linear, NormedTokenEmbedding, PairedRotaryPosition,
                     PostNormBlock, RMSNorm, RoutedExperts, ShortConvolution)
from .decoder import DecoderModel

MIXER_NAMES = LatentAttentionNames(q="q", down="dkv", down_norm="dkv.norm", up_keys="uk", up_values="uv", out="o", sink="sink", gate="g")
BLOCK_NAMES = ("mix", "norm1", "mlp", "norm2", "canon1", "ls1", "ls2")
MODEL_NAMES = ("embed", "l", "final.norm")
HEAD_NAME = "head"
NORM_OFFSET = 1.0           # the norms' stored weights lie around zero


def build_zepolix(config: ZepolixConfig) -> DecoderModel:
    eps, width = config.norm_eps, config.width

    def norm():
        return RMSNorm(width, eps, offset=NORM_OFFSET, tensor="")

    positions = {}
    blocks = []
    for index, layer in enumerate(config.layers):
        sizes = layer.mixer
        position = positions.setdefault((sizes.rot_dims, sizes.rot_base), PairedRotaryPosition(sizes.rot_dims, sizes.rot_base))
        mixer = LatentAttention(width, sizes.heads, sizes.dim, sizes.rot_dim, sizes.vdim, sizes.kv_rank, position, sizes.scale, eps,
                                names=MIXER_NAMES)
        experts = None
        if layer.mlp is not None:
            experts = RoutedExperts(width, layer.mlp.ff, layer.mlp.experts, layer.mlp.top)
        conv = ShortConvolution(width, config.canon_taps, tensor="") if config.canon_taps else None
        blocks.append(PostNormBlock(mixer, norm(), experts, norm() if experts is not None else None, conv=conv, scales=True,
                                    average=DepthAverage(index, len(config.layers) + 1), names=BLOCK_NAMES))
    head = Linear(width, (HEAD_NAME,), (config.vocab,), out_float32=True, bare_names=True)
    return DecoderModel(config, NormedTokenEmbedding(config.vocab, width, norm()), blocks, norm(), head, tie_head=False,
                        names=MODEL_NAMES, layer_name=lambda i: f"l{i}")


register_architecture(ZepolixConfig.MODEL_TYPE, ZepolixConfig, build_zepolix, replace=True)
