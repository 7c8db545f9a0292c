"""Barotar put together from parts, layer by layer, from its typed configuration.

The stream starts as the embedding row and stays in 32-bit.  Every layer is a
:class:`~llmserver_amd.parts.block.SandwichBlock`: a norm in front of each sublayer and one behind it.  A layer's mixer
is a gated linear recurrence (:class:`~llmserver_amd.parts.recurrent.GatedLinearAttention`) or two mixers side by side
(:class:`~llmserver_amd.parts.parallel.ParallelMixers`): windowed softmax attention with grouped heads, q/k norm, a
rotation of neighbouring pairs on part of a head, capped scores and a sink, beside an RWKV-style time mixing
(:class:`~llmserver_amd.parts.recurrent.TimeMixing`).  Its feed-forward is dense and gated (tanh form of GELU), routed
experts with sigmoid scores and groups, or absent.  The head is the embedding table.  Tensor names: ``embed``,
``l<i>.<...>``, ``final.norm``; every name is the tensor's whole name (no ``.weight`` behind it).
"""
from __future__ import annotations

from ..config.barotar import DEFAULT_LOW_RANK, BarotarConfig, DenseSizes, GLASizes
from ..config.registry import register_architecture
from ..parts import (AttentionNames, GatedLinearAttention, GatedMLP, GatedMLPNames, GQAttention, Linear, NoPosition, PairedRotaryPosition,
                     ParallelMixers, RMSNorm, RoutedExperts, SandwichBlock, TimeMixing, TokenEmbedding)
from .decoder import DecoderModel

ATTENTION_NAMES = AttentionNames(qkv=("q", "k", "v"), out="o", q_norm="q.norm", k_norm="k.norm")
MLP_NAMES = GatedMLPNames(gate_up=("gate", "up"), down="down")
BLOCK_NAMES = ("norm1", "mix", "norm1b", "norm2", "mlp", "norm2b")
MODEL_NAMES = ("embed", "l", "final.norm")
HEAD_NAME = "head"          # (no checkpoint has it: the head is the embedding table)
EXPERT_SLOPE = 1.702        # the experts' activation is g * sigmoid(1.702 g) (fixed by the design, as is the tanh form of GELU)


def build_barotar(config: BarotarConfig) -> DecoderModel:
    eps, width = config.norm_eps, config.width

    def norm():
        return RMSNorm(width, eps, tensor="")

    positions = {}
    blocks = []
    for layer in config.layers:
        sizes = layer.mixer
        if isinstance(sizes, GLASizes):
            mixer = GatedLinearAttention(width, sizes.heads, sizes.dim, sizes.vdim, sizes.tau, eps, low=sizes.low, default_low=DEFAULT_LOW_RANK)
        else:
            left, right = sizes.left, sizes.right
            key = (left.rot_dims, left.rot_base)
            if key not in positions:
                positions[key] = PairedRotaryPosition(left.rot_dims, left.rot_base) if left.rot_dims else NoPosition()
            attention = GQAttention(width, left.heads, left.kv_heads, left.dim, positions[key], qk_norm_eps=eps, window=left.window,
                                    scale=left.scale, names=ATTENTION_NAMES, sinks="sink", softcap=left.softcap, value_dim=left.vdim,
                                    bare_names=True)
            mixing = TimeMixing(width, right.heads, right.dim, eps, low=right.low, default_low=DEFAULT_LOW_RANK)
            mixer = ParallelMixers(attention, mixing, sizes.left_scale, sizes.right_scale)
        if layer.mlp is None:
            blocks.append(SandwichBlock(norm(), mixer, norm(), names=BLOCK_NAMES))
            continue
        if isinstance(layer.mlp, DenseSizes):
            feed = GatedMLP(width, layer.mlp.ff, "gelu_tanh", names=MLP_NAMES, bare_names=True)
        else:
            feed = RoutedExperts(width, layer.mlp.ff, layer.mlp.experts, layer.mlp.top, scoring="sigmoid",
                                 groups=(layer.mlp.groups, layer.mlp.keep), activation="clamped", limit=layer.mlp.limit, reads_stream=False)
        blocks.append(SandwichBlock(norm(), mixer, norm(), norm(), feed, norm(), names=BLOCK_NAMES))
    head = Linear(width, (HEAD_NAME,), (config.vocab,), out_float32=True, bare_names=True)
    return DecoderModel(config, TokenEmbedding(config.vocab, width, tensor="", wide=True), blocks, norm(), head, tie_head=True,
                        names=MODEL_NAMES, layer_name=lambda i: f"l{i}")


register_architecture(BarotarConfig.MODEL_TYPE, BarotarConfig, build_barotar, replace=True)
