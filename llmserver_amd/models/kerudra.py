"""Kerudra put together from parts, layer by layer, from its typed configuration.

The embedding row, times a constant, starts ``streams`` equal residual streams in 32-bit (one, where the
configuration names none).  Every layer is a :class:`~llmserver_amd.parts.block.MultiStreamBlock`: a mixer and,
unless the layer has none, a plain feed-forward with the squared rectifier, each under an RMS norm of what it reads
from the streams and each writing its result, times ``residual_mult``, back through its hyper-connection.  A layer's
mixer is softmax attention with grouped heads whose values are its keys
(:class:`~llmserver_amd.parts.attention.GQAttention`), windowed attention over a shared latent with a gate per channel
(:class:`~llmserver_amd.parts.latent_attention.LatentAttention`), or a matrix memory with exponential gates
(:class:`~llmserver_amd.parts.recurrent.MatrixMemory`).  A run of layers may be passed several times with the same
weights; every pass keeps a cache or state of its own, so the order of calls names a block several times and a
cache once.  The head is the embedding table (unscaled) behind the model's norm of the summed streams, times
``logit_scale``.  Tensor names: ``embed``, ``l<i>.<...>``, ``final.norm``; every name is the tensor's whole name.
"""
from __future__ import annotations

from ..config.kerudra import KerudraConfig, MatrixMemorySizes, SharedValueAttentionSizes
from ..config.registry import register_architecture
from ..parts import (AttentionNames, GQAttention, HyperConnection, LatentAttention, LatentAttentionNames, Linear, MatrixMemory,
                     MatrixMemoryNames, MultiStreamBlock, NoPosition, PairedRotaryPosition, PlainMLP, RotaryPosition, StreamReadNorm,
                     TokenEmbedding)
from .decoder import DecoderModel, LayerCall

ATTENTION_NAMES = AttentionNames(qkv=("q", "k"), out="o")
LATENT_NAMES = LatentAttentionNames(q="q", down="dkv", down_norm="dkv.norm", up_keys="uk", up_values="uv", out="o", sink=None, gate="g")
MEMORY_NAMES = MatrixMemoryNames()
BLOCK_NAMES = ("norm1", "mix", "norm2", "mlp", "hc1", "hc2")
CONNECTION_NAMES = ("in", "out", "mix")
MODEL_NAMES = ("embed", "l", "final.norm")
HEAD_NAME = "head"          # (no checkpoint has it: the head is the embedding table)
BIAS_SUFFIX = ".b"
ACTIVATION = "relu2"        # fixed by the design, as are the biases of queries and keys and the floor of the memory's denominator
MEMORY_FLOOR = 1e-6


def build_kerudra(config: KerudraConfig) -> DecoderModel:
    eps, width = config.norm_eps, config.width
    streams = config.streams or 1
    learned = config.streams > 0

    def norm(scale=1.0):
        return StreamReadNorm(width, eps, streams, tensor="", scale=scale)

    def connection():
        return HyperConnection(streams, config.residual_mult, learned, CONNECTION_NAMES)

    positions = {}

    def position(kind, dims, base):
        if not dims:
            return NoPosition()
        if (kind, dims, base) not in positions:
            positions[(kind, dims, base)] = kind(dims, base) if kind is PairedRotaryPosition else kind(dims, base, precise=True)
        return positions[(kind, dims, base)]

    blocks = []
    for layer in config.layers:
        sizes = layer.mixer
        if isinstance(sizes, SharedValueAttentionSizes):
            mixer = GQAttention(width, sizes.heads, sizes.kv_heads, sizes.dim, position(RotaryPosition, sizes.rot_dims, sizes.rot_base),
                                bias=True, out_bias=False, window=sizes.window, scale=sizes.scale, names=ATTENTION_NAMES, bare_names=True,
                                bias_suffix=BIAS_SUFFIX, values_are_keys=True)
        elif isinstance(sizes, MatrixMemorySizes):
            mixer = MatrixMemory(width, sizes.heads, sizes.dim, sizes.vdim, sizes.gate_cap, eps, MEMORY_FLOOR, MEMORY_NAMES)
        else:
            mixer = LatentAttention(width, sizes.heads, sizes.dim, sizes.rot_dim, sizes.vdim, sizes.kv_rank,
                                    position(PairedRotaryPosition, sizes.rot_dims, sizes.rot_base), sizes.scale, eps, names=LATENT_NAMES,
                                    window=sizes.window, gate_per_channel=True)
        if layer.mlp is None:
            blocks.append(MultiStreamBlock(norm(), mixer, connection(), names=BLOCK_NAMES))
        else:
            feed = PlainMLP(width, layer.mlp.ff, ACTIVATION, names=("up", "down"), bare_names=True)
            blocks.append(MultiStreamBlock(norm(), mixer, connection(), norm(), feed, connection(), names=BLOCK_NAMES))
    # every run of a layer has a cache or state of its own; the weights are the block's
    order = [LayerCall(block, run) for run, block in enumerate(config.layer_runs())]
    head = Linear(width, (HEAD_NAME,), (config.vocab,), out_float32=True, bare_names=True)
    embedding = TokenEmbedding(config.vocab, width, tensor="", wide=True, scale=config.embedding_scale, streams=streams)
    return DecoderModel(config, embedding, blocks, norm(config.logit_scale), head, tie_head=True, order=order, names=MODEL_NAMES,
                        layer_name=lambda i: f"l{i}")


register_architecture(KerudraConfig.MODEL_TYPE, KerudraConfig, build_kerudra, replace=True)
