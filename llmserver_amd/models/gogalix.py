"""Gogalix put together from parts, layer by layer, from its typed configuration.

The embedding row, times a constant, starts a residual stream in 32-bit.  Every layer is a
:class:`~llmserver_amd.parts.block.ParallelGatedBlock`: one RMS norm whose weight is a single number, read by the
mixer and by the feed-forward alike; each result is multiplied by a per-channel scale and by a sigmoid gate per channel
(a projection of the normed rows, with a bias) before both join the stream.  A layer's mixer is differential attention
over a window (:class:`~llmserver_amd.parts.differential.DifferentialAttention`; a layer may read the keys and values of
an earlier one instead of having its own), or a gated delta rule with one decay per head or one per key channel
(:class:`~llmserver_amd.parts.delta.GatedDeltaRule`).  Its feed-forward is a gated one with silu and biases
(:class:`~llmserver_amd.parts.mlp.GatedMLP`), routed experts without biases whose router has one
(:class:`~llmserver_amd.parts.experts.RoutedExperts`), or none.  The head is a matrix of its own behind the model's norm.
Tensor names: ``embed``, ``l<i>.<...>``, ``final.norm``, ``head``; every name is the tensor's whole name.
"""
from __future__ import annotations

from ..config.gogalix import DeltaSizes, DenseSizes, GogalixConfig
from ..config.registry import register_architecture
from ..parts import (DifferentialAttention, DifferentialNames, GatedDeltaNames, GatedDeltaRule, GatedMLP, GatedMLPNames, Linear,
                     ParallelGatedBlock, RMSNorm, RoutedExperts, TokenEmbedding)
from .decoder import DecoderModel, LayerCall

ATTENTION_NAMES = DifferentialNames()
DELTA_NAMES = GatedDeltaNames()
MLP_NAMES = GatedMLPNames(gate_up=("gate", "up"), down="down")
BLOCK_NAMES = ("norm1", "mix", "mlp", "ls1", "ls2", "rg1", "rg2")
MODEL_NAMES = ("embed", "l", "final.norm")
HEAD_NAME = "head"
BIAS_SUFFIX = ".b"
ACTIVATION = "silu"         # fixed by the design, as are the biases of the dense feed-forward, of the router and of the stream's gates


def _longest(windows):
    """How long shared pages are kept: as long as the longest window of those that read them (None: for ever)."""
    return None if any(window is None for window in windows) else max(windows)


def build_gogalix(config: GogalixConfig) -> DecoderModel:
    eps, width = config.norm_eps, config.width
    # the pages of a layer's keys and values: its own, or those of the layer it names; a page is kept for the
    # longest of the windows of all layers that read it
    source = [layer.mixer.kv_from if layer.type == "attention" and layer.mixer.kv_from is not None else index
              for index, layer in enumerate(config.layers)]
    readers = {}
    for index, layer in enumerate(config.layers):
        if layer.type == "attention":
            readers.setdefault(source[index], []).append(layer.mixer.window)
    blocks = []
    for index, layer in enumerate(config.layers):
        sizes = layer.mixer
        if isinstance(sizes, DeltaSizes):
            mixer = GatedDeltaRule(width, sizes.heads, sizes.kv_heads, sizes.dim, sizes.vdim, sizes.taps, eps,
                                   decay_per_channel=sizes.per_channel, low_rank_gate=sizes.per_channel, low=sizes.low,
                                   gate_low=sizes.gate_low, names=DELTA_NAMES)
        else:
            mixer = DifferentialAttention(width, sizes.heads, sizes.kv_heads, sizes.dim, sizes.vdim, sizes.scale, sizes.diff, eps,
                                          window=sizes.window, shares_cache=sizes.kv_from is not None,
                                          cache_window=_longest(readers[source[index]]), names=ATTENTION_NAMES)
        if layer.mlp is None:
            feed = None
        elif isinstance(layer.mlp, DenseSizes):
            feed = GatedMLP(width, layer.mlp.ff, ACTIVATION, bias=True, names=MLP_NAMES, bare_names=True, bias_suffix=BIAS_SUFFIX)
        else:
            feed = RoutedExperts(width, layer.mlp.ff, layer.mlp.experts, layer.mlp.top, router_bias="router" + BIAS_SUFFIX)
        blocks.append(ParallelGatedBlock(RMSNorm(width, eps, tensor="", single=True), mixer, feed, names=BLOCK_NAMES, bias_suffix=BIAS_SUFFIX))
    order = [LayerCall(index, source[index], source[index] == index) for index in range(len(blocks))]
    head = Linear(width, (HEAD_NAME,), (config.vocab,), out_float32=True, bare_names=True)
    embedding = TokenEmbedding(config.vocab, width, tensor="", wide=True, scale=config.embedding_scale)
    return DecoderModel(config, embedding, blocks, RMSNorm(width, eps, tensor="", single=True), head, tie_head=False, order=order,
                        names=MODEL_NAMES, layer_name=lambda i: f"l{i}")


register_architecture(GogalixConfig.MODEL_TYPE, GogalixConfig, build_gogalix, replace=True)
