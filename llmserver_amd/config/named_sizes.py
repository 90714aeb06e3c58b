"""Model sizes that the command lines know by name, for runs with random weights: each entry is a ``config.json`` in
small, ``model_type`` included, so whoever asks for a name gets a configuration of whatever architecture the entry
names.  The sizes are those of published checkpoints (their ``config.json`` files) and of the tests' tiny models."""
from __future__ import annotations

from typing import Optional

from .base import ModelConfig
from .registry import config_from_dict

NAMED_SIZES = {
    "tiny-a": dict(model_type="qwen3", num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
                   intermediate_size=128, vocab_size=256, rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=True),
    "tiny-b": dict(model_type="qwen3", num_hidden_layers=3, hidden_size=96, num_attention_heads=8, num_key_value_heads=2, head_dim=32,
                   intermediate_size=224, vocab_size=384, rope_theta=1e6, rms_norm_eps=1e-5, attention_bias=True),
    "qwen3-0.6b": dict(model_type="qwen3", num_hidden_layers=28, hidden_size=1024, num_attention_heads=16, num_key_value_heads=8,
                       head_dim=128, intermediate_size=3072, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
                       tie_word_embeddings=True),
    "qwen3-1.7b": dict(model_type="qwen3", num_hidden_layers=28, hidden_size=2048, num_attention_heads=16, num_key_value_heads=8,
                       head_dim=128, intermediate_size=6144, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
                       tie_word_embeddings=True),
    "qwen3-4b": dict(model_type="qwen3", num_hidden_layers=36, hidden_size=2560, num_attention_heads=32, num_key_value_heads=8,
                     head_dim=128, intermediate_size=9728, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
                     tie_word_embeddings=True),
    "qwen3-8b": dict(model_type="qwen3", num_hidden_layers=36, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8,
                     head_dim=128, intermediate_size=12288, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6),
    "qwen3-14b": dict(model_type="qwen3", num_hidden_layers=40, hidden_size=5120, num_attention_heads=40, num_key_value_heads=8,
                      head_dim=128, intermediate_size=17408, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6),
    "qwen3-32b": dict(model_type="qwen3", num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, num_key_value_heads=8,
                      head_dim=128, intermediate_size=25600, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6),
}




def _zepolix(width, layers, heads, dim, rot_dim, vdim, kv_rank, ff, experts, top, vocab=32768, taps=4):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": (dim + rot_dim) ** -0.5,
             "rot": {"base": 10000.0, "dims": rot_dim}}
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    return {"architecture": "Zepolix", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "canon": {"taps": taps},
            "layers": [{"type": "latent_attention", "mixer": dict(mixer), "mlp": dict(mlp)} for _ in range(layers)]}


# Zepolix at sizes that resemble a published mixture-of-experts model's layers (16 heads of 128 + 64 query dimensions and a
# value size of 128 over a width of 2,048, 64 experts of 1,408 of which a token uses 6; the latent is 192 wide, so that a
# cache row fills the widest head the attention kernels take), and one twice as wide; and, for each, the dense decoder of
# this package with the same width, depth, heads and head size whose feed-forward is as large as the experts a token uses.
NAMED_SIZES.update({
    "zepolix-2k": _zepolix(2048, 8, 16, 128, 64, 128, 192, 1408, 64, 6),
    "zepolix-4k": _zepolix(4096, 8, 32, 128, 64, 128, 192, 2048, 32, 4),
    "dense-2k": dict(model_type="qwen3", num_hidden_layers=8, hidden_size=2048, num_attention_heads=16, num_key_value_heads=8,
                     head_dim=128, intermediate_size=6 * 1408, vocab_size=32768, rope_theta=10000.0, rms_norm_eps=1e-6),
    "dense-4k": dict(model_type="qwen3", num_hidden_layers=8, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8,
                     head_dim=128, intermediate_size=4 * 2048, vocab_size=32768, rope_theta=10000.0, rms_norm_eps=1e-6),
})


def _barotar(width, layers, heads, kv_heads, dim, window, recurrent_heads, gla_heads, gla_dim, gla_vdim, ff, expert_ff, experts, top, groups, keep,
             vocab=32768):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "mask": {"size": window}, "rot": {"base": 10000.0, "dims": dim // 2},
            "scale": dim ** -0.5, "softcap": 50.0}
    parallel = {"left": left, "right": {"heads": recurrent_heads, "dim": width // recurrent_heads, "low": 64}, "left_scale": 1.0, "right_scale": 1.0}
    gla = {"heads": gla_heads, "dim": gla_dim, "vdim": gla_vdim, "tau": 16.0, "low": 16}
    dense = {"kind": "dense", "ff": ff}
    moe = {"kind": "moe", "expert": {"ff": expert_ff, "limit": 7.0}, "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}
    four = [("parallel", parallel, dense), ("gla", gla, moe), ("parallel", parallel, dense), ("parallel", parallel, moe)]
    return {"architecture": "Barotar", "vocab": vocab, "width": width, "norm": {"eps": 1e-6},
            "layers": [{"type": kind, "mixer": dict(mixer), "mlp": dict(mlp)} for kind, mixer, mlp in (four * (-(-layers // 4)))[:layers]]}


# Barotar at the widths of the sizes above: windowed attention of 16 (32) heads of 128 over 8 key/value heads and a window
# of 1,024 keys beside a time mixing of as many heads of 128; a gated linear recurrence of 8 (16) heads with keys of 128 and
# values of 256; dense feed-forwards as large as the dense decoders' beside them, and experts of the Zepolix sizes' shape
# in groups of eight.  Three layers in four mix side by side, one in four is the linear recurrence; half the layers route.
NAMED_SIZES.update({
    "barotar-2k": _barotar(2048, 8, 16, 8, 128, 1024, 16, 8, 128, 256, 6 * 1408, 1408, 64, 6, 8, 4),
    "barotar-4k": _barotar(4096, 8, 32, 8, 128, 1024, 32, 16, 128, 256, 4 * 2048, 2048, 32, 4, 4, 2),
})


def _kerudra(width, layers, heads, kv_heads, dim, window, rot_dim, kv_rank, memory_heads, memory_dim, memory_vdim, ff, streams=2, vocab=32768):
    memory = ("mlstm", {"heads": memory_heads, "dim": memory_dim, "vdim": memory_vdim, "gate_cap": 15.0})
    latent = ("latent_attention", {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": dim, "kv_rank": kv_rank, "scale": (dim + rot_dim) ** -0.5,
                                   "rot": {"base": 10000.0, "dims": rot_dim}, "mask": {"size": window}})
    attention = ("attention", {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5, "rot": {"base": 10000.0, "dims": dim}})
    four = [memory, latent, attention, memory]
    return {"architecture": "Kerudra", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "streams": streams, "residual_mult": 0.5,
            "embedding": {"scale": 1.0}, "logit_scale": 1.0,
            "layers": [{"type": kind, "mixer": dict(mixer), "mlp": {"kind": "dense", "ff": ff}} for kind, mixer in (four * (-(-layers // 4)))[:layers]]}


# Kerudra at the widths of the sizes above, two residual streams: of every four layers two are matrix memories of 8 (16)
# heads with keys of 128 and values of 256 (a state of 1 MB a layer and request), one is latent attention of the Zepolix
# sizes' shape under a window of 1,024 keys and a gate per channel, one is attention of 16 (32) heads of 128 over 8 key/value
# heads whose values are its keys; plain feed-forwards as wide as the dense decoders' gated ones beside them.
NAMED_SIZES.update({
    "kerudra-2k": _kerudra(2048, 8, 16, 8, 128, 1024, 64, 192, 8, 128, 256, 6 * 1408),
    "kerudra-4k": _kerudra(4096, 8, 32, 8, 128, 1024, 64, 192, 16, 128, 256, 4 * 2048),
})


def _gogalix(width, layers, heads, kv_heads, dim, vdim, window, delta_heads, delta_kv_heads, delta_dim, delta_vdim, ff, expert_ff, experts, top,
             vocab=32768):
    attention = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "diff": 0.6, "mask": {"size": window}}
    delta = {"heads": delta_heads, "kv_heads": delta_kv_heads, "dim": delta_dim, "vdim": delta_vdim, "conv": 4}
    dense = {"kind": "dense", "ff": ff}
    moe = {"kind": "moe", "expert": {"ff": expert_ff}, "router": {"experts": experts, "top": top}}
    made = []
    for index in range(layers):
        kind = index % 4
        if kind == 0:
            made.append({"type": "attention", "mixer": dict(attention), "mlp": dict(dense)})
        elif kind == 1:
            made.append({"type": "delta", "mixer": dict(delta), "mlp": dict(moe)})
        elif kind == 2:
            made.append({"type": "channel_delta", "mixer": {**delta, "low": 64, "gate_low": 64}, "mlp": dict(dense)})
        else:
            made.append({"type": "attention", "mixer": {**attention, "kv_from": index - 3}, "mlp": dict(moe)})
    return {"architecture": "Gogalix", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0}, "layers": made}


# Gogalix at the widths of the sizes above: of every four layers one is differential attention of 16 (32) heads with two maps
# of 64 and values of 128 over 8 key/value heads under a window of 1,024 keys, one reads that layer's pages with queries of
# its own, and two are gated delta rules of 16 (32) heads with keys and values of 128 over 8 (16) key heads (a state of 1 MB
# (2 MB) a layer and request), one with a decay per head and one with a decay per key channel; dense feed-forwards as large
# as the dense decoders' beside them in two layers of four, experts of the Zepolix sizes' shape in the other two.
NAMED_SIZES.update({
    "gogalix-2k": _gogalix(2048, 8, 16, 8, 64, 128, 1024, 16, 8, 128, 128, 6 * 1408, 1408, 64, 6),
    "gogalix-4k": _gogalix(4096, 8, 32, 8, 64, 128, 1024, 32, 16, 128, 128, 4 * 2048, 2048, 32, 4),
})


def named_size(name: str) -> dict:
    """The entry's keys, a copy the caller may change (fewer layers, say)."""
    try:
        return dict(NAMED_SIZES[name])
    except KeyError:
        raise KeyError(f"no size is named {name!r}; known: {', '.join(sorted(NAMED_SIZES))}") from None


def named_config(name: str, layers: Optional[int] = None) -> ModelConfig:
    """The typed configuration of a named size, with at most ``layers`` layers if given (shapes do not depend on depth)."""
    return config_from_dict(with_layers(named_size(name), layers))


def with_layers(raw: dict, layers: Optional[int]) -> dict:
    """The same configuration with at most ``layers`` layers (0 or None: all), however the architecture counts them."""
    raw = dict(raw)
    if layers:
        if isinstance(raw.get("layers"), list):
            raw["layers"] = raw["layers"][:int(layers)]
        else:
            raw["num_hidden_layers"] = min(int(raw["num_hidden_layers"]), int(layers))
    return raw
