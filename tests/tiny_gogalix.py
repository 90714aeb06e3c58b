"""The tests' own small Gogalix configurations; they differ in every size, constant and option: the order of the
layers, layers without a feed-forward, dense and routed feed-forwards (a token using some experts, one, or all of them),
attention with grouped and ungrouped heads, values wider and narrower than keys, windows of a few keys, of one key and
none, layers that read another layer's keys and values through a shorter and a longer window of their own, delta rules
with one and several key heads, one to five convolution taps, key channels from a handful to more than a wavefront,
values that fill a workgroup's columns exactly and that do not, low-rank maps of several inner sizes."""
from __future__ import annotations

import functools
import tempfile

import plain_gogalix as plain
from llmserver_amd.config import config_from_dict
from llmserver_amd.weights import RandomInit, write_random_model


def attention(heads, kv_heads, dim, vdim, scale, diff, window=None, kv_from=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff}
    if window is not None:
        mixer["mask"] = {"size": window}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "attention", "mixer": mixer}


def delta(heads, kv_heads, dim, vdim, taps):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": taps}}


def channel_delta(heads, kv_heads, dim, vdim, taps, low, gate_low):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": taps, "low": low,
                                               "gate_low": gate_low}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def config(vocab, width, eps, layers, **top):
    return {"architecture": "Gogalix", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "layers": [{**mixer, "mlp": mlp} for mixer, mlp in layers], **top}


GA = config(97, 48, 1e-5, [
    (attention(4, 2, 6, 10, 0.3, 0.6, window=7), dense(40)),
    (delta(4, 2, 8, 6, 3), moe(16, 6, 2)),
    (channel_delta(2, 1, 12, 5, 4, 5, 7), None),
    (attention(4, 2, 6, 10, 0.45, 0.3, window=11, kv_from=0), moe(8, 3, 3)),
    (delta(3, 3, 5, 9, 2), dense(24))],
    embedding={"scale": 3.0})
GB = config(130, 64, 1e-6, [
    (delta(1, 1, 40, 7, 2), dense(70)),
    (attention(2, 2, 16, 16, 0.2, 0.8, window=5), moe(20, 4, 1)),
    (attention(3, 1, 32, 20, 0.15, 0.5), None),
    (channel_delta(3, 3, 10, 4, 1, 3, 2), dense(33)),
    (attention(3, 1, 32, 20, 0.1, 0.2, window=9, kv_from=2), dense(20))])
# Sizes in the kernels' own steps (heads of 32 and 64, pages of 16, sixteen value columns to a workgroup), a window of one
# key, a layer that reads a cache through a shorter window than its owner, more key channels than a wavefront has lanes
GC = config(200, 64, 1e-5, [
    (attention(4, 2, 32, 64, 0.18, 0.6, window=40), dense(96)),
    (delta(2, 2, 64, 64, 4), moe(32, 8, 2)),
    (channel_delta(4, 2, 32, 32, 3, 8, 8), dense(64)),
    (attention(4, 2, 32, 64, 0.2, 0.4, window=33, kv_from=0), moe(32, 8, 3)),
    (attention(2, 2, 16, 48, 0.3, 0.7, window=1), None),
    (delta(1, 1, 80, 16, 5), None)],
    embedding={"scale": 8.0})
GD = config(50, 32, 3e-4, [(channel_delta(2, 2, 8, 8, 2, 4, 4), moe(12, 5, 5))], embedding={"scale": 0.5})
GE = config(61, 40, 1e-5, [(delta(2, 1, 16, 20, 3), dense(16)), (attention(2, 1, 8, 8, 0.35, 0.6, window=3), dense(16))])

CASES = {"GA": (GA, RandomInit(seed=3, std=0.15, norm_noise=0.3, bias_std=0.4), 16),
         "GB": (GB, RandomInit(seed=8, std=0.12, norm_noise=0.2, bias_std=0.5), 8),
         "GC": (GC, RandomInit(seed=5, std=0.1, norm_noise=0.3, bias_std=0.3), 16),
         "GD": (GD, RandomInit(seed=2, std=0.25, norm_noise=0.3, bias_std=0.6), 8),
         "GE": (GE, RandomInit(seed=21, std=0.2, norm_noise=0.25, bias_std=0.3), 4)}

_FOLDERS = {}


def model_folder(case: str) -> str:
    if case not in _FOLDERS:
        raw, init, _ = CASES[case]
        folder = tempfile.mkdtemp(prefix=f"llmserver_amd_test_{case}_")
        write_random_model(config_from_dict(dict(raw)), folder, init)
        _FOLDERS[case] = folder
    return _FOLDERS[case]


@functools.lru_cache(maxsize=None)
def plain_model(case: str):
    return plain.read_folder(model_folder(case))


@functools.lru_cache(maxsize=None)
def plain_logits(case: str, tokens: tuple):
    raw, tensors = plain_model(case)
    return plain.forward(raw, tensors, list(tokens))
