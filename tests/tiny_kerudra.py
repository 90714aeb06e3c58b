"""The tests' own small Kerudra configurations; they differ in every size, constant and option: the order of the
layers, layers without a feed-forward, one, two, three streams and none, loops over several layers, over one layer and
none, windows on either kind of attention and on neither, rotations of a part of a head, of the whole head and of
nothing, one and several key/value heads, heads that are no multiple of anything, memories whose values are wider and
narrower than their keys and exactly one wavefront wide, scales of one and others."""
from __future__ import annotations

import functools
import tempfile

import plain_kerudra as plain
from llmserver_amd.config import config_from_dict
from llmserver_amd.weights import RandomInit, write_random_model


def attention(heads, kv_heads, dim, scale, rot=None, window=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if rot is not None:
        mixer["rot"] = {"dims": rot[0], "base": rot[1]}
    if window is not None:
        mixer["mask"] = {"size": window}
    return {"type": "attention", "mixer": mixer}


def latent(heads, dim, rot_dim, vdim, rank, scale, rot, window=None):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale, "rot": {"dims": rot[0], "base": rot[1]}}
    if window is not None:
        mixer["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": mixer}


def memory(heads, dim, vdim, cap):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def config(vocab, width, eps, layers, **top):
    return {"architecture": "Kerudra", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "layers": [{**mixer, "mlp": mlp} for mixer, mlp in layers], **top}


KA = config(97, 48, 1e-5, [
    (memory(2, 6, 10, 4.0), dense(40)),
    (latent(3, 8, 4, 6, 10, 0.3, (4, 100.0), window=7), dense(24)),
    (attention(4, 2, 12, 0.25, rot=(4, 50.0)), None),
    (memory(3, 10, 4, 9.0), dense(30))],
    streams=3, loop={"start": 1, "stop": 3, "times": 2}, residual_mult=0.6, logit_scale=1.5, embedding={"scale": 3.0})
KB = config(130, 64, 1e-6, [
    (attention(2, 2, 16, 0.2, rot=(16, 1e4), window=5), dense(70)),
    (latent(2, 12, 6, 20, 26, 0.22, (6, 1e6)), None),
    (memory(1, 40, 7, 1.0), dense(33)),
    (attention(3, 1, 32, 0.15), dense(20))])
KC = config(61, 40, 3e-4, [
    (latent(5, 6, 6, 3, 7, 0.4, (2, 77.0), window=1), dense(16)),
    (attention(5, 5, 10, 0.3, rot=(10, 300.0), window=20), dense(50)),
    (memory(4, 5, 12, 30.0), None)],
    streams=1, loop={"start": 1, "stop": 2, "times": 3}, residual_mult=1.25, logit_scale=0.7)
# Sizes in the kernels' own steps (heads of 32 and 64, cache rows of 48, pages of 16): the padded rows have nothing to pad,
# and a memory whose values fill a wavefront exactly, so that its normaliser is a workgroup of its own.
KD = config(200, 64, 1e-5, [
    (attention(4, 2, 32, 0.18, rot=(32, 2e4), window=40), dense(96)),
    (memory(2, 64, 64, 12.0), dense(64)),
    (latent(4, 32, 16, 32, 32, 0.14, (16, 5e4), window=33), dense(96))],
    streams=2, loop={"start": 0, "stop": 3, "times": 2}, residual_mult=0.5, embedding={"scale": 8.0}, logit_scale=2.5)
KE = config(50, 32, 1e-5, [(memory(2, 8, 8, 2.0), dense(24))], streams=4)

INIT = RandomInit(seed=3, std=0.15, norm_noise=0.3, bias_std=0.4)
CASES = {"KA": (KA, INIT, 16), "KB": (KB, RandomInit(seed=8, std=0.12, norm_noise=0.2, bias_std=0.5), 8),
         "KC": (KC, RandomInit(seed=21, std=0.2, norm_noise=0.25, bias_std=0.3), 4), "KD": (KD, RandomInit(seed=5, std=0.1, norm_noise=0.3, bias_std=0.3), 16),
         "KE": (KE, RandomInit(seed=2, std=0.25, norm_noise=0.3, bias_std=0.6), 8)}

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
