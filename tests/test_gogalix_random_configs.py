"""Seeded random Gogalix configurations: any order of the three mixers, with a dense or a routed feed-forward or none;
any number of heads and key heads; key, value and state sizes that are multiples of nothing, up to sizes of real
models' heads; windows from one key to more than any request, or none; layers that read an earlier layer's keys and
values through a window of their own; one to five convolution taps; routers that choose one, some or all experts;
widths and vocabularies that are no multiple of four.  Every configuration goes through a mixed trace (pages and state
slots used again): on the CPU with the kernels' twins, on the GPU through ``bin/trace_run`` in both types."""
import io
import os
import random
import subprocess
import sys
import tempfile

import numpy as np
import pytest
import torch

import plain_gogalix as plain
import traces
from helpers import random_tokens, relative_error
from llmserver_amd.config import config_from_dict
from llmserver_amd.engine.replay import make_runner, replay
from llmserver_amd.weights import RandomInit, write_random_model
from tiny_gogalix import attention, channel_delta, config, delta, dense, moe
from torch_ops import TorchOps

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SEEDS = list(range(10))
FLOAT32_ERROR = 3e-5
_MADE = {}


def random_config(seed):
    rng = random.Random(7000 + seed)
    big = seed % 2 == 1                      # every other seed has heads of the sizes real models use
    layers, owners = [], []
    count = rng.randint(1, 5)
    for index in range(count):
        kind = rng.choice(("attention", "attention", "delta", "channel_delta"))
        window = rng.choice([None, None, 1, 2, 5, 16, 33, 64, 100, 1000])
        if kind == "attention":
            if owners and rng.random() < 0.5:           # read an earlier layer's keys and values, through a window of its own
                source = rng.choice(owners)
                sizes = layers[source][0]["mixer"]
                mixer = attention(sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"], rng.uniform(0.05, 0.5), rng.uniform(0.1, 0.9),
                                  window=window, kv_from=source)
            else:
                kv_heads = rng.randint(1, 3)
                dim = rng.choice([32, 64, 48]) if big else rng.randint(1, 24)
                vdim = rng.choice([64, 128, 96]) if big else rng.randint(1, 40)
                mixer = attention(kv_heads * rng.randint(1, 4), kv_heads, dim, vdim, rng.uniform(0.05, 0.5), rng.uniform(0.1, 0.9), window=window)
                owners.append(index)
        else:
            kv_heads = rng.randint(1, 3)
            dim = rng.choice([64, 128, 130, 256]) if big else rng.randint(1, 40)
            vdim = rng.choice([64, 128, 63, 65]) if big else rng.randint(1, 70)
            make = delta if kind == "delta" else lambda *sizes: channel_delta(*sizes, rng.randint(1, 20), rng.randint(1, 20))
            mixer = make(kv_heads * rng.randint(1, 3), kv_heads, dim, vdim, rng.randint(1, 5))
        feed = rng.random()
        if feed < 0.2:
            mlp = None
        elif feed < 0.6:
            mlp = dense(rng.randint(3, 90))
        else:
            experts = rng.randint(1, 12)
            mlp = moe(rng.choice([32, 64]) if big else rng.randint(2, 40), experts, rng.randint(1, experts))
        layers.append((mixer, mlp))
    width = rng.choice([64, 128, 256]) if big else rng.choice([24, 40, 50, 64, 72, 100, 134])
    top = {}
    if rng.random() < 0.7:
        top["embedding"] = {"scale": rng.uniform(0.5, 12.0)}
    raw = config(rng.randint(30, 400), width, 10.0 ** rng.uniform(-6, -3), layers, **top)
    return raw, RandomInit(seed=seed, std=rng.uniform(0.08, 0.2), norm_noise=0.25, bias_std=0.4), rng.choice([4, 8, 16, 32])


def made(seed):
    """(config.json, folder, page size, requests, steps, exact logits per request, tensors) of a seed, made once."""
    if seed not in _MADE:
        raw, init, page = random_config(seed)
        folder = tempfile.mkdtemp(prefix=f"llmserver_amd_test_gr{seed}_")
        write_random_model(config_from_dict(dict(raw)), folder, init)
        lengths = (1, 37, 90, 5, 64, 2, 130, 18)
        requests = {f"q{i}": random_tokens(raw["vocab"], n, 50 * seed + i) for i, n in enumerate(lengths)}
        steps = traces.mixed(requests, seed=seed, budget_tokens=256)
        tensors = plain.read_folder(folder)[1]
        exact = {rid: plain.forward(raw, tensors, tokens).numpy() for rid, tokens in requests.items()}
        _MADE[seed] = (raw, folder, page, requests, steps, exact, tensors)
    return _MADE[seed]


_BOUNDS = {}


def float32_bound(seed, rid, position):
    """What a position's logits may differ by in float32, in units of their largest magnitude: three times what the plain
    implementation itself loses when it computes in float32 (the 99th percentile over the seed's positions), and never
    less than FLOAT32_ERROR; a badly conditioned position (a read-out or a norm over terms that nearly cancel) is allowed
    ten times the plain implementation's own loss there: still far below what a wrong key, window or state does."""
    if seed not in _BOUNDS:
        raw, folder, _, requests, _, exact, _ = made(seed)
        single = plain.read_folder(folder, dtype=torch.float32)[1]
        lost = {(r, p): relative_error(row, want) for r, tokens in requests.items()
                for p, (row, want) in enumerate(zip(plain.forward(raw, single, tokens).numpy(), exact[r]))}
        _BOUNDS[seed] = (max(FLOAT32_ERROR, 3.0 * float(np.quantile(list(lost.values()), 0.99))), lost)
    everywhere, lost = _BOUNDS[seed]
    return max(everywhere, 10.0 * lost[(rid, position)])


def test_the_seeds_cover_every_mixer_and_option():
    raws = [random_config(seed)[0] for seed in SEEDS]
    layers = [layer for raw in raws for layer in raw["layers"]]
    assert {layer["type"] for layer in layers} == {"attention", "delta", "channel_delta"}
    assert any(layer["mlp"] is None for layer in layers) and {layer["mlp"]["kind"] for layer in layers if layer["mlp"]} == {"dense", "moe"}
    assert any(layer["mixer"].get("kv_from") is not None for layer in layers)
    assert any(layer["mixer"].get("mask") for layer in layers) and any(layer["type"] == "attention" and not layer["mixer"].get("mask") for layer in layers)
    assert any(layer["mixer"]["heads"] > layer["mixer"]["kv_heads"] for layer in layers if layer["type"] != "attention")
    assert any(layer["mixer"]["heads"] > layer["mixer"]["kv_heads"] for layer in layers if layer["type"] == "attention")


@pytest.mark.parametrize("seed", SEEDS)
def test_random_configurations_with_the_twins(seed, tmp_path):
    raw, folder, page, requests, steps, exact, _ = made(seed)
    runner = make_runner(folder, "float32", traces.peak_tokens(steps), page, device="cpu", ops=TorchOps())
    replay(runner, traces.to_lines(steps).splitlines(), str(tmp_path), io.StringIO())
    runner.cache.check_invariants()
    results = traces.collect(steps, str(tmp_path), raw["vocab"])
    assert len(results) == sum(len(t) for t in requests.values())
    for (rid, position), logits in results.items():
        assert relative_error(logits, exact[rid][position]) <= float32_bound(seed, rid, position), f"seed {seed} {rid} {position}: {raw}"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", SEEDS)
def test_random_configurations_on_the_gpu(seed, dtype, tmp_path):
    raw, folder, page, requests, steps, exact, tensors = made(seed)
    print(f"random configuration {seed} {dtype}: {raw}", flush=True)
    out = tmp_path / "out"
    command = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out),
               "--max-tokens", str(traces.peak_tokens(steps)), "--page-size", str(page)]
    done = subprocess.run(command, input=traces.to_lines(steps), capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-3000:]
    results = traces.collect(steps, str(out), raw["vocab"])
    assert len(results) == sum(len(t) for t in requests.values())
    errors = []
    for (rid, position), logits in results.items():
        if dtype == "float32":
            assert relative_error(logits, exact[rid][position]) <= float32_bound(seed, rid, position), f"seed {seed} {rid} {position}: {raw}"
        else:
            errors.append(relative_error(logits, exact[rid][position]))
    if errors:
        # what the plain implementation loses on the same sequences when it rounds where 16-bit kernels round
        rounding = plain.rounding_to(torch.bfloat16)
        lost = [relative_error(row, want) for rid, tokens in requests.items()
                for row, want in zip(plain.forward(raw, tensors, tokens, r=rounding).numpy(), exact[rid])]
        assert np.isfinite(errors).all()
        print(f"  median {np.median(errors):.2e} / {np.median(lost):.2e}, 90th {np.quantile(errors, 0.9):.2e} / {np.quantile(lost, 0.9):.2e}", flush=True)
        assert np.median(errors) <= 1.3 * np.median(lost), (seed, np.median(errors), np.median(lost))
        assert np.quantile(errors, 0.9) <= 3.0 * np.quantile(lost, 0.9), (seed, np.quantile(errors, 0.9), np.quantile(lost, 0.9))
