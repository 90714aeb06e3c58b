"""Gogalix on the GPU as a user runs it: ``bin/trace_run`` as a subprocess over the same requests whole, with a
decoded tail, in changing portions and mixed with others on a pool so small that pages and state slots are used
again; float32 against the plain implementation, bfloat16 against what the plain implementation loses when it rounds
where 16-bit kernels round; long decoding from the first token; sharpened weights (windows' edges, far keys, far
writes of the delta rule, convolution taps) on the kernels themselves; greedy generation through the entry point."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_gogalix as plain
import traces
from helpers import random_tokens, relative_error
from test_zepolix_gpu import check_rounding
from tiny_gogalix import CASES, model_folder, plain_logits, plain_model

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
pytestmark = pytest.mark.gpu
BF16 = plain.rounding_to(torch.bfloat16)


def rounded_logits(case, tokens):
    raw, tensors = plain_model(case)
    return plain.forward(raw, tensors, list(tokens), r=BF16).numpy()


def run_folder(folder, vocab, dtype, steps, out, max_tokens, page_size):
    command = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
               "--out", str(out), "--max-tokens", str(max_tokens), "--page-size", str(page_size)]
    done = subprocess.run(command, input=traces.to_lines(steps), capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-3000:]
    assert done.stdout.split() == [w for s in steps for w in ("done", str(s["step"]))]
    return traces.collect(steps, str(out), vocab)


def run_trace(case, dtype, steps, tmp_path, max_tokens, page_size):
    return run_folder(model_folder(case), CASES[case][0]["vocab"], dtype, steps, tmp_path / f"out-{case}-{dtype}", max_tokens, page_size)


def build_trace(case):
    vocab = CASES[case][0]["vocab"]
    requests, steps = {}, []

    def add(prefix, lengths, maker, seed0):
        mine = {f"{prefix}{i}": random_tokens(vocab, n, seed0 + i) for i, n in enumerate(lengths)}
        requests.update(mine)
        for step in maker(mine):
            step["step"] = len(steps)
            steps.append(step)

    base = (70, 33, 100, 1, 2)
    add("w", base, traces.whole, 100)
    add("t", base, lambda r: traces.tail_decoded(r, 32), 100)
    add("p", base, lambda r: traces.changing_portions(r, sizes=(2, 7, 1, 3, 33, 2, 2, 16, 5)), 100)
    add("m", (5, 17, 33, 70, 100, 41, 64, 1, 90, 130, 20, 77), lambda r: traces.mixed(r, seed=7, budget_tokens=256), 200)
    return steps, requests


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", sorted(CASES))
def test_all_schedules_match_the_plain_implementation(case, dtype, tmp_path):
    print(f"replay {case} {dtype}", flush=True)
    steps, requests = build_trace(case)
    results = run_trace(case, dtype, steps, tmp_path, traces.peak_tokens(steps), CASES[case][2])
    assert len(results) == sum(len(t) for t in requests.values())
    errors, lost = [], []
    for (rid, position), logits in results.items():
        expected = plain_logits(case, tuple(requests[rid]))[position].numpy()
        if dtype == "float32":
            np.testing.assert_allclose(logits, expected, atol=1.5e-4, rtol=3e-4, err_msg=f"{rid} position {position}")
        else:
            errors.append(relative_error(logits, expected))
    if errors:
        for rid, tokens in requests.items():
            exact = plain_logits(case, tuple(tokens)).numpy()
            lost += [relative_error(row, want) for row, want in zip(rounded_logits(case, tuple(tokens)), exact)]
        check_rounding(errors, lost, f"case {case} against the plain implementation")
    # the same request cut differently agrees with itself
    between = []
    for index in range(5):
        for position in range(len(requests[f"w{index}"])):
            for other in ("t", "p"):
                a, b = results[(f"w{index}", position)], results[(f"{other}{index}", position)]
                if dtype == "float32":
                    assert float(np.abs(a - b).max()) <= 1e-4 * max(1.0, float(np.abs(a).max())), (index, other, position)
                else:
                    between.append(relative_error(b, a))
    if between:
        check_rounding(between, lost, f"case {case} between two cuts of the same request", factor=2.0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_from_the_first_token(dtype, tmp_path):
    """A one-token prompt decoded for 600 tokens: the delta rules' states carry on for hundreds of steps of one token, the
    windows pass over decoded tokens and give their pages back, the replayed graphs of decoding steps see every context."""
    print(f"long decoding {dtype}", flush=True)
    case = "GC"
    tokens = random_tokens(CASES[case][0]["vocab"], 601, 31)
    steps = traces.tail_decoded({"long": tokens}, tail=600)
    results = run_trace(case, dtype, steps, tmp_path, 640, 16)
    expected = plain_logits(case, tuple(tokens)).numpy()
    errors = []
    for position in range(601):
        if dtype == "float32":
            np.testing.assert_allclose(results[("long", position)], expected[position], atol=1.5e-4, rtol=3e-4, err_msg=f"position {position}")
        else:
            errors.append(relative_error(results[("long", position)], expected[position]))
    if errors:
        lost = [relative_error(row, want) for row, want in zip(rounded_logits(case, tuple(tokens)), expected)]
        check_rounding(errors, lost, "long decoding")


def test_sharpened_weights_on_the_kernels(tmp_path):
    """What random weights could hide, in float32 on the kernels: delta rules that forget nothing over 300 tokens, a key
    hundreds back among hundreds in attention without a window, the edges of windows (also of layers that read another
    layer's pages) and convolution taps that weigh the oldest input most, each whole, with a decoded tail and in portions."""
    from test_gogalix_cpu import sharpened

    def far_write(layer):
        def change(tensors):
            tensors[f"l{layer}.mix.A_log"][:] = -9.0
        return change

    def far_key(tensors):
        tensors["l2.mix.q"] *= 6.0
        tensors["l2.mix.k"] *= 6.0

    def edge(layer, source):
        def change(tensors):
            tensors[f"l{layer}.mix.q"] *= 5.0
            tensors[f"l{source}.mix.k"] *= 3.0
        return change

    def taps(tensors):
        for layer, count in ((1, 4), (5, 5)):
            for name in ("q", "k", "v"):
                weight = tensors[f"l{layer}.mix.{name}.conv"]
                weight *= torch.linspace(3.0, 0.3, count, dtype=weight.dtype)

    for number, (case, change, length, page) in enumerate((("GC", far_write(1), 300, 16), ("GC", far_write(2), 300, 16), ("GB", far_key, 260, 8),
                                                           ("GA", edge(0, 0), 90, 16), ("GA", edge(3, 0), 90, 4), ("GB", edge(4, 2), 90, 8),
                                                           ("GC", edge(4, 4), 90, 16), ("GC", edge(3, 0), 90, 16), ("GC", taps, 60, 16))):
        print(f"sharpened {number} {case}", flush=True)
        folder, raw, tensors = sharpened(case, change)
        tokens = random_tokens(raw["vocab"], length, 40 + number)
        expected = plain.forward(raw, tensors, tokens).numpy()
        requests = {"a": tokens}
        for name, steps in (("whole", traces.whole(requests)), ("tail", traces.tail_decoded(requests, 40)),
                            ("portions", traces.changing_portions(requests, sizes=(2, 7, 1, 3, 33, 2, 2, 16, 5)))):
            results = run_folder(folder, raw["vocab"], "float32", steps, tmp_path / f"{number}-{name}", 64 * -(-length // 64), page)
            for position in range(length):
                np.testing.assert_allclose(results[("a", position)], expected[position], atol=2e-4, rtol=5e-4, err_msg=f"{number} {name} {position}")


def test_greedy_generation_through_the_entry_point():
    from llmserver_amd.entrypoints import generate
    print("generation", flush=True)
    raw, tensors = plain_model("GA")
    prompts = [random_tokens(97, n, 700 + n) for n in (19, 3, 41, 8, 1, 27)]
    expected = [plain.greedy_generate(raw, tensors, prompt, 7) for prompt in prompts]
    got = generate(model_folder("GA"), prompts, max_new_tokens=7, dtype="float32", device="cuda", block_size=8, num_blocks=26,
                   max_batch_size=3, max_num_batched_tokens=24, prefill_chunk_size=16)
    assert got == expected
    rounded = generate(model_folder("GA"), prompts, max_new_tokens=7, dtype="bfloat16", device="cuda", block_size=8)
    same = sum(a == b for g, e in zip(rounded, expected) for a, b in zip(g, e))
    assert same >= 0.6 * sum(len(e) for e in expected), (rounded, expected)


def test_the_benchmark_command_line_and_the_design_option_of_bench(tmp_path, capsys):
    """The framework's command line serves a Gogalix folder like any other (matrix of prompt lengths and batch sizes, one
    prompt's tokens equal to the oracle's; the mixed workload); ``bench.py --design gogalix`` prints one JSON line with
    every named size beside its neighbours (three layers each here)."""
    from llmserver_amd.cli import benchmark
    print("command lines", flush=True)
    folder, raw = model_folder("GC"), CASES["GC"][0]
    report = tmp_path / "report.json"
    assert benchmark.main(["--model", folder, "--dtype", "float32", "--prompt-tokens", "9,40", "--batch-sizes", "1,3", "--output-tokens", "6",
                           "--repeats", "1", "--block-size", "16", "--json", str(report)]) == 0
    results = json.loads(report.read_text())["results"]
    assert [(r["prompt_tokens"], r["batch"]) for r in results] == [(9, 1), (9, 3), (40, 1), (40, 3)]
    config, tensors = plain_model("GC")
    prompt = benchmark.matrix_prompts(raw["vocab"], 9, 1, "whole-run", 0, 0)[0]
    assert results[0]["tokens"][0] == plain.greedy_generate(config, tensors, prompt, 6)
    capsys.readouterr()
    assert benchmark.main(["--model", folder, "--mixed-requests", "6", "--mixed-prompt-range", "4,40", "--shared-prefix-tokens", "16",
                           "--output-tokens", "5", "--block-size", "8", "--max-num-batched-tokens", "64"]) == 0
    assert "mixed: 6 requests" in capsys.readouterr().out
    done = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--design", "gogalix", "--layers", "3", "--steps", "4", "--warmup", "1",
                           "--prefill-tokens", "256"], capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-3000:]
    record = json.loads([line for line in done.stdout.splitlines() if line.strip()][-1])
    assert set(record["sizes"]) == {"gogalix-2k", "barotar-2k", "dense-2k", "gogalix-4k", "barotar-4k", "dense-4k"} and record["value"] > 0
    assert all(entry["layers"] == 3 and entry["decode_b8_tok_s"] > 0 and entry["prefill_256_ms"] > 0 for entry in record["sizes"].values())
