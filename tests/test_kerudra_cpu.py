"""Kerudra through the engine's own step function, cache manager, scheduler and entry point on the CPU (torch twins
of the kernels) against the plain implementation: configuration and weights, each mechanism, every way of cutting
and batching, pages and state slots used again, windows' edges, far keys, looped layers, and greedy generation."""
import io
import json
import os
import tempfile

import numpy as np
import pytest
import torch

import plain_kerudra as plain
import traces
from helpers import random_tokens
from llmserver_amd.config import ConfigError, UnsupportedModelError, config_from_dict
from llmserver_amd.engine.batch import StepEntry
from llmserver_amd.engine.replay import make_runner, replay
from llmserver_amd.parts import PagedKVSpec, StateSpec
from llmserver_amd.weights import build_model
from tiny_kerudra import CASES, KA, KB, KC, KD, model_folder, plain_logits, plain_model
from torch_ops import ChunkedMemoryOps, TorchOps


def runner_for(case, max_tokens, page=None, live=4):
    return make_runner(model_folder(case), "float32", max_tokens, page or CASES[case][2], device="cpu", ops=TorchOps(), max_live=live)


def run(case, steps, tmp_path, page=None):
    runner = runner_for(case, traces.peak_tokens(steps), page)
    replay(runner, traces.to_lines(steps).splitlines(), str(tmp_path), io.StringIO())
    runner.cache.check_invariants()
    assert not runner.cache.requests and runner.cache.state_slots_free() in (None, 4)
    assert all(free == group.pool.num_pages for free, group in zip(runner.cache.available_pages(), runner.cache.groups))
    return traces.collect(steps, str(tmp_path), CASES[case][0]["vocab"])


def check(case, results, requests, atol=1.5e-4):          # (float32 twins against float64)
    for (rid, position), logits in results.items():
        expected = plain_logits(case, tuple(requests[rid]))[position].numpy()
        np.testing.assert_allclose(logits, expected, atol=atol, rtol=3e-4, err_msg=f"{case} {rid} position {position}")
    assert len(results) == sum(len(tokens) for tokens in requests.values())


def requests_of(case, lengths, seed0=300):
    return {f"q{i}": random_tokens(CASES[case][0]["vocab"], n, seed0 + i) for i, n in enumerate(lengths)}


def copy_of(raw):
    return json.loads(json.dumps(raw))


# -- configuration and weights ---------------------------------------------------------------------------------------
def test_the_configuration_reads_back_and_refuses_what_is_not_built():
    config = config_from_dict(dict(KA))
    assert config_from_dict(config.to_dict()) == config
    assert config.layers[2].mlp is None and config.layers[0].mixer.gate_cap == 4.0 and config.layers[1].mixer.window == 7
    assert config.layers[2].mixer.window is None and config.layers[2].mixer.rot_dims == 4 and config.streams == 3
    assert config.layer_runs() == (0, 1, 2, 1, 2, 3) and config.norm_eps == 1e-5 and config.embedding_scale == 3.0
    plain_one = config_from_dict(dict(KB))
    assert plain_one.streams == 0 and plain_one.loop is None and plain_one.layer_runs() == (0, 1, 2, 3) and plain_one.logit_scale == 1.0
    assert plain_one.layers[3].mixer.rot_dims == 0 and plain_one.layers[3].mixer.kv_heads == 1
    assert config_from_dict(dict(KC)).layer_runs() == (0, 1, 1, 1, 2)
    other = copy_of(KA)
    other["layers"][1]["type"] = "something else"
    with pytest.raises(UnsupportedModelError, match="something else"):
        config_from_dict(other)
    other = copy_of(KA)
    other["layers"][1]["mlp"]["kind"] = "other"
    with pytest.raises(UnsupportedModelError, match="other"):
        config_from_dict(other)
    other = copy_of(KA)
    del other["layers"][0]["mixer"]["gate_cap"]
    with pytest.raises(ConfigError, match="gate_cap"):
        config_from_dict(other)
    other = copy_of(KA)
    other["layers"][2]["mixer"]["rot"]["dims"] = 5
    with pytest.raises(ConfigError, match="even"):
        config_from_dict(other)
    other = copy_of(KA)
    other["layers"][2]["mixer"]["kv_heads"] = 3             # four query heads over three key/value heads
    with pytest.raises(ConfigError, match="multiple"):
        config_from_dict(other)
    other = copy_of(KA)
    other["loop"]["stop"] = 9
    with pytest.raises(ConfigError, match="loop"):
        config_from_dict(other)
    other = copy_of(KA)
    other["streams"] = 9
    with pytest.raises(UnsupportedModelError, match="streams"):
        config_from_dict(other)


def test_the_model_declares_the_checkpoints_tensors_and_its_caches():
    model = build_model(config_from_dict(dict(KA)))
    specs = model.param_specs()
    assert {"embed", "final.norm", "l0.norm1", "l0.norm2", "l0.mix.q", "l0.mix.i", "l0.mix.i.b", "l0.mix.f.b", "l0.mix.norm", "l0.mix.g", "l0.hc1.in",
            "l0.hc2.mix", "l1.mix.dkv", "l1.mix.dkv.norm", "l1.mix.uk", "l1.mix.uv", "l1.mix.g", "l2.mix.q.b", "l2.mix.k.b", "l2.mix.o", "l2.hc1.out",
            "l3.mlp.up", "l3.mlp.down"} <= set(specs)
    assert not {"l2.mix.v", "l2.norm2", "l2.mlp.up", "l2.hc2.in", "l1.mix.q.b", "l2.mix.o.b", "l0.mix.o.b", "l4.norm1"} & set(specs)
    assert specs["l0.mix.q"].shape == (12, 48) and specs["l0.mix.v"].shape == (20, 48) and specs["l0.mix.o"].shape == (48, 20)
    assert specs["l0.mix.i"].shape == (2, 48) and specs["l0.mix.norm"].shape == (20,) and specs["l0.hc1.mix"].shape == (3, 3)
    assert specs["l1.mix.q"].shape == (36, 48) and specs["l1.mix.dkv"].shape == (14, 48) and specs["l1.mix.uk"].shape == (24, 10)
    assert specs["l1.mix.uv"].shape == (18, 10) and specs["l1.mix.g"].shape == (18, 48) and specs["l1.mix.o"].shape == (48, 18)
    assert specs["l2.mix.q"].shape == (48, 48) and specs["l2.mix.k"].shape == (24, 48) and specs["l2.mix.o"].shape == (48, 48)
    caches = model.cache_specs()
    assert len(caches) == 6                                  # a cache or state for every run of a layer, looped ones twice
    assert caches[0] == StateSpec((2 * 6 * 10 + 2 * 6 + 2,), "float32") and caches[5] == StateSpec((3 * 10 * 4 + 3 * 10 + 3,), "float32")
    for run in (1, 3):
        assert isinstance(caches[run], PagedKVSpec) and caches[run].window == 7 and caches[run].n_kv_heads == 1
    for run in (2, 4):
        assert isinstance(caches[run], PagedKVSpec) and caches[run].window is None and caches[run].n_kv_heads == 2
    assert model.tie_head and model.head.param_specs().keys() <= model.ignored_names()
    plain_one = build_model(config_from_dict(dict(KB)))
    assert not any(".hc" in name for name in plain_one.param_specs())


# -- schedules ---------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("case", sorted(CASES))
@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed"])
def test_every_schedule_matches_the_plain_implementation(case, schedule, tmp_path):
    lengths = (5, 17, 33, 70, 41, 1, 64, 90, 20, 2) if schedule == "mixed" else (70, 33, 1, 2)
    requests = requests_of(case, lengths)
    if schedule == "whole":
        steps = traces.whole(requests)
    elif schedule == "tail":
        steps = traces.tail_decoded(requests, 32)
    elif schedule == "portions":
        steps = traces.changing_portions(requests, sizes=(2, 7, 1, 3, 33, 2, 2, 16, 5))
    else:
        steps = traces.mixed(requests, seed=11, budget_tokens=256)
        assert max(len(s["entries"]) for s in steps) >= 3 and sum(lengths) > traces.peak_tokens(steps)
    check(case, run(case, steps, tmp_path), requests)


def test_the_stream_behind_every_layer_run_is_the_plain_implementations():
    """The summed streams behind each run of a layer, a looped layer once a pass."""
    raw, tensors = plain_model("KA")
    tokens = random_tokens(97, 23, 2)
    kept = []
    plain.forward(raw, tensors, tokens, keep=kept)
    runner = runner_for("KA", 64)
    runner.cache.open("r")
    seen = []
    runner.model.after_call = lambda run, streams, pending: seen.append(streams.sum(dim=0).clone())
    runner.step([StepEntry("r", tokens, [])])
    assert len(seen) == len(kept) == 6
    for run, (got, expected) in enumerate(zip(seen, kept)):
        np.testing.assert_allclose(got.numpy(), expected.numpy(), atol=1e-4, rtol=1e-4, err_msg=f"run {run}")


def test_prefill_equals_token_by_token_decoding_from_the_first_token(tmp_path):
    """Every token alone, from position 0: memories, maxima and cache rows start from nothing."""
    for case in ("KA", "KD"):
        requests = requests_of(case, (40,))
        check(case, run(case, traces.tail_decoded(requests, 64), tmp_path / case), requests)


@pytest.mark.parametrize("case", ["KA", "KD"])
@pytest.mark.parametrize("chunk", [5, 16, 64])
def test_long_portions_through_the_chunked_form_of_the_memory(case, chunk, tmp_path):
    """Steps that bring many tokens run their memories in chunks (products over a chunk's tokens, the state walked from
    chunk to chunk), steps of single tokens as the scan; both leave the same state and logits, whatever the chunks' size
    and wherever a portion ends: in the middle of a chunk, at its last token, one token into the next."""
    requests = requests_of(case, (3 * chunk + 1, 2 * chunk, chunk - 1 if chunk > 2 else 2, 70))
    steps = traces.changing_portions(requests, sizes=(chunk + 3, 2, 2 * chunk, 1, chunk))
    ops = ChunkedMemoryOps(chunk=chunk, chunked_from=chunk // 2)
    runner = make_runner(model_folder(case), "float32", traces.peak_tokens(steps), CASES[case][2], device="cpu", ops=ops, max_live=4)
    replay(runner, traces.to_lines(steps).splitlines(), str(tmp_path), io.StringIO())
    runner.cache.check_invariants()
    assert ops.chunked_steps > 0
    check(case, traces.collect(steps, str(tmp_path), CASES[case][0]["vocab"]), requests)


@pytest.mark.parametrize("page", [4, 8, 64])
def test_page_sizes_and_page_borders(page, tmp_path):
    requests = requests_of("KA", (2 * page + 1, page, page - 1, page + 1))
    steps = traces.changing_portions(requests, sizes=(page - 1, 2, page, 1, page + 1))
    check("KA", run("KA", steps, tmp_path, page=page), requests)


def test_state_slots_and_pages_are_used_again_in_any_order():
    """Eight requests through four slots: a slot's next holder must start from zeros (matrix, normaliser and maximum),
    not from its predecessor's state, and windows give pages back while the requests still run."""
    runner = runner_for("KA", 4 * 64, live=4)
    tokens = {i: random_tokens(97, 28 + 5 * i, 900 + i) for i in range(8)}
    got = {}
    for first in (0, 4):
        live = list(range(first, first + 4))
        for rid in live:
            runner.cache.open(rid)
        assert sorted(runner.cache.record(rid).state_slot for rid in live) == [0, 1, 2, 3]
        done = {rid: 0 for rid in live}
        turn = 0
        while any(done[rid] < len(tokens[rid]) for rid in live):
            entries = []
            for rid in live[::-1] if turn % 2 else live:
                size = (1, 3, 2, 7)[(rid + turn) % 4]
                if done[rid] < len(tokens[rid]):
                    piece = tokens[rid][done[rid]:done[rid] + size]
                    entries.append(StepEntry(rid, piece, list(range(len(piece)))))
            logits = runner.step(entries)
            row = 0
            for entry in entries:
                for _ in entry.tokens:
                    got[(entry.request_id, done[entry.request_id])] = logits[row].numpy()
                    done[entry.request_id] += 1
                    row += 1
            turn += 1
        windowed = [group for group in runner.cache.groups if getattr(group.spec, "window", None) == 7]
        assert windowed                                   # the layers with a window of 7 keys: at most two pages of 16 are held
        for group in windowed:
            assert all(sum(page >= 0 for page in runner.cache.record(rid).tables[group.index]) <= 2 for rid in live)
        for rid in live[::-1]:
            runner.cache.close(rid)
    for (rid, position), logits in got.items():
        expected = plain_logits("KA", tuple(tokens[rid]))[position].numpy()
        np.testing.assert_allclose(logits, expected, atol=1e-4, rtol=3e-4, err_msg=f"{rid} {position}")


# -- mechanisms that random weights could hide ---------------------------------------------------------------------
def sharpened(case, change, change_config=None):
    """The case's tensors with ``change(tensors)`` applied, written to a folder of its own; (folder, config, tensors)."""
    from safetensors.torch import save_file
    raw, tensors = plain_model(case)
    tensors = {name: tensor.clone() for name, tensor in tensors.items()}
    change(tensors)
    raw = copy_of(raw)
    if change_config is not None:
        change_config(raw)
    folder = tempfile.mkdtemp(prefix="llmserver_amd_test_sharp_")
    save_file({name: tensor.to(torch.bfloat16).contiguous() for name, tensor in tensors.items()}, os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(raw, handle)
    return (folder, *plain.read_folder(folder))


def logits_of(folder, tokens, cuts, page=8):
    runner = make_runner(folder, "float32", 64 * (-(-len(tokens) // 64)), page, device="cpu", ops=TorchOps())
    runner.cache.open("r")
    rows, start = [], 0
    for size in cuts:
        piece = tokens[start:start + size]
        if not piece:
            break
        rows.append(runner.step([StepEntry("r", piece, list(range(len(piece))))]).clone())
        start += len(piece)
    assert start == len(tokens)
    return torch.cat(rows).numpy()


def test_a_token_hundreds_back_decides_through_the_matrix_memory():
    """Forget gates pushed to one keep everything for ever: what the memory took in hundreds of tokens ago decides the
    logits, in a prompt and for decoded tokens (both attentions of this case see 40 keys at most, so nothing else
    reaches that far); a state that is lost, or cut off where a portion starts, shows."""
    def change(tensors):
        tensors["l1.mix.f.b"][:] = 40.0                    # under the cap of 12: logsigmoid(12), the state loses six millionths a token
        tensors["l1.mix.i"] *= 0.2                         # (inputs of about equal weight, so that early ones stay a part of the sum)
        tensors["l1.mix.i.b"][:] = 0.0
    folder, raw, tensors = sharpened("KD", change)
    tokens = random_tokens(200, 300, 5)
    expected = plain.forward(raw, tensors, tokens).numpy()
    other = plain.forward(raw, tensors, random_tokens(200, 20, 6) + tokens[20:]).numpy()
    assert np.abs(other[-1] - expected[-1]).max() > 1e-2
    for cuts in ([300], [280] + [1] * 20, [3, 150, 2, 100, 45]):
        np.testing.assert_allclose(logits_of(folder, tokens, cuts, page=16), expected, atol=2e-4, rtol=5e-4, err_msg=str(cuts))


def test_a_key_hundreds_back_among_hundreds_decides_in_full_attention():
    """Queries and keys of the attention without a window scaled up: a few keys carry all the weight, and which ones
    depends on the whole context; the plain implementation with a window of 150 gives other logits at the end."""
    def change(tensors):
        tensors["l3.mix.q"] *= 5.0
        tensors["l3.mix.k"] *= 5.0
        tensors["l1.mix.q"] *= 3.0
    folder, raw, tensors = sharpened("KB", change)
    tokens = random_tokens(130, 260, 15)
    expected = plain.forward(raw, tensors, tokens).numpy()
    short = copy_of(raw)
    short["layers"][3]["mixer"]["mask"] = {"size": 150}
    short["layers"][1]["mixer"]["mask"] = {"size": 150}
    assert np.abs(plain.forward(short, tensors, tokens).numpy()[200:] - expected[200:]).max() > 1e-2
    for cuts in ([260], [230] + [1] * 30, [129, 2, 64, 65]):
        for page in (8, 64):
            np.testing.assert_allclose(logits_of(folder, tokens, cuts, page), expected, atol=2e-4, rtol=5e-4, err_msg=f"{cuts} {page}")


@pytest.mark.parametrize("case,layer,names,window", [("KA", 1, ("q", "uk"), 7), ("KB", 0, ("q", "k"), 5), ("KC", 0, ("q", "uk"), 1)])
def test_keys_just_inside_and_just_outside_the_window_in_prompts_and_decoding(case, layer, names, window):
    """Attention made sharp: a layer with a window of w keys sees exactly the token itself and the w - 1 before it; the
    plain implementation with a window one longer or one shorter gives other logits, so an edge that is one off shows."""
    def change(tensors):
        for name in names:
            tensors[f"l{layer}.mix.{name}"] *= 4.0
    folder, raw, tensors = sharpened(case, change)
    assert raw["layers"][layer]["mixer"]["mask"]["size"] == window
    tokens = random_tokens(raw["vocab"], 90, 7)
    expected = plain.forward(raw, tensors, tokens).numpy()
    for off in (window - 1, window + 1):
        if off:
            wrong = copy_of(raw)
            wrong["layers"][layer]["mixer"]["mask"]["size"] = off
            assert np.abs(plain.forward(wrong, tensors, tokens).numpy()[10:] - expected[10:]).max() > 1e-2
    for cuts in ([90], [60] + [1] * 30, [5, 2, 7, 1, 6, 8, 9, 2, 50], [window, 90 - window], [window - 1 or 2, 91 - (window - 1 or 2)], [window + 1, 89 - window]):
        for page in (4, 16):
            np.testing.assert_allclose(logits_of(folder, tokens, cuts, page), expected, atol=1e-4, rtol=5e-4, err_msg=f"{cuts} {page}")


def test_the_values_are_the_keys_before_their_rotation():
    """The plain implementation with the rotated keys as values gives other logits; the engine gives the design's."""
    folder, raw, tensors = sharpened("KB", lambda tensors: None)
    tokens = random_tokens(130, 50, 3)
    expected = plain.forward(raw, tensors, tokens).numpy()
    kept = plain.softmax_attention
    try:
        plain.softmax_attention = lambda q, k, v, scale, window, r=plain.same: kept(q, k, k if v.shape == k.shape else v, scale, window, r)
        assert np.abs(plain.forward(raw, tensors, tokens).numpy() - expected).max() > 1e-2
    finally:
        plain.softmax_attention = kept
    for cuts in ([50], [20] + [1] * 30):
        np.testing.assert_allclose(logits_of(folder, tokens, cuts), expected, atol=1e-4, rtol=3e-4)


def test_streams_mix_from_row_to_column_and_every_stream_gets_its_own_share():
    """Mixing matrices far from symmetric, reads and writes that differ by stream and in sign: a matrix read the other
    way round, or a result written with one weight into all streams, gives other logits."""
    def change(tensors):
        generator = torch.Generator().manual_seed(4)
        for name in list(tensors):
            if name.endswith(".mix") and ".hc" in name:
                size = tensors[name].shape[0]
                tensors[name] = 0.6 * torch.eye(size, dtype=torch.float64) + 0.5 * torch.triu(torch.rand(size, size, generator=generator, dtype=torch.float64), 1)
            elif name.endswith(".out") and ".hc" in name:
                tensors[name] = torch.linspace(-1.0, 1.5, tensors[name].shape[0], dtype=torch.float64)
            elif name.endswith(".in") and ".hc" in name:
                tensors[name] = torch.linspace(1.2, -0.4, tensors[name].shape[0], dtype=torch.float64)
    folder, raw, tensors = sharpened("KA", change)
    tokens = random_tokens(97, 60, 9)
    expected = plain.forward(raw, tensors, tokens).numpy()
    turned = {name: (tensor.T.contiguous() if name.endswith(".mix") and ".hc" in name else tensor) for name, tensor in tensors.items()}
    assert np.abs(plain.forward(raw, turned, tokens).numpy() - expected).max() > 1e-2
    for cuts in ([60], [1] * 60, [2, 1, 3, 4, 5, 1, 1, 6, 2, 35]):
        np.testing.assert_allclose(logits_of(folder, tokens, cuts), expected, atol=1e-4, rtol=3e-4, err_msg=str(cuts))


@pytest.mark.parametrize("bias", [-6.0, 5.0])
def test_the_gates_cap_and_both_sides_of_the_memorys_denominator(bias):
    """Gate projections scaled far beyond the cap, so that the cap decides the gates; input gates pushed far down
    (exp(-m) stands below the read-out) and far up (|n . q| does).  Another cap gives other logits."""
    def change(tensors):
        for layer in (0, 3):
            tensors[f"l{layer}.mix.i"] *= 25.0
            tensors[f"l{layer}.mix.f"] *= 25.0
            tensors[f"l{layer}.mix.i.b"][:] = bias
    folder, raw, tensors = sharpened("KA", change)
    tokens = random_tokens(97, 70, 21)
    expected = plain.forward(raw, tensors, tokens).numpy()
    other = copy_of(raw)
    for layer in (0, 3):
        other["layers"][layer]["mixer"]["gate_cap"] *= 2.0
    assert np.abs(plain.forward(other, tensors, tokens).numpy() - expected).max() > 1e-2
    for cuts in ([70], [1] * 70, [3, 40, 2, 25]):
        np.testing.assert_allclose(logits_of(folder, tokens, cuts), expected, atol=2e-4, rtol=5e-4, err_msg=str(cuts))


def test_every_pass_of_a_looped_layer_keeps_a_cache_and_a_state_of_its_own():
    """A case whose every layer is passed twice: with one cache or state shared by the passes, decoding would read the
    other pass's rows.  The same weights unrolled into twice as many layers give the same logits."""
    raw, tensors = plain_model("KD")
    tokens = random_tokens(200, 75, 13)
    unrolled = copy_of(raw)
    del unrolled["loop"]
    unrolled["layers"] = raw["layers"] * 2
    doubled = dict(tensors)
    for name, tensor in tensors.items():
        if name.startswith("l"):
            index, rest = name[1:].split(".", 1)
            doubled[f"l{int(index) + 3}.{rest}"] = tensor
    expected = plain.forward(raw, tensors, tokens).numpy()
    np.testing.assert_allclose(plain.forward(unrolled, doubled, tokens).numpy(), expected, atol=1e-9)
    for cuts in ([75], [50] + [1] * 25, [2, 33, 7, 33]):
        np.testing.assert_allclose(logits_of(model_folder("KD"), tokens, cuts, page=16), expected, atol=1e-4, rtol=3e-4, err_msg=str(cuts))


# -- the oracle itself -------------------------------------------------------------------------------------------------
def test_the_oracles_mechanisms_by_hand():
    f64 = lambda values: torch.tensor(values, dtype=torch.float64)
    assert torch.allclose(plain.norm(f64([[3.0, 4.0]]), f64([1.0, 2.0]), 0.0), f64([[3.0, 8.0]]) / 12.5 ** 0.5)
    # the halves layout turns dimension 0 with dimension 1 of a two-dimensional rotation and leaves the third
    quarter = plain.rotate_halves(f64([[[1.0, 0.0, 5.0]]]), torch.tensor([1]), 10.0, 2)
    assert torch.allclose(quarter, f64([[[np.cos(1.0), np.sin(1.0), 5.0]]]))
    # four dimensions: halves pair (0, 2) and (1, 3), neighbours pair (0, 1) and (2, 3); the second pair turns by p / base^(1/2)
    x = f64([[[1.0, 2.0, 3.0, 4.0]]])
    a, b = 3.0, 3.0 / 100.0 ** 0.5
    halves = plain.rotate_halves(x, torch.tensor([3]), 100.0, 4)
    assert torch.allclose(halves, f64([[[np.cos(a) - 3 * np.sin(a), 2 * np.cos(b) - 4 * np.sin(b), 3 * np.cos(a) + np.sin(a), 4 * np.cos(b) + 2 * np.sin(b)]]]))
    pairs = plain.rotate_neighbours(x, torch.tensor([3]), 100.0, 4)
    assert torch.allclose(pairs, f64([[[np.cos(a) - 2 * np.sin(a), 2 * np.cos(a) + np.sin(a), 3 * np.cos(b) - 4 * np.sin(b), 4 * np.cos(b) + 3 * np.sin(b)]]]))
    # a shift of all positions changes no score
    q, k = torch.randn(4, 1, 6, dtype=torch.float64), torch.randn(4, 1, 6, dtype=torch.float64)
    for turn in (plain.rotate_halves, plain.rotate_neighbours):
        scores = lambda shift: turn(q, torch.arange(4) + shift, 50.0, 4)[:, 0] @ turn(k, torch.arange(4) + shift, 50.0, 4)[:, 0].T
        assert torch.allclose(scores(0), scores(900), atol=1e-9)
    assert plain.visible(5, 2).tolist() == [[True, False, False, False, False], [True, True, False, False, False], [False, True, True, False, False],
                                            [False, False, True, True, False], [False, False, False, True, True]]
    assert plain.layer_runs({"layers": [0] * 5, "loop": {"start": 1, "stop": 3, "times": 3}}) == [0, 1, 2, 1, 2, 1, 2, 3, 4]
    # the squared rectifier
    t = {"p.up": f64([[1.0], [-1.0]]), "p.down": f64([[1.0, 1.0]])}
    assert torch.allclose(plain.feed_forward(f64([[3.0], [-2.0]]), t, "p."), f64([[9.0], [4.0]]))
    # two streams by hand: x_t <- sum_s mix[s, t] x_s + mult * out[t] * y
    x = f64([[[1.0]], [[10.0]]])
    t = {"c.mix": f64([[1.0, 2.0], [0.0, 3.0]]), "c.out": f64([1.0, -1.0])}
    assert torch.allclose(plain.connect(x, f64([[4.0]]), t, "c.", 0.5), f64([[[1.0 + 2.0]], [[2.0 + 30.0 - 2.0]]]))
    # the memory by hand, one head of one channel, keys, values and queries of one, gates' projections zero:
    # i = 0, f = log(1/2), m stays 0: S = n = 1, 1.5, 1.75; the read-outs S / max(n, 1) are all 1, and the unit norm keeps 1
    one = f64([[1.0]])
    t = {"p.q": one, "p.k": one, "p.v": one, "p.g": one * 0, "p.o": one, "p.norm": f64([2.0]), "p.i": one * 0, "p.f": one * 0, "p.i.b": f64([0.0]),
         "p.f.b": f64([0.0])}
    out = plain.matrix_memory(torch.ones(3, 1, dtype=torch.float64), t, "p.", {"heads": 1, "dim": 1, "vdim": 1, "gate_cap": 5.0}, 0.0, floor=0.0)
    assert torch.allclose(out, torch.ones(3, 1, dtype=torch.float64))          # 2 (the norm's weight) * sigmoid(0)
    # an input gate of log 3 at every token: m = log 3 from the first token on, S = n = 1, 1.5, ..; exp(-m) = 1/3 lies below
    t["p.i.b"] = f64([np.log(3.0)])
    assert abs(float(plain.capped(f64(100.0), 5.0)) - 5.0) < 1e-9 and abs(float(plain.capped(f64(0.1), 5.0)) - 0.1) < 1e-4
    out = plain.matrix_memory(torch.ones(2, 1, dtype=torch.float64), t, "p.", {"heads": 1, "dim": 1, "vdim": 1, "gate_cap": 50.0}, 0.0, floor=0.0)
    assert torch.allclose(out, torch.ones(2, 1, dtype=torch.float64), atol=1e-6)


# -- generation through the entry point, the scheduler and the engine ------------------------------------------------------
def test_greedy_generation_through_the_entry_point_equals_the_oracles():
    """More requests than places, prompts cut into portions by the token budget, a pool so small that requests wait
    for pages: the engine's own scheduler, cache manager, step function and sampler produce the oracle's tokens."""
    from llmserver_amd.entrypoints import generate
    for case, vocab in (("KA", 97), ("KB", 130)):
        raw, tensors = plain_model(case)
        prompts = [random_tokens(vocab, n, 700 + n) for n in (19, 3, 41, 8, 1, 27)]
        expected = [plain.greedy_generate(raw, tensors, prompt, 7) for prompt in prompts]
        got = generate(model_folder(case), prompts, max_new_tokens=7, dtype="float32", device="cpu", block_size=8, num_blocks=26,
                       max_batch_size=3, max_num_batched_tokens=24, prefill_chunk_size=16, ops=TorchOps())
        assert got == expected
