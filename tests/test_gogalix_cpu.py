"""Gogalix through the engine's own step function, cache manager, scheduler and entry point on the CPU (torch twins
of the kernels) against the plain implementation: configuration and weights, each mechanism, every way of cutting
and batching, pages and state slots used again, windows' edges, far keys and far writes, layers that read another
layer's pages, and greedy generation."""
import io
import json
import os
import tempfile

import numpy as np
import pytest
import torch

import plain_gogalix as plain
import traces
from helpers import random_tokens
from llmserver_amd.config import ConfigError, UnsupportedModelError, config_from_dict
from llmserver_amd.engine.batch import StepEntry
from llmserver_amd.engine.replay import make_runner, replay
from llmserver_amd.parts import PagedKVSpec, StateSpec
from llmserver_amd.weights import build_model
from tiny_gogalix import CASES, GA, GB, GC, model_folder, plain_logits, plain_model
from torch_ops import TorchOps


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
    config = config_from_dict(dict(GA))
    assert config_from_dict(config.to_dict()) == config
    assert config.layers[2].mlp is None and config.layers[0].mixer.window == 7 and config.layers[3].mixer.kv_from == 0
    assert config.layers[1].mixer.taps == 3 and not config.layers[1].mixer.per_channel and config.layers[2].mixer.per_channel
    assert config.layers[1].mlp.experts == 6 and config.layers[1].mlp.top == 2 and config.layers[0].mlp.ff == 40
    assert config.norm_eps == 1e-5 and config.embedding_scale == 3.0 and config.layers[3].mixer.diff == 0.3
    other = config_from_dict(dict(GB))
    assert other.embedding_scale == 1.0 and other.layers[2].mixer.window is None and other.layers[2].mixer.kv_heads == 1
    for change, error, match in (
            (lambda raw: raw["layers"][1].update(type="something else"), UnsupportedModelError, "something else"),
            (lambda raw: raw["layers"][1]["mlp"].update(kind="other"), UnsupportedModelError, "other"),
            (lambda raw: raw["layers"][0]["mixer"].pop("diff"), ConfigError, "diff"),
            (lambda raw: raw["layers"][1]["mixer"].pop("conv"), ConfigError, "conv"),
            (lambda raw: raw["layers"][0]["mixer"].update(kv_heads=3), ConfigError, "multiple"),
            (lambda raw: raw["layers"][1]["mixer"].update(kv_heads=3), ConfigError, "multiple"),
            (lambda raw: raw["layers"][3]["mixer"].update(kv_from=1), ConfigError, "kv_from"),
            (lambda raw: raw["layers"][3]["mixer"].update(kv_from=3), ConfigError, "kv_from"),
            (lambda raw: raw["layers"][3]["mixer"].update(vdim=12), ConfigError, "differ"),
            (lambda raw: raw["layers"][1]["mlp"]["router"].update(top=7), ConfigError, "experts"),
            (lambda raw: raw["layers"][1]["mixer"].update(dim=300), UnsupportedModelError, "key channels"),
            (lambda raw: raw["layers"][0]["mixer"].update(vdim=300), UnsupportedModelError, "heads of")):
        raw = copy_of(GA)
        change(raw)
        with pytest.raises(error, match=match):
            config_from_dict(raw)


def test_the_model_declares_the_checkpoints_tensors_and_its_caches():
    model = build_model(config_from_dict(dict(GA)))
    specs = model.param_specs()
    assert {"embed", "head", "final.norm", "l0.norm1", "l0.mix.q", "l0.mix.k", "l0.mix.v", "l0.mix.lq1", "l0.mix.lk2", "l0.mix.o", "l0.ls1", "l0.ls2",
            "l0.rg1", "l0.rg1.b", "l0.rg2.b", "l0.mlp.gate.b", "l0.mlp.down.b", "l1.mix.q.conv", "l1.mix.v.conv", "l1.mix.b", "l1.mix.a", "l1.mix.A_log",
            "l1.mix.dt_bias", "l1.mix.g", "l1.mix.norm", "l1.mlp.router", "l1.mlp.router.b", "l1.mlp.e5.down", "l2.mix.a1", "l2.mix.a2", "l2.mix.g1",
            "l2.mix.g2", "l2.rg1", "l3.mix.q", "l3.mix.lq2"} <= set(specs)
    assert not {"l3.mix.k", "l3.mix.v", "l2.mlp.gate", "l2.ls2", "l2.rg2", "l2.rg2.b", "l1.mix.a1", "l2.mix.a", "l2.mix.g", "l0.norm2", "l1.mlp.e6.up",
                "l1.mlp.e0.gate.b", "l0.mix.q.b", "l5.norm1"} & set(specs)
    assert specs["l0.norm1"].shape == () and specs["final.norm"].shape == () and specs["head"].shape == (97, 48)
    assert specs["l0.mix.q"].shape == (4 * 2 * 6, 48) and specs["l0.mix.k"].shape == (2 * 2 * 6, 48) and specs["l0.mix.v"].shape == (2 * 10, 48)
    assert specs["l0.mix.o"].shape == (48, 40) and specs["l0.mix.lq1"].shape == (6,) and specs["l0.rg1"].shape == (48, 48)
    assert specs["l1.mix.q"].shape == (16, 48) and specs["l1.mix.v"].shape == (24, 48) and specs["l1.mix.q.conv"].shape == (16, 3)
    assert specs["l1.mix.v.conv"].shape == (24, 3) and specs["l1.mix.b"].shape == (4, 48) and specs["l1.mix.dt_bias"].shape == (4,)
    assert specs["l2.mix.a1"].shape == (5, 48) and specs["l2.mix.a2"].shape == (24, 5) and specs["l2.mix.g2"].shape == (10, 7)
    assert specs["l2.mix.dt_bias"].shape == (24,) and specs["l2.mix.A_log"].shape == (2,) and specs["l2.mix.norm"].shape == (5,)
    caches = model.cache_specs()
    assert sorted(caches) == [0, 1, 2, 4]                    # the fourth layer reads the first one's pages
    assert caches[0] == PagedKVSpec(4, 16, 11)               # two maps of two key heads; kept for the longer of the two windows
    # (a delta rule's matrices are kept in blocks of 16 value columns, the last one filled up)
    assert caches[1] == StateSpec((4 * 8 * 16 + 2 * (16 + 16 + 24),), "float32") and caches[2] == StateSpec((2 * 12 * 16 + 3 * (12 + 12 + 10) + 2,), "float32")
    assert [(call.block, call.cache, call.writes_cache) for call in model.order] == [(0, 0, True), (1, 1, True), (2, 2, True), (3, 0, False), (4, 4, True)]
    assert not model.tie_head and not model.ignored_names()
    assert build_model(config_from_dict(dict(GB))).cache_specs()[2] == PagedKVSpec(2, 32, None)      # read through a window, kept for ever


def test_inner_sizes_that_no_key_names_are_read_off_the_tensors(tmp_path):
    """A folder whose configuration does not say the inner sizes of the low-rank maps loads as the one that does."""
    raw, tensors = plain_model("GA")
    bare = copy_of(raw)
    for key in ("low", "gate_low"):
        del bare["layers"][2]["mixer"][key]
    folder = str(tmp_path / "bare")
    os.makedirs(folder)
    os.symlink(os.path.join(model_folder("GA"), "model.safetensors"), os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(bare, handle)
    tokens = random_tokens(97, 20, 4)
    np.testing.assert_allclose(logits_of(folder, tokens, [13, 7]), plain_logits("GA", tuple(tokens)).numpy(), atol=1e-4, rtol=3e-4)


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


def test_the_stream_behind_every_layer_is_the_plain_implementations():
    raw, tensors = plain_model("GA")
    tokens = random_tokens(97, 23, 2)
    kept = []
    plain.forward(raw, tensors, tokens, layer_outputs=kept)
    runner = runner_for("GA", 64)
    runner.cache.open("r")
    seen = []
    runner.model.after_call = lambda run, stream, pending: seen.append(stream.clone())
    runner.step([StepEntry("r", tokens, [])])
    assert len(seen) == len(kept) == 5
    for layer, (got, expected) in enumerate(zip(seen, kept)):
        np.testing.assert_allclose(got.numpy(), expected.numpy(), atol=1e-4, rtol=1e-4, err_msg=f"layer {layer}")


def test_prefill_equals_token_by_token_decoding_from_the_first_token(tmp_path):
    """Every token alone, from position 0: states, convolutions' inputs and cache rows start from nothing."""
    for case in ("GA", "GC"):
        requests = requests_of(case, (40,))
        check(case, run(case, traces.tail_decoded(requests, 64), tmp_path / case), requests)


def test_portions_down_to_two_tokens_and_shorter_than_the_convolutions_reach(tmp_path):
    """Portions of two tokens and single tokens in turn: a convolution of five taps reads four inputs back, over several
    earlier steps."""
    requests = requests_of("GC", (37, 12))
    check("GC", run("GC", traces.changing_portions(requests, sizes=(2, 2, 1, 2, 1, 1, 2, 3)), tmp_path), requests)


@pytest.mark.parametrize("page", [4, 8, 64])
def test_page_sizes_and_page_borders(page, tmp_path):
    requests = requests_of("GA", (2 * page + 1, page, page - 1, page + 1))
    steps = traces.changing_portions(requests, sizes=(page - 1, 2, page, 1, page + 1))
    check("GA", run("GA", steps, tmp_path, page=page), requests)


def test_state_slots_and_pages_are_used_again_in_any_order():
    """Eight requests through four slots: a slot's next holder must start from zeros (matrices and the convolutions' last
    inputs), not from its predecessor's state, and windows give pages back while the requests still run."""
    runner = runner_for("GA", 4 * 64, live=4)
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
        windowed = [group for group in runner.cache.groups if getattr(group.spec, "window", None) == 11]
        assert windowed                                   # the pages two layers read through windows of 7 and 11 keys: at most two of 16 are held
        for group in windowed:
            assert all(sum(page >= 0 for page in runner.cache.record(rid).tables[group.index]) <= 2 for rid in live)
        for rid in live[::-1]:
            runner.cache.close(rid)
    for (rid, position), logits in got.items():
        expected = plain_logits("GA", tuple(tokens[rid]))[position].numpy()
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


@pytest.mark.parametrize("layer", [1, 2])
def test_a_write_hundreds_of_tokens_back_decides_through_the_delta_rules_state(layer):
    """Decays pushed to one keep what the state took in for ever: tokens hundreds of places back decide the logits, in a
    prompt and for decoded tokens (the attentions of this case see 40 keys at most); a state that is lost, or cut off
    where a portion starts, shows."""
    def change(tensors):
        tensors[f"l{layer}.mix.A_log"][:] = -9.0
    folder, raw, tensors = sharpened("GC", change)
    tokens = random_tokens(200, 300, 5)
    expected = plain.forward(raw, tensors, tokens).numpy()
    other = plain.forward(raw, tensors, random_tokens(200, 20, 6) + tokens[20:]).numpy()
    assert np.abs(other[-1] - expected[-1]).max() > 1e-2
    for cuts in ([300], [280] + [1] * 20, [3, 150, 2, 100, 45]):
        np.testing.assert_allclose(logits_of(folder, tokens, cuts, page=16), expected, atol=2e-4, rtol=5e-4, err_msg=str(cuts))


def test_a_key_hundreds_back_among_hundreds_decides_in_attention_without_a_window():
    """Queries and keys of the attention without a window scaled up: a few keys carry all the weight, and which ones
    depends on the whole context; the plain implementation with a window of 150 gives other logits at the end.  The last
    layer reads the same pages through its own window of nine keys."""
    def change(tensors):
        tensors["l2.mix.q"] *= 6.0
        tensors["l2.mix.k"] *= 6.0
    folder, raw, tensors = sharpened("GB", change)
    tokens = random_tokens(130, 260, 15)
    expected = plain.forward(raw, tensors, tokens).numpy()
    short = copy_of(raw)
    short["layers"][2]["mixer"]["mask"] = {"size": 150}
    assert np.abs(plain.forward(short, tensors, tokens).numpy()[200:] - expected[200:]).max() > 1e-2
    for cuts in ([260], [230] + [1] * 30, [129, 2, 64, 65]):
        for page in (8, 64):
            np.testing.assert_allclose(logits_of(folder, tokens, cuts, page), expected, atol=2e-4, rtol=5e-4, err_msg=f"{cuts} {page}")


@pytest.mark.parametrize("case,layer,window", [("GA", 0, 7), ("GA", 3, 11), ("GB", 1, 5), ("GB", 4, 9), ("GC", 4, 1), ("GC", 3, 33)])
def test_keys_just_inside_and_just_outside_the_window_in_prompts_and_decoding(case, layer, window):
    """Attention made sharp: a layer with a window of w keys sees exactly the token itself and the w - 1 before it; the
    plain implementation with a window one longer or one shorter gives other logits, so an edge that is one off shows.
    Among the layers are some that read another layer's pages through a window shorter or longer than their owner's."""
    def change(tensors):
        tensors[f"l{layer}.mix.q"] *= 5.0
        source = CASES[case][0]["layers"][layer]["mixer"].get("kv_from", layer)
        tensors[f"l{source}.mix.k"] *= 3.0
    folder, raw, tensors = sharpened(case, change)
    assert raw["layers"][layer]["mixer"]["mask"]["size"] == window
    tokens = random_tokens(raw["vocab"], 90, 7)
    expected = plain.forward(raw, tensors, tokens).numpy()
    for off in (window - 1, window + 1):
        if off:
            wrong = copy_of(raw)
            wrong["layers"][layer]["mixer"]["mask"]["size"] = off
            assert np.abs(plain.forward(wrong, tensors, tokens).numpy()[window:] - expected[window:]).max() > 1e-2
    for cuts in ([90], [60] + [1] * 30, [5, 2, 7, 1, 6, 8, 9, 2, 50], [window, 90 - window], [window - 1 or 2, 91 - (window - 1 or 2)], [window + 1, 89 - window]):
        for page in (4, 16):
            np.testing.assert_allclose(logits_of(folder, tokens, cuts, page), expected, atol=1e-4, rtol=5e-4, err_msg=f"{cuts} {page}")


def test_the_second_map_counts_with_the_layers_lambda_and_both_maps_share_the_values():
    """The vectors behind lambda made large: a difference without the second map, with another lambda, or with the maps
    exchanged gives other logits."""
    def change(tensors):
        for layer in (0, 3):
            tensors[f"l{layer}.mix.lq1"][:] = 0.5
            tensors[f"l{layer}.mix.lk1"][:] = 0.3
            tensors[f"l{layer}.mix.lq2"][:] = -0.4
            tensors[f"l{layer}.mix.lk2"][:] = 0.25
    folder, raw, tensors = sharpened("GA", change)
    tokens = random_tokens(97, 50, 3)
    expected = plain.forward(raw, tensors, tokens).numpy()
    for name in ("l0.mix.lq1", "l3.mix.lk2"):
        other = dict(tensors)
        other[name] = tensors[name] * 0.0
        assert np.abs(plain.forward(raw, other, tokens).numpy() - expected).max() > 1e-2
    exchanged = dict(tensors)
    exchanged["l3.mix.q"] = tensors["l3.mix.q"].view(4, 2, 6, 48).flip(1).reshape(48, 48)
    assert np.abs(plain.forward(raw, exchanged, tokens).numpy() - expected).max() > 1e-2
    for cuts in ([50], [20] + [1] * 30, [2, 7, 41]):
        np.testing.assert_allclose(logits_of(folder, tokens, cuts), expected, atol=1e-4, rtol=3e-4, err_msg=str(cuts))


def test_a_layer_reads_the_pages_of_the_layer_it_names():
    """The same weights with the fourth layer reading another layer's keys and values give other logits."""
    raw, tensors = plain_model("GC")
    tokens = random_tokens(200, 60, 8)
    expected = plain.forward(raw, tensors, tokens).numpy()
    own = copy_of(raw)
    del own["layers"][3]["mixer"]["kv_from"]
    with_own = dict(tensors)
    with_own["l3.mix.k"], with_own["l3.mix.v"] = tensors["l0.mix.k"].flip(0), tensors["l0.mix.v"].flip(0)
    assert np.abs(plain.forward(own, with_own, tokens).numpy() - expected).max() > 1e-2
    for cuts in ([60], [35] + [1] * 25, [2, 33, 25]):
        np.testing.assert_allclose(logits_of(model_folder("GC"), tokens, cuts, page=16), expected, atol=1e-4, rtol=3e-4, err_msg=str(cuts))


def test_the_convolutions_taps_reach_back_over_earlier_steps_in_their_order():
    """Taps that weigh the oldest input most: taps read in the other order, or inputs lost where a portion starts, show."""
    def change(tensors):
        for layer, taps in ((1, 4), (5, 5)):
            for name in ("q", "k", "v"):
                weight = tensors[f"l{layer}.mix.{name}.conv"]
                weight *= torch.linspace(3.0, 0.3, taps, dtype=weight.dtype)
    folder, raw, tensors = sharpened("GC", change)
    tokens = random_tokens(200, 40, 19)
    expected = plain.forward(raw, tensors, tokens).numpy()
    turned = {name: (tensor.flip(1) if name.endswith(".conv") else tensor) for name, tensor in tensors.items()}
    assert np.abs(plain.forward(raw, turned, tokens).numpy() - expected).max() > 1e-2
    for cuts in ([40], [1] * 40, [2, 1, 3, 2, 2, 1, 1, 4, 24], [3, 1, 1, 1, 34]):
        np.testing.assert_allclose(logits_of(folder, tokens, cuts, page=16), expected, atol=1e-4, rtol=3e-4, err_msg=str(cuts))


def test_decays_per_key_channel_act_on_the_states_rows_and_grouped_key_heads_serve_their_value_heads():
    """A bias that spreads the decays of a head's key channels from none to strong: one decay per head (their mean), or
    decays laid out channel by head, give other logits.  Value heads 0, 1 read key head 0 and 2, 3 read key head 1."""
    def change(tensors):
        tensors["l2.mix.dt_bias"][:] = torch.linspace(-6.0, 3.0, 4 * 32, dtype=torch.float64)
        tensors["l2.mix.A_log"][:] = torch.tensor([0.5, -1.0, 0.0, 1.0], dtype=torch.float64)
    folder, raw, tensors = sharpened("GC", change)
    tokens = random_tokens(200, 50, 23)
    expected = plain.forward(raw, tensors, tokens).numpy()
    other = dict(tensors)
    other["l2.mix.dt_bias"] = tensors["l2.mix.dt_bias"].view(4, 32).T.reshape(-1)
    assert np.abs(plain.forward(raw, other, tokens).numpy() - expected).max() > 1e-2
    other = dict(tensors)
    other["l2.mix.k"] = tensors["l2.mix.k"].view(2, 32, 64).flip(0).reshape(64, 64)         # the key heads exchanged
    assert np.abs(plain.forward(raw, other, tokens).numpy() - expected).max() > 1e-2
    for cuts in ([50], [1] * 50, [17, 2, 31]):
        np.testing.assert_allclose(logits_of(folder, tokens, cuts, page=16), expected, atol=1e-4, rtol=3e-4, err_msg=str(cuts))


def test_the_routers_bias_decides_and_the_weights_are_the_softmax_over_the_chosen():
    """A bias far above the logits' spread fixes the choice: without it other experts are chosen and the logits differ."""
    def change(tensors):
        tensors["l1.mlp.router.b"][:] = torch.tensor([0.0, 9.0, -9.0, 0.0, 6.0, -3.0], dtype=torch.float64)
        tensors["l1.ls2"] *= 3.0
    folder, raw, tensors = sharpened("GA", change)
    tokens = random_tokens(97, 30, 29)
    expected = plain.forward(raw, tensors, tokens).numpy()
    other = dict(tensors)
    other["l1.mlp.router.b"] = tensors["l1.mlp.router.b"] * 0.0
    assert np.abs(plain.forward(raw, other, tokens).numpy() - expected).max() > 1e-2
    for cuts in ([30], [1] * 30):
        np.testing.assert_allclose(logits_of(folder, tokens, cuts), expected, atol=1e-4, rtol=3e-4, err_msg=str(cuts))


def test_the_streams_gates_and_scales_belong_to_their_sublayers():
    """Gates' biases and scales that differ widely between the two sublayers: exchanged, they give other logits."""
    def change(tensors):
        for layer in range(5):
            tensors[f"l{layer}.rg1.b"] += 2.0
            tensors[f"l{layer}.ls1"] *= 1.5
            if f"l{layer}.rg2.b" in tensors:
                tensors[f"l{layer}.rg2.b"] -= 2.0
    folder, raw, tensors = sharpened("GA", change)
    tokens = random_tokens(97, 25, 31)
    expected = plain.forward(raw, tensors, tokens).numpy()
    other = dict(tensors)
    other["l0.rg1.b"], other["l0.rg2.b"] = tensors["l0.rg2.b"], tensors["l0.rg1.b"]
    assert np.abs(plain.forward(raw, other, tokens).numpy() - expected).max() > 1e-2
    for cuts in ([25], [1] * 25):
        np.testing.assert_allclose(logits_of(folder, tokens, cuts), expected, atol=1e-4, rtol=3e-4, err_msg=str(cuts))


# -- the oracle itself -------------------------------------------------------------------------------------------------
def test_the_oracles_mechanisms_by_hand():
    f64 = lambda values: torch.tensor(values, dtype=torch.float64)
    assert torch.allclose(plain.scalar_norm(f64([[3.0, 4.0]]), f64(2.0), 0.0), f64([[6.0, 8.0]]) / 12.5 ** 0.5)
    # a convolution of three taps: the last column weighs the token itself, zeros stand in front of the sequence
    out = plain.causal_convolution(f64([[1.0], [10.0], [100.0]]), f64([[3.0, 2.0, 1.0]]))
    assert torch.allclose(out, f64([[1.0], [12.0], [123.0]]))
    assert torch.allclose(plain.unit_vectors(f64([[3.0, 4.0]])), f64([[0.6, 0.8]]), atol=1e-6)
    # the delta rule by hand, one head of two key channels and one value: write v = 2 under k = e1 with beta = 1, read it back;
    # write again under the same key with beta = 1/2: the state moves half the way to the new value; a decay halves it first
    q = k = f64([[[1.0, 0.0]], [[1.0, 0.0]], [[0.0, 1.0]]])
    out = plain.delta_rule(q, k, f64([[[2.0]], [[6.0]], [[5.0]]]), f64([[1.0], [0.5], [1.0]]), f64([[1.0], [0.5], [1.0]]))
    assert torch.allclose(out.flatten(), f64([2.0, 1.0 + 0.5 * (6.0 - 1.0), 5.0]))
    # decays per key channel act on the state's rows: the first channel keeps its content, the second loses it
    out = plain.delta_rule(f64([[[1.0, 1.0]], [[1.0, 1.0]]]), f64([[[1.0, 1.0]], [[0.0, 0.0]]]), f64([[[4.0]], [[0.0]]]), f64([[0.5], [1.0]]),
                           f64([[[1.0, 1.0]], [[1.0, 0.0]]]))
    assert torch.allclose(out.flatten(), f64([2.0 * 0.5 * 4.0, 0.5 * 4.0]))
    weights = plain.windowed_softmax(torch.zeros(1, 4, 4, dtype=torch.float64), 2)[0]
    assert torch.allclose(weights, f64([[1, 0, 0, 0], [0.5, 0.5, 0, 0], [0, 0.5, 0.5, 0], [0, 0, 0.5, 0.5]]))
    # differential attention by hand: one head, keys that score nothing (uniform maps), values 1 then 3: a1 = a2, so the
    # difference is (1 - lambda) a, normed to +-1, times 1 - diff
    t = {"p.q": torch.zeros(2, 1, dtype=torch.float64), "p.k": torch.zeros(2, 1, dtype=torch.float64), "p.v": f64([[1.0]]), "p.o": f64([[1.0]]),
         "p.lq1": f64([0.0]), "p.lk1": f64([0.0]), "p.lq2": f64([0.0]), "p.lk2": f64([0.0])}
    out, _ = plain.differential_attention(f64([[1.0], [3.0]]), t, "p", {"heads": 1, "kv_heads": 1, "dim": 1, "vdim": 1, "scale": 1.0, "diff": 0.25}, 0.0)
    assert torch.allclose(out.flatten(), f64([0.75, 0.75]))          # lambda = 1 - 1 + 0.25: (1 - 0.25) a, positive
    # two of three experts: the weights are the softmax over the chosen logits only
    t = {"m.router": f64([[1.0], [2.0], [0.0]]), "m.router.b": f64([0.0, 0.0, 5.0])}
    for e in range(3):
        t.update({f"m.e{e}.gate": f64([[1.0]]), f"m.e{e}.up": f64([[float(e + 1)]]), f"m.e{e}.down": f64([[1.0]])})
    out = plain.routed_feed_forward(f64([[1.0]]), t, "m", {"router": {"experts": 3, "top": 2}})
    share = 1.0 / (1.0 + np.exp(2.0 - 5.0))
    silu = 1.0 / (1.0 + np.exp(-1.0))
    assert torch.allclose(out, f64([[silu * (share * 3.0 + (1.0 - share) * 2.0)]]))


# -- generation through the entry point, the scheduler and the engine ------------------------------------------------------
def test_greedy_generation_through_the_entry_point_equals_the_oracles():
    """More requests than places, prompts cut into portions by the token budget, a pool so small that requests wait
    for pages: the engine's own scheduler, cache manager, step function and sampler produce the oracle's tokens."""
    from llmserver_amd.entrypoints import generate
    for case, vocab in (("GA", 97), ("GB", 130)):
        raw, tensors = plain_model(case)
        prompts = [random_tokens(vocab, n, 700 + n) for n in (19, 3, 41, 8, 1, 27)]
        expected = [plain.greedy_generate(raw, tensors, prompt, 7) for prompt in prompts]
        got = generate(model_folder(case), prompts, max_new_tokens=7, dtype="float32", device="cpu", block_size=8, num_blocks=26,
                       max_batch_size=3, max_num_batched_tokens=24, prefill_chunk_size=16, ops=TorchOps())
        assert got == expected
