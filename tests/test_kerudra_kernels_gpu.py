"""The kernels that Kerudra brought: several residual streams (their start, the read under a norm, the update behind a
sublayer with the next read folded in), the matrix memory with exponential gates and its normalised, gated read-out,
the squared rectifier, a gate per channel behind latent attention, and queries and keys turned in halves in front of
attention whose values are the keys; each against its plain torch twin, in float32 and in bfloat16, on sizes that are
no multiples of anything."""
import numpy as np
import pytest
import torch

from test_latent_experts_kernels_gpu import batch, close
from torch_ops import TorchOps

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from llmserver_amd.kernels import default_ops
    return default_ops()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("streams,width", [(1, 100), (2, 256), (3, 1027), (4, 4400)])
def test_streams_start_read_and_update(ops, dtype, streams, width):
    print(f"streams {dtype} {streams} {width}", flush=True)
    twin = TorchOps()
    n = 7
    table = torch.randn(19, width, device="cuda").to(dtype)
    ids = torch.randint(0, 19, (n,), device="cuda", dtype=torch.int32)
    start = [torch.empty(streams, n, width, device="cuda") for _ in range(2)]
    for which, out in zip((ops, twin), start):
        which.embedding_wide(table, ids, out, scale=3.5)
    assert torch.equal(start[0], start[1]) and torch.equal(start[0][0], start[0][-1])
    x = torch.randn(streams, n, width, device="cuda")
    read, write = torch.randn(streams, device="cuda"), torch.randn(streams, device="cuda")
    mix = torch.eye(streams, device="cuda") + 0.5 * torch.randn(streams, streams, device="cuda")
    weight = 1 + 0.2 * torch.randn(width, device="cuda")
    rows = torch.tensor([5, 0, 3], dtype=torch.int32, device="cuda")
    for picked, count in ((None, n), (rows, 3)):
        outs = [torch.empty(count, width, device="cuda", dtype=dtype) for _ in range(2)]
        for which, out in zip((ops, twin), outs):
            which.streams_read(x, read, weight, 1e-5, out, rows=picked)
        close(outs[0], outs[1], dtype, "read")
    y = (2 * torch.randn(n, width, device="cuda")).to(dtype)
    for following in (False, True):
        kept = [x.clone() for _ in range(2)]
        normed = [torch.zeros(n, width, device="cuda", dtype=dtype) for _ in range(2)]
        for which, s, nm in zip((ops, twin), kept, normed):
            which.streams_update(s, y, mix, write, read if following else None, weight if following else None, 3e-6, nm if following else None)
        close(kept[0], kept[1], torch.float32, "update")
        close(normed[0], normed[1], dtype, "the next read")
    # a matrix that is not symmetric: stream t is the sum over s of mix[s, t] x_s
    if streams > 1:
        one_way = torch.zeros(streams, streams, device="cuda")
        one_way[0, 1] = 1.0
        moved = x.clone()
        ops.streams_update(moved, torch.zeros_like(y), one_way, torch.zeros(streams, device="cuda"))
        assert torch.equal(moved[1], x[0]) and float(moved[0].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,vdim,cap", [(3, 24, 40, 4.0), (2, 64, 64, 15.0), (5, 7, 100, 1.0), (1, 130, 9, 30.0), (2, 300, 65, 8.0),
                                                (4, 128, 128, 15.0), (2, 48, 63, 15.0)])
@pytest.mark.parametrize("chunked", [False, True])
def test_matrix_memory_over_steps_and_slots(ops, dtype, heads, dim, vdim, cap, chunked):
    """Rows of unequal portions, an empty row, single tokens, portions longer than the kernel's chunks; a request that
    starts again in a used slot starts from zeros (matrix, normaliser and maximum).  ``chunked``: every step in the
    chunked form (chunks of one token up to whole ones, rows of several chunks)."""
    print(f"matrix_memory {dtype} {heads} {dim} {vdim} {cap} chunked={chunked}", flush=True)
    twin = TorchOps()
    size = heads * dim * vdim + heads * dim + heads
    states = [torch.randn(4, size + 3, device="cuda") for _ in range(2)]
    states[1].copy_(states[0])
    slots = torch.tensor([2, 0, 3], dtype=torch.int32, device="cuda")
    firsts = [0, 0, 0]
    for step, lengths in enumerate(([5, 1, 37], [1, 1, 1], [18, 0, 2], [1, 1, 1], [2, 140, 1], [64, 65, 128], [200, 0, 3])):
        if step == 3:
            firsts[1] = 0                          # the second request ends; another one starts in its slot
        token_row, positions, row_start, row_len, row_ctx = batch(lengths, firsts, "cuda")
        n = sum(lengths)
        proj = (0.5 * torch.randn(n, 2 * heads * dim + heads * vdim + 3, device="cuda")).to(dtype)
        q, k, v = proj[:, :heads * dim], proj[:, heads * dim:2 * heads * dim], proj[:, 2 * heads * dim:2 * heads * dim + heads * vdim]
        gates = 3 * cap * torch.randn(n, 2 * heads, device="cuda")
        gates[:, heads:] += cap                                            # (forget gates mostly open)
        outs = [torch.zeros(n, heads * vdim, device="cuda") for _ in range(2)]
        belows = [torch.zeros(n, heads, 2, device="cuda") for _ in range(2)]
        coefs = [torch.zeros(n, heads, 2, device="cuda") for _ in range(2)]
        scratch = {}
        if chunked:
            # (filled with what is no number: nothing may be read that has not been written)
            scratch = {"run": torch.full((n, heads), float("nan"), device="cuda", dtype=torch.float64),
                       "sums": torch.full((n // 64 + len(lengths), heads, dim, vdim + 1), float("nan"), device="cuda")}
        for which, state, out, below, coef in zip((ops, twin), states, outs, belows, coefs):
            which.matrix_memory(q, k, v, gates, cap, dim ** -0.5, state, slots, row_start, row_len, row_ctx, out, below, coef, heads, dim, vdim,
                                **(scratch if which is ops else {}))
        close(coefs[0], coefs[1], torch.float32, f"coefficients, step {step}")
        close(outs[0], outs[1], torch.float32, f"read-out, step {step}")
        close(belows[0], belows[1], torch.float32, f"below, step {step}")
        close(states[0], states[1], torch.float32, f"state, step {step}")
        assert torch.equal(states[0][1], states[1][1]) and torch.equal(states[0][:, size:], states[1][:, size:])
        # the division, the heads' norm and the sigmoid gate behind it
        gate = torch.randn(n, heads * vdim, device="cuda").to(dtype)
        weight = 1 + 0.3 * torch.randn(heads * vdim, device="cuda")
        gated = [torch.empty(n, heads * vdim, device="cuda", dtype=dtype) for _ in range(2)]
        for which, out in zip((ops, twin), gated):
            which.heads_norm_gate(outs[1], weight, True, 1e-5, gate, out, heads, vdim, gate_activation="sigmoid", below=belows[1], floor=1e-6)
        close(gated[0], gated[1], dtype, "normalised, gated read-out")
        firsts = [f + n for f, n in zip(firsts, lengths)]


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_memory_does_not_depend_on_how_its_tokens_are_cut(ops, dtype):
    """The same bits, state and read-out, whether 150 tokens come at once, in portions or one by one."""
    heads, dim, vdim, n = 2, 48, 32, 150
    proj = torch.randn(n, 2 * heads * dim + heads * vdim, device="cuda").to(dtype)
    q, k, v = proj[:, :heads * dim], proj[:, heads * dim:2 * heads * dim], proj[:, 2 * heads * dim:]
    gates = 4 * torch.randn(n, 2 * heads, device="cuda")
    make = lambda a: torch.tensor(a, dtype=torch.int32, device="cuda")
    results = []
    for cuts in ([150], [7, 16, 1, 64, 62], [1] * 150):
        state = torch.randn(1, heads * dim * vdim + heads * dim + heads, device="cuda")       # (leftovers of whoever held the slot)
        out, below, coef = torch.zeros(n, heads * vdim, device="cuda"), torch.zeros(n, heads, 2, device="cuda"), torch.zeros(n, heads, 2, device="cuda")
        at = 0
        for count in cuts:
            piece = slice(at, at + count)
            ops.matrix_memory(q[piece], k[piece], v[piece], gates[piece].contiguous(), 6.0, 0.2, state, make([0]), make([0]), make([count]),
                              make([at + count]), out[piece], below[piece], coef[piece], heads, dim, vdim)
            at += count
        results.append((out, below, state))
    for out, below, state in results[1:]:
        assert torch.equal(out, results[0][0]) and torch.equal(below, results[0][1]) and torch.equal(state, results[0][2])


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_memory_in_chunks_equals_the_memory_token_by_token(ops, dtype):
    """A prompt of 700 tokens beside two short rows, at the sizes of a real model's heads and from a state that is there:
    the chunked form against the scan, read-outs, normalisers and states; then the step's shape decides by itself."""
    heads, dim, vdim = 3, 128, 192
    lengths, firsts = [700, 1, 90], [40, 7, 0]
    n = sum(lengths)
    _, _, row_start, row_len, row_ctx = batch(lengths, firsts, "cuda")
    slots = torch.tensor([1, 2, 0], dtype=torch.int32, device="cuda")
    proj = (0.5 * torch.randn(n, 2 * heads * dim + heads * vdim, device="cuda")).to(dtype)
    q, k, v = proj[:, :heads * dim], proj[:, heads * dim:2 * heads * dim], proj[:, 2 * heads * dim:]
    gates = 5 * torch.randn(n, 2 * heads, device="cuda")
    gates[:, heads:] += 6.0
    size = heads * dim * vdim + heads * dim + heads
    start = torch.randn(3, size, device="cuda")
    start[:, -heads:] = 0.5
    results = []
    for chunked in (False, True):
        state = start.clone()
        out, below, coef = torch.zeros(n, heads * vdim, device="cuda"), torch.zeros(n, heads, 2, device="cuda"), torch.zeros(n, heads, 2, device="cuda")
        scratch = {}
        if chunked:
            chunks = ops.matrix_memory_chunks(n, len(lengths))
            assert chunks >= sum(-(-length // 64) for length in lengths)
            scratch = {"run": torch.empty(n, heads, device="cuda", dtype=torch.float64), "sums": torch.empty(chunks, heads, dim, vdim + 1, device="cuda")}
        ops.matrix_memory(q, k, v, gates, 15.0, dim ** -0.5, state, slots, row_start, row_len, row_ctx, out, below, coef, heads, dim, vdim, **scratch)
        results.append((out, below, state, coef))
    assert torch.equal(results[0][3], results[1][3]) and torch.equal(results[0][1][..., 1], results[1][1][..., 1])     # the gates' walk is one
    for index, what in enumerate(("read-out", "below", "state")):
        close(results[1][index], results[0][index], torch.float32, what)
    assert ops.matrix_memory_chunks(3, 3) == 0 and ops.matrix_memory_chunks(40, 3) == 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_plain_activations_and_a_gate_per_channel(ops, dtype):
    twin = TorchOps()
    x = (3 * torch.randn(13, 301, device="cuda")).to(dtype)
    for activation in ("relu2", "gelu_tanh", "silu"):
        a, b = x.clone(), x.clone()
        ops.activation_(a, activation)
        twin.activation_(b, activation)
        close(a, b, dtype, activation)
    assert float(ops_relu2(ops, torch.tensor([[-2.0, 3.0]], device="cuda"))[0, 0]) == 0.0
    assert float(ops_relu2(ops, torch.tensor([[-2.0, 3.0]], device="cuda"))[0, 1]) == 9.0
    heads, n, v = 5, 9, 24
    y = torch.randn(heads, n, v, device="cuda").to(dtype)
    proj = torch.randn(n, 7 + heads * v, device="cuda").to(dtype)
    outs = [torch.empty(n, heads * v, device="cuda", dtype=dtype) for _ in range(2)]
    for which, out in zip((ops, twin), outs):
        which.gate_heads(y, proj, 7, out, per_channel=True)
    close(outs[0], outs[1], dtype, "a gate per channel")


def ops_relu2(ops, x):
    ops.activation_(x, "relu2")
    return x


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_q,n_kv,dim,pairs", [(6, 2, 24, 5), (8, 2, 64, 32), (3, 3, 10, 0), (4, 1, 48, 12)])
def test_queries_and_keys_turned_in_halves_and_values_left_as_projected(ops, dtype, n_q, n_kv, dim, pairs):
    print(f"qkv_prepare in halves {dtype} {n_q} {n_kv} {dim} {pairs}", flush=True)
    twin = TorchOps()
    page, row = 8, -(-dim // 16) * 16
    lengths, firsts = [21, 1, 1, 6], [0, 77, 9, 60]
    token_row, positions, row_start, row_len, row_ctx = batch(lengths, firsts, "cuda")
    n = sum(lengths)
    pages_per_row = -(-max(row_ctx.tolist()) // page)
    order = np.random.default_rng(3).permutation(len(lengths) * pages_per_row)
    table = torch.tensor(order.reshape(len(lengths), pages_per_row), dtype=torch.int32, device="cuda")
    qkv = torch.randn(n, (n_q + 2 * n_kv) * dim, device="cuda").to(dtype)
    angles = positions.float()[:, None] * (100.0 ** (-torch.arange(pairs, device="cuda").float() / max(pairs, 1)))[None, :]
    cos_sin = torch.cat([angles.cos(), angles.sin()], dim=1).contiguous() if pairs else None
    results = []
    for which in (ops, twin):
        keys = torch.zeros(len(order), n_kv, page, row, device="cuda", dtype=dtype)
        values = torch.zeros(len(order), n_kv, row, page, device="cuda", dtype=dtype)
        q = torch.zeros(n, n_q * row, device="cuda", dtype=dtype)
        which.qkv_prepare(qkv, keys, values, table, token_row, positions, None, None, 0.0, cos_sin, page, n_q, n_kv, dim, dim, q, True,
                          pairing="halves")
        results.append((q, keys, values))
    for got, want, what in zip(results[0], results[1], ("queries", "keys", "values")):
        close(got, want, dtype, what)
    # the first token of the first row by hand: dimension i turns with dimension i + pairs; the values are the projection itself
    q = results[0][0].float().view(n, n_q, row)
    t = 5
    src = qkv[t].float().view(n_q + 2 * n_kv, dim)
    if pairs:
        c, s = cos_sin[t, :pairs], cos_sin[t, pairs:]
        want = torch.cat([src[0, :pairs] * c - src[0, pairs:2 * pairs] * s, src[0, pairs:2 * pairs] * c + src[0, :pairs] * s, src[0, 2 * pairs:]])
    else:
        want = src[0]
    close(q[t, 0, :dim], want, dtype, "a query by hand")
    slot = int(table[0, t // page])
    close(results[0][2][slot, 0, :dim, t % page], src[n_q + n_kv], dtype, "a value by hand")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [1, 5, 16, 40, 300])
def test_a_product_with_its_activation_in_the_epilogue(ops, dtype, rows):
    """Few rows: the few-row kernel applies the activation to its 32-bit sums; many rows: the library's product and the
    activation kernel behind it."""
    twin = TorchOps()
    x = torch.randn(rows, 136, device="cuda").to(dtype)
    weight = (0.2 * torch.randn(203, 136, device="cuda")).to(dtype)
    for activation in ("relu2", "gelu_tanh", "silu"):
        close(ops.linear_activated(x, weight, activation), twin.linear_activated(x, weight, activation), dtype, f"{activation} {rows}")
