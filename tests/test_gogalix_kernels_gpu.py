"""The kernels that Gogalix brought: the joint update of the stream behind two gated sublayers, the difference of two
attention maps, the delta rule's inputs (short convolutions with state, unit vectors, decays, write strengths) and the
delta rule itself, a router with a bias, and key heads that share value heads in front of attention; each against its
plain torch twin, in float32 and in bfloat16, on sizes that are no multiples of anything."""
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
@pytest.mark.parametrize("width", [8, 100, 320, 1027, 2048, 4400])
@pytest.mark.parametrize("second", [None, torch.float32, "same"])
def test_gated_pair_update(ops, dtype, width, second):
    print(f"gated_pair_update {dtype} {width} {second}", flush=True)
    twin = TorchOps()
    n = 5
    x = torch.randn(n, width, device="cuda")
    y1 = torch.randn(n, width, device="cuda").to(dtype)
    y2 = None if second is None else torch.randn(n, width, device="cuda").to(dtype if second == "same" else second)
    gates = (2 * torch.randn(n, width * (1 if y2 is None else 2), device="cuda")).to(dtype)
    s1, s2 = torch.randn(width, device="cuda"), torch.randn(width, device="cuda")
    weight = 1 + 0.2 * torch.randn(width, device="cuda")
    for following in (False, True):
        kept = [x.clone() for _ in range(2)]
        normed = [torch.zeros(n, width, device="cuda", dtype=dtype) for _ in range(2)]
        for which, stream, nm in zip((ops, twin), kept, normed):
            which.gated_pair_update(stream, gates, y1, s1, y2, s2 if y2 is not None else None, weight if following else None, 2e-5,
                                    nm if following else None)
        close(kept[0], kept[1], torch.float32, "stream")
        close(normed[0], normed[1], dtype, "the next norm")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kv_heads,group,vdim,row", [(2, 3, 40, 48), (1, 1, 80, 80), (3, 2, 7, 16), (2, 1, 130, 144)])
def test_differential_heads(ops, dtype, kv_heads, group, vdim, row):
    print(f"differential_heads {dtype} {kv_heads} {group} {vdim} {row}", flush=True)
    twin = TorchOps()
    n = 6
    attended = torch.randn(n, kv_heads * 2 * group * row, device="cuda").to(dtype)
    outs = [torch.empty(n, kv_heads * group * vdim, device="cuda", dtype=dtype) for _ in range(2)]
    for which, out in zip((ops, twin), outs):
        which.differential_heads(attended, 0.37, 0.4, 1e-5, out, kv_heads, group, vdim, row)
    close(outs[0], outs[1], dtype, "heads")


def _delta_step(which, dtype, sizes, taps, proj, extra, weights, state, slots, lengths, firsts, per_channel):
    heads, kv_heads, dim, vdim = sizes
    keys, values = kv_heads * dim, heads * vdim
    channels = 2 * keys + values
    token_row, positions, row_start, row_len, row_ctx = batch(lengths, firsts, "cuda")
    n = proj.shape[0]
    conv, scale, bias = weights
    matrix = heads * dim * (-(-vdim // 16) * 16)
    prepared = torch.empty(n, channels, device="cuda")
    strengths = torch.empty(n, heads, device="cuda")
    decays = torch.empty(n, heads * dim if per_channel else heads, device="cuda")
    strength = proj[:, channels:channels + heads]
    decay = extra if per_channel else proj[:, channels + heads:channels + 2 * heads]
    single = all(length == 1 for length in lengths)
    which.delta_prepare(proj, conv, state, matrix, slots, token_row, positions, row_start, prepared, kv_heads, heads, dim, vdim,
                        dim ** -0.5, 1e-6, strength, decay, scale, bias, per_channel, strengths, decays, keep=single)
    if not single and taps > 1:
        which.delta_conv_keep(proj, channels, taps, state, matrix, slots, row_start, row_len, row_ctx)
    out = torch.empty(n, values, device="cuda")
    which.delta_rule(prepared, strengths, decays, per_channel, state, 0, slots, row_start, row_len, row_ctx, out, heads, kv_heads, dim, vdim)
    return prepared, strengths, decays, out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("per_channel", [False, True])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,taps", [(3, 3, 24, 40, 3), (4, 2, 64, 64, 4), (2, 1, 7, 100, 2), (1, 1, 130, 9, 1),
                                                          (2, 2, 256, 17, 3), (6, 3, 24, 48, 5), (2, 2, 128, 128, 4)])
def test_delta_rule_over_steps_and_slots(ops, dtype, per_channel, heads, kv_heads, dim, vdim, taps):
    """Rows of unequal portions, an empty row, single tokens, portions longer than the kernel's chunks and shorter than
    the convolution's reach; a request that starts again in a used slot starts from zeros."""
    print(f"delta_rule {dtype} {per_channel} {heads} {kv_heads} {dim} {vdim} {taps}", flush=True)
    twin = TorchOps()
    keys, values = kv_heads * dim, heads * vdim
    channels = 2 * keys + values
    size = heads * dim * (-(-vdim // 16) * 16) + (taps - 1) * channels
    states = [torch.randn(4, -(-size // 4) * 4 + 4, device="cuda") for _ in range(2)]        # (slots start at multiples of 16 bytes)
    states[1].copy_(states[0])
    slots = torch.tensor([2, 0, 3], dtype=torch.int32, device="cuda")
    conv = torch.randn(channels, taps, device="cuda") * 0.6
    scale = torch.randn(heads, device="cuda") * 0.5
    bias = torch.randn(heads * dim if per_channel else heads, device="cuda")
    firsts = [0, 0, 0]
    for step, lengths in enumerate(([5, 1, 37], [1, 1, 1], [18, 0, 2], [1, 1, 1], [2, 70, 1], [1, 1, 1], [33, 0, 3])):
        if step == 3:
            firsts[1] = 0                          # the second request ends; another one starts in its slot
        n = sum(lengths)
        proj = torch.randn(n, channels + 2 * heads + 5, device="cuda").to(dtype)
        extra = torch.randn(n, heads * dim, device="cuda") if per_channel else None
        results = [_delta_step(which, dtype, (heads, kv_heads, dim, vdim), taps, proj, extra, (conv, scale, bias), state, slots, lengths,
                               firsts, per_channel) for which, state in ((ops, states[0]), (twin, states[1]))]
        for name, got, want in zip(("prepared", "strengths", "decays", "read-out"), *results):
            close(got, want, torch.float32, f"{name} at step {step}")
        close(states[0][:, :size], states[1][:, :size], torch.float32, f"state behind step {step}")
        assert torch.equal(states[0][:, size:], states[1][:, size:])
        firsts = [first + length for first, length in zip(firsts, lengths)]


def test_a_delta_rule_does_not_depend_on_how_its_tokens_are_cut(ops):
    """State and read-out are the same bits whether a sequence comes whole, in portions or token by token."""
    heads, kv_heads, dim, vdim, taps = 2, 1, 48, 20, 3
    channels = 2 * kv_heads * dim + heads * vdim
    size = heads * dim * (-(-vdim // 16) * 16) + (taps - 1) * channels
    conv, scale, bias = torch.randn(channels, taps, device="cuda") * 0.6, torch.randn(heads, device="cuda") * 0.5, torch.randn(heads, device="cuda")
    total = 45
    proj = torch.randn(total, channels + 2 * heads, device="cuda")
    slots = torch.tensor([1], dtype=torch.int32, device="cuda")
    kept = []
    for cuts in ([total], [7, 1, 16, 17, 2, 2], [1] * total):
        state = torch.randn(2, size, device="cuda")
        outs, first = [], 0
        for length in cuts:
            piece = proj[first:first + length].contiguous()
            outs.append(_delta_step(ops, torch.float32, (heads, kv_heads, dim, vdim), taps, piece, None, (conv, scale, bias), state, slots,
                                    [length], [first], False)[3])
            first += length
        kept.append((torch.cat(outs), state[1].clone()))
    for out, state in kept[1:]:
        assert torch.equal(out, kept[0][0]) and torch.equal(state, kept[0][1])


@pytest.mark.parametrize("experts,top", [(12, 4), (5, 5), (130, 2)])
def test_a_router_with_a_bias(ops, experts, top):
    twin = TorchOps()
    for n in (3, 70):
        x = torch.randn(n, 48, device="cuda")
        router, bias = torch.randn(experts, 48, device="cuda"), 3 * torch.randn(experts, device="cuda")
        results = []
        for which in (ops, twin):
            chosen = torch.empty(n, top, device="cuda", dtype=torch.int32)
            weights = torch.empty(n, top, device="cuda")
            which.route_experts(x, router, top, chosen, weights, bias=bias)
            results.append((chosen, weights))
        assert torch.equal(results[0][0], results[1][0])
        close(results[0][1], results[1][1], torch.float32, "weights")


@pytest.mark.parametrize("dtype", DTYPES)
def test_key_heads_that_share_value_heads(ops, dtype):
    twin = TorchOps()
    n_q, n_kv, dim, vdim, row, page, share = 8, 4, 24, 40, 48, 8, 2
    lengths, firsts = [5, 1], [3, 9]
    token_row, positions, _, _, _ = batch(lengths, firsts, "cuda")
    n = sum(lengths)
    qkv = torch.randn(n, (n_q + n_kv) * dim + (n_kv // share) * vdim, device="cuda").to(dtype)
    table = torch.tensor([[2, 0], [1, 3]], dtype=torch.int32, device="cuda")
    results = []
    for which in (ops, twin):
        keys = torch.zeros(4, n_kv, page, row, device="cuda", dtype=dtype)
        values = torch.zeros(4, n_kv, row, page, device="cuda", dtype=dtype)
        out_q = torch.empty(n, n_q * row, device="cuda", dtype=dtype)
        which.qkv_prepare(qkv, keys, values, table, token_row, positions, None, None, 0.0, None, page, n_q, n_kv, dim, vdim, out_q, True,
                          value_share=share)
        only_q = torch.empty(n, n_q * row, device="cuda", dtype=dtype)
        which.qkv_prepare(qkv[:, :n_q * dim].contiguous(), keys, values, table, token_row, positions, None, None, 0.0, None, page, n_q, n_kv,
                          dim, vdim, only_q, False, value_share=share)
        assert torch.equal(only_q, out_q)
        results.append((keys, values, out_q))
    for got, want in zip(*results):
        assert torch.equal(got, want)
    assert torch.equal(results[0][1][:, 0], results[0][1][:, 1]) and not torch.equal(results[0][1][:, 1], results[0][1][:, 2])
