"""Mixers that carry a matrix per head from token to token instead of a cache that grows: a linear recurrence
``S_t = diag(d_t) S_(t-1) + k_t v_t^T`` with a decay per key channel, read out by a query.

Two readings of the state are built on one kernel (``ops.linear_recurrence``):

* ``bonus`` None: ``o_t = S_t^T q_t`` (the token's own key and value are in the state it reads);
* ``bonus [heads, dim]``: ``o_t = (S_(t-1) + diag(bonus) k_t v_t^T)^T q_t``, then the state moves on (the token itself
  enters the output through the bonus only).

A third reading, on a kernel of its own (``ops.matrix_memory``), is the matrix memory with exponential gates
(:class:`MatrixMemory`): one input and one forget gate a head, kept in range by a running maximum of their logarithms,
and a normaliser vector beside the matrix.

The decay comes from a low-rank map of the mixer's input whose result stays in 32-bit; how it becomes a number in
(0, 1) is the kernel's ``decay`` mode: ``"sigmoid_root"`` (``sigmoid(z)^(1/tau)``) or ``"double_exp"`` (``exp(-exp(z))``).
The state ``[heads, dim, vdim]`` is float32, one slot per live request, zeros before a sequence's first token, and it is
the only thing a request keeps: whatever the length of the context, a step reads and writes the same few numbers.

:class:`TokenShift` is the other piece of state such mixers use: every projection may read its own mix of a token's
row and the row of the token before it.
"""
from __future__ import annotations

import dataclasses
from typing import Optional, Sequence

import torch

from .base import VECTOR, Mixer, ParamSpec, Part, StateSpec
from .linear import Linear

DECAYS = ("sigmoid_root", "double_exp")


class TokenShift(Part):
    """``mix_s = h + (h' - h) * mu_s`` for each of the named mixes ``s``, with ``h'`` the row of the token before in the
    same sequence (zeros before the first).  The last row of a request is a state of ``width`` float32 numbers."""

    def __init__(self, width: int, mixes: Sequence[str], prefix: str = "mu."):
        self.width, self.mixes, self.prefix = width, tuple(mixes), prefix
        self._mu = {}
        self.mu = None          # float32 [mixes, width]

    def param_specs(self):
        return {self.prefix + name: ParamSpec((self.width,), VECTOR, "bias") for name in self.mixes}

    def owns(self, name: str) -> bool:
        return name.startswith(self.prefix) and name[len(self.prefix):] in self.mixes

    def assign(self, name, tensor):
        self._mu[name[len(self.prefix):]] = tensor

    def finalize(self):
        self.mu = torch.stack([self._mu[name] for name in self.mixes]).contiguous()
        self._mu.clear()

    @property
    def state_size(self) -> int:
        return self.width

    def forward(self, h, ctx, state, offset: int):
        """``h [T, W]`` -> ``[mixes, T, W]`` in the compute type; ``state [slots, n]`` holds a request's last row in
        columns ``offset .. offset + W`` and is brought up to date."""
        out = ctx.empty((len(self.mixes), h.shape[0], self.width))
        single = ctx.n_tokens == ctx.n_rows         # one token a row: the workgroup that reads a row's state also moves it on
        ctx.ops.token_shift(h, self.mu, state, offset, ctx.state_slots, ctx.token_row, ctx.positions, ctx.row_start, out, keep=single)
        if not single:
            ctx.ops.token_shift_keep(h, state, offset, ctx.state_slots, ctx.row_start, ctx.row_len)
        return out


@dataclasses.dataclass(frozen=True)
class GatedLinearAttentionNames:
    q: str = "q"
    k: str = "k"
    v: str = "v"
    gate: str = "g"
    out: str = "o"
    norm: str = "norm"
    decay_down: str = "a1"
    decay_up: str = "a2"
    decay_bias: str = "a2.b"


class GatedLinearAttention(Mixer):
    """``q = W_q h * dim^-1/2``, ``k``, ``v``; decay ``sigmoid(W_a2 (W_a1 h) + b)^(1/tau)`` per head and key channel;
    ``S_t = diag(decay_t) S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t``; each head's ``o`` RMS-normed over its value size with
    one weight shared by the heads, times ``silu(W_g h)``, then the output projection.  ``low``: the inner size of the
    decay's map, or None where the checkpoint's tensors say it."""
    graph_safe = True

    def __init__(self, width: int, heads: int, dim: int, value_dim: int, tau: float, norm_eps: float, low: Optional[int] = None,
                 default_low: int = 16, names: GatedLinearAttentionNames = GatedLinearAttentionNames()):
        self.width, self.heads, self.dim, self.value_dim = width, heads, dim, value_dim
        self.tau, self.norm_eps, self.names = float(tau), float(norm_eps), names
        self.low, self.low_is_free = (low, False) if low is not None else (default_low, True)
        self.q_scale = float(dim) ** -0.5
        self.norm_weight = None
        self.decay_bias = None
        self._build()

    def _build(self):
        n = self.names
        keys, values = self.heads * self.dim, self.heads * self.value_dim
        # queries, keys, values, gates and the decay's inner rows read the same input: one product
        self.proj = Linear(self.width, (n.q, n.k, n.v, n.gate, n.decay_down), (keys, keys, values, values, self.low), bare_names=True)
        self.decay_up = Linear(self.low, (n.decay_up,), (keys,), out_float32=True, bare_names=True)
        self.o = Linear(values, (n.out,), (self.width,), bare_names=True)

    def cache_spec(self):
        return StateSpec((self.heads * self.dim * self.value_dim,), "float32")

    def param_specs(self):
        specs = {**self.proj.param_specs(), **self.decay_up.param_specs(), **self.o.param_specs()}
        if self.low_is_free:
            specs[self.names.decay_down] = dataclasses.replace(specs[self.names.decay_down], free_dims=(0,))
            specs[self.names.decay_up] = dataclasses.replace(specs[self.names.decay_up], free_dims=(1,))
        specs[self.names.norm] = ParamSpec((self.value_dim,), VECTOR, "norm")
        specs[self.names.decay_bias] = ParamSpec((self.heads * self.dim,), VECTOR, "bias")
        return specs

    def assign(self, name, tensor):
        n = self.names
        if name == n.norm:
            self.norm_weight = tensor
        elif name == n.decay_bias:
            self.decay_bias = tensor
        elif name == n.decay_up:
            self.decay_up.assign(name, tensor)
        elif name == n.out:
            self.o.assign(name, tensor)
        elif name in self.proj.pieces:
            if name == n.decay_down:          # (where the size was free, the checkpoint says it)
                self.low = int(tensor.shape[0])
                self.proj.piece_out = self.proj.piece_out[:-1] + (self.low,)
                self.proj.out_features = sum(self.proj.piece_out)
            self.proj.assign(name, tensor)
        else:
            raise KeyError(name)

    def finalize(self):
        self.decay_up.in_features = self.low
        for part in (self.proj, self.decay_up, self.o):
            part.finalize()
        if self.decay_up.weight.shape[1] != self.low:
            raise ValueError(f"the decay's two matrices disagree about their inner size: {self.low} and {self.decay_up.weight.shape[1]}")

    def mixing_flops(self, new_tokens: int, context: int) -> float:
        """Per token, head and state element: the decay, the outer product's sum and the read-out."""
        return 6.0 * new_tokens * self.heads * self.dim * self.value_dim

    def forward(self, x, ctx, cache):
        ops = ctx.ops
        n = x.shape[0]
        keys, values = self.heads * self.dim, self.heads * self.value_dim
        proj = self.proj.forward(x, ctx)
        q, k = proj[:, :keys], proj[:, keys:2 * keys]
        v, gate = proj[:, 2 * keys:2 * keys + values], proj[:, 2 * keys + values:2 * keys + 2 * values]
        inner = proj[:, 2 * keys + 2 * values:].contiguous()
        decay = self.decay_up.forward(inner, ctx)                                    # float32 [T, heads * dim]
        mixed = ctx.empty((n, values), dtype=torch.float32)
        ops.linear_recurrence(q, k, v, decay, self.decay_bias, "sigmoid_root", self.tau, None, self.q_scale, cache.state, 0,
                              ctx.state_slots, ctx.row_start, ctx.row_len, ctx.row_ctx, mixed, self.heads, self.dim, self.value_dim)
        gated = ctx.empty((n, values))
        ops.heads_norm_gate(mixed, self.norm_weight, False, self.norm_eps, gate, gated, self.heads, self.value_dim)
        return self.o.forward(gated, ctx)


@dataclasses.dataclass(frozen=True)
class TimeMixingNames:
    r: str = "r"
    k: str = "k"
    v: str = "v"
    gate: str = "g"
    out: str = "o"
    norm: str = "norm"
    bonus: str = "u"
    decay_down: str = "w1"
    decay_up: str = "w2"
    decay_bias: str = "w0"
    shift: str = "mu."


class TimeMixing(Mixer):
    """RWKV-style time mixing.  ``r``, ``k``, ``v``, the gate and the decay each read their own mix of a token's row and
    the row before (:class:`TokenShift`); decay ``w = exp(-exp(W_w2 tanh(W_w1 mix_w) + w0))`` per head and key channel;
    ``o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t``, then ``S_t = diag(w_t) S_(t-1) + k_t v_t^T``; each head's ``o`` is
    divided by its root mean square, the heads side by side are multiplied by a weight per channel and by
    ``silu(W_g mix_g)``, then the output projection.  Keys and values have the same size.  State: the matrix per
    head and, behind it, the last row the mixer was given."""
    graph_safe = True
    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, width: int, heads: int, dim: int, norm_eps: float, low: Optional[int] = None, default_low: int = 16,
                 names: TimeMixingNames = TimeMixingNames()):
        self.width, self.heads, self.dim, self.norm_eps, self.names = width, heads, dim, float(norm_eps), names
        self.low, self.low_is_free = (low, False) if low is not None else (default_low, True)
        self.shift = TokenShift(width, self.MIXES, names.shift)
        inner = heads * dim
        self._four = {}
        self.four = None            # [4, heads * dim, width]: r, k, v, gate, one batched product over their four mixes
        self.decay_down = Linear(width, (names.decay_down,), (self.low,), bare_names=True)
        self.decay_up = Linear(self.low, (names.decay_up,), (inner,), out_float32=True, bare_names=True)
        self.o = Linear(inner, (names.out,), (width,), bare_names=True)
        self.norm_weight = self.decay_bias = self.bonus = None
        self.state_matrix = heads * dim * dim

    def cache_spec(self):
        return StateSpec((self.state_matrix + self.shift.state_size,), "float32")

    def param_specs(self):
        n, inner = self.names, self.heads * self.dim
        specs = {name: ParamSpec((inner, self.width)) for name in (n.r, n.k, n.v, n.gate)}
        specs.update({**self.decay_down.param_specs(), **self.decay_up.param_specs(), **self.o.param_specs(), **self.shift.param_specs()})
        if self.low_is_free:
            specs[n.decay_down] = dataclasses.replace(specs[n.decay_down], free_dims=(0,))
            specs[n.decay_up] = dataclasses.replace(specs[n.decay_up], free_dims=(1,))
        specs[n.norm] = ParamSpec((inner,), VECTOR, "norm")
        specs[n.decay_bias] = ParamSpec((inner,), VECTOR, "bias")
        specs[n.bonus] = ParamSpec((self.heads, self.dim), VECTOR, "normal")
        return specs

    def assign(self, name, tensor):
        n = self.names
        if name in (n.r, n.k, n.v, n.gate):
            self._four[name] = tensor
        elif name == n.norm:
            self.norm_weight = tensor
        elif name == n.decay_bias:
            self.decay_bias = tensor
        elif name == n.bonus:
            self.bonus = tensor
        elif name == n.decay_down:
            self.low = int(tensor.shape[0])
            self.decay_down.piece_out, self.decay_down.out_features = (self.low,), self.low
            self.decay_down.assign(name, tensor)
        elif name == n.decay_up:
            self.decay_up.assign(name, tensor)
        elif name == n.out:
            self.o.assign(name, tensor)
        elif self.shift.owns(name):
            self.shift.assign(name, tensor)
        else:
            raise KeyError(name)

    def finalize(self):
        n = self.names
        self.four = torch.stack([self._four[name] for name in (n.r, n.k, n.v, n.gate)]).contiguous()
        self._four.clear()
        self.decay_up.in_features = self.low
        for part in (self.decay_down, self.decay_up, self.o, self.shift):
            part.finalize()
        if self.decay_up.weight.shape[1] != self.low:
            raise ValueError(f"the decay's two matrices disagree about their inner size: {self.low} and {self.decay_up.weight.shape[1]}")

    def mixing_flops(self, new_tokens: int, context: int) -> float:
        return 8.0 * new_tokens * self.heads * self.dim * self.dim

    def forward(self, x, ctx, cache):
        ops = ctx.ops
        n, inner = x.shape[0], self.heads * self.dim
        mixes = self.shift.forward(x, ctx, cache.state, self.state_matrix)          # [5, T, W]: r, k, v, g, w
        four = ops.batched_linear(mixes[:4], self.four)                              # [4, T, heads * dim]
        low = self.decay_down.forward(mixes[4], ctx)
        ops.tanh_(low)
        decay = self.decay_up.forward(low, ctx)                                      # float32 [T, heads * dim]
        mixed = ctx.empty((n, inner), dtype=torch.float32)
        ops.linear_recurrence(four[0], four[1], four[2], decay, self.decay_bias, "double_exp", 1.0, self.bonus, 1.0, cache.state, 0,
                              ctx.state_slots, ctx.row_start, ctx.row_len, ctx.row_ctx, mixed, self.heads, self.dim, self.dim)
        gated = ctx.empty((n, inner))
        ops.heads_norm_gate(mixed, self.norm_weight, True, self.norm_eps, four[3], gated, self.heads, self.dim)
        return self.o.forward(gated, ctx)


@dataclasses.dataclass(frozen=True)
class MatrixMemoryNames:
    q: str = "q"
    k: str = "k"
    v: str = "v"
    gate: str = "g"
    out: str = "o"
    norm: str = "norm"
    input_gate: str = "i"
    forget_gate: str = "f"
    bias_suffix: str = ".b"


class MatrixMemory(Mixer):
    """A matrix-valued memory per head with exponential gates (the mLSTM cell).  Per head, ``q = W_q h * dim^-1/2``, ``k``, ``v``; a log input gate
    ``i = cap * tanh((W_i h + b_i) / cap)`` and a log forget gate ``f = logsigmoid(cap * tanh((W_f h + b_f) / cap))``.
    A stabiliser ``m`` (0 in front of the first token) keeps the exponentials in range: ``m_t = max(f + m_(t-1), i)``, ``a = exp(f + m_(t-1) - m_t)``,
    ``b = exp(i - m_t)``, ``S_t = a S_(t-1) + b k v^T``, ``n_t = a n_(t-1) + b k``,
    ``o = S_t^T q / (max(|n_t . q|, exp(-m_t)) + floor)``.  Each head's ``o`` is divided by its root mean square, the
    heads side by side are multiplied by a weight per channel and by ``sigmoid(W_g h)``, then the output projection.

    The gates' product leaves 32-bit numbers, and everything behind it (caps, logarithms, exponentials, maximum, state,
    normaliser, read-out, norm) is 32-bit.  State per request: the matrices ``[heads, dim, vdim]``, behind them the
    normalisers ``[heads, dim]`` and the maxima ``[heads]``; zeros before a sequence's first token."""
    graph_safe = True

    def __init__(self, width: int, heads: int, dim: int, value_dim: int, gate_cap: float, norm_eps: float, floor: float = 1e-6,
                 names: MatrixMemoryNames = MatrixMemoryNames()):
        self.width, self.heads, self.dim, self.value_dim = width, heads, dim, value_dim
        self.gate_cap, self.norm_eps, self.floor, self.names = float(gate_cap), float(norm_eps), float(floor), names
        self.q_scale = float(dim) ** -0.5
        keys, values = heads * dim, heads * value_dim
        # queries, keys, values and output gates read the same input: one product; the two gates of the recurrence are a
        # product of their own, whose sums stay in 32-bit
        self.proj = Linear(width, (names.q, names.k, names.v, names.gate), (keys, keys, values, values), bare_names=True)
        self.gates = Linear(width, (names.input_gate, names.forget_gate), (heads, heads), bias=True, out_float32=True, bare_names=True,
                            bias_suffix=names.bias_suffix)
        self.o = Linear(values, (names.out,), (width,), bare_names=True)
        self.norm_weight = None
        self.matrix_size, self.normaliser_size = heads * dim * value_dim, heads * dim

    def cache_spec(self):
        return StateSpec((self.matrix_size + self.normaliser_size + self.heads,), "float32")

    def param_specs(self):
        specs = {**self.proj.param_specs(), **self.gates.param_specs(), **self.o.param_specs()}
        specs[self.names.norm] = ParamSpec((self.heads * self.value_dim,), VECTOR, "norm")
        return specs

    def assign(self, name, tensor):
        if name == self.names.norm:
            self.norm_weight = tensor
        elif self.gates.owns(name):
            self.gates.assign(name, tensor)
        elif self.o.owns(name):
            self.o.assign(name, tensor)
        elif self.proj.owns(name):
            self.proj.assign(name, tensor)
        else:
            raise KeyError(name)

    def finalize(self):
        for part in (self.proj, self.gates, self.o):
            part.finalize()

    def mixing_flops(self, new_tokens: int, context: int) -> float:
        """Per token, head and state element: the decay, the outer product's sum and the read-out."""
        return 6.0 * new_tokens * self.heads * self.dim * self.value_dim

    def forward(self, x, ctx, cache):
        ops = ctx.ops
        n = x.shape[0]
        keys, values = self.heads * self.dim, self.heads * self.value_dim
        proj = self.proj.forward(x, ctx)
        q, k = proj[:, :keys], proj[:, keys:2 * keys]
        v, gate = proj[:, 2 * keys:2 * keys + values], proj[:, 2 * keys + values:]
        gates = self.gates.forward(x, ctx)                                           # float32 [T, input gates | forget gates]
        # the memory leaves the read-outs' numerators and, per token and head, what stands below them (n . q and exp(-m));
        # the division is the first thing the kernel of the heads' norm does
        mixed = ctx.empty((n, values), dtype=torch.float32)
        below = ctx.empty((n, self.heads, 2), dtype=torch.float32)
        coefficients = ctx.empty((n, self.heads, 2), dtype=torch.float32)
        # long portions run in chunks, as matrix products; the kernels then want scratch memory of the step's size
        chunks = ops.matrix_memory_chunks(n, ctx.row_len.shape[0])
        scratch = {}
        if chunks:
            scratch = {"run": ctx.empty((n, self.heads), dtype=torch.float64),
                       "sums": ctx.empty((chunks, self.heads, self.dim, self.value_dim + 1), dtype=torch.float32)}
        ops.matrix_memory(q, k, v, gates, self.gate_cap, self.q_scale, cache.state, ctx.state_slots, ctx.row_start, ctx.row_len, ctx.row_ctx,
                          mixed, below, coefficients, self.heads, self.dim, self.value_dim, **scratch)
        gated = ctx.empty((n, values))
        ops.heads_norm_gate(mixed, self.norm_weight, True, self.norm_eps, gate, gated, self.heads, self.value_dim, gate_activation="sigmoid",
                            below=below, floor=self.floor)
        return self.o.forward(gated, ctx)
