"""A mixer that carries a matrix per head from token to token and corrects it by the delta rule: what the state
already returns for a key is taken off the value before the key and the value are written.

Per head, with a decay ``g_t`` (one number, or one per key channel acting on the state's rows), a write strength
``beta_t`` in (0, 1), unit vectors ``q_t`` (times ``dim^-1/2``) and ``k_t``::

    S <- g_t * S;   u = beta_t * (v_t - S^T k_t);   S <- S + k_t u^T;   o_t = S^T q_t

so the read-out sees the token's own write.  ``q``, ``k`` and ``v`` each pass a short causal convolution over time per
channel and silu before they are used; ``q`` and ``k`` have ``kv_heads`` heads that groups of the ``heads`` value heads
share.  The decay is ``exp(-exp(A_log) * softplus(z + dt_bias))`` with ``z`` a projection of the mixer's input (per head)
or a low-rank map of it (per head and key channel).  Each head's ``o`` is divided by its root mean square, multiplied
by a weight shared by the heads and by a gate (``silu`` of a projection, or ``sigmoid`` of a low-rank map), then the
output projection.

What a request keeps: the matrices in float32 (per head blocks of 16 value columns, ``[heads, vdim / 16, dim, 16]``, so
that a workgroup's share is one contiguous piece) and, behind them, the last ``taps - 1`` inputs
of the three convolutions, oldest first; zeros before a sequence's first token.  Everything behind the projections
and convolutions (unit norms, softplus, exponentials, sigmoid of the write strength, state, read-out, per-head norm) is
32-bit.
"""
from __future__ import annotations

import dataclasses
from typing import Optional

import torch

from .base import VECTOR, Mixer, ParamSpec, StateSpec
from .linear import Linear

UNIT_EPS = 1e-6         # q / sqrt(sum(q^2) + UNIT_EPS)
STATE_COLUMNS = 16      # a head's matrix is kept as blocks of this many value columns, [vdim / 16][dim][16], the last one filled up


def matrix_floats(heads: int, dim: int, value_dim: int) -> int:
    """The size of a request's matrices as the kernels keep them."""
    return heads * dim * (-(-value_dim // STATE_COLUMNS) * STATE_COLUMNS)


@dataclasses.dataclass(frozen=True)
class GatedDeltaNames:
    q: str = "q"
    k: str = "k"
    v: str = "v"
    conv_suffix: str = ".conv"
    strength: str = "b"
    decay: str = "a"                # per head: the projection; per channel: the two maps ``<decay>1``, ``<decay>2``
    decay_scale: str = "A_log"
    decay_bias: str = "dt_bias"
    gate: str = "g"                 # silu gate: the projection; low-rank sigmoid gate: ``<gate>1``, ``<gate>2``
    norm: str = "norm"
    out: str = "o"


class GatedDeltaRule(Mixer):
    """``decay_per_channel``: one decay per head and key channel through a low-rank map (inner size ``low``), otherwise
    one per head.  ``low_rank_gate``: the output gate is ``sigmoid(W_g2 (W_g1 h))`` (inner size ``gate_low``), otherwise
    ``silu(W_g h)``.  Inner sizes left None are read off the checkpoint's tensors."""
    graph_safe = True

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, value_dim: int, taps: int, norm_eps: float,
                 decay_per_channel: bool = False, low_rank_gate: bool = False, low: Optional[int] = None,
                 gate_low: Optional[int] = None, default_low: int = 16, names: GatedDeltaNames = GatedDeltaNames()):
        if heads % kv_heads:
            raise ValueError(f"{heads} value heads are no multiple of {kv_heads} key heads")
        if taps < 1:
            raise ValueError(f"a convolution needs at least one tap, got {taps}")
        self.width, self.heads, self.kv_heads, self.dim, self.value_dim, self.taps = width, heads, kv_heads, dim, value_dim, int(taps)
        self.norm_eps, self.names = float(norm_eps), names
        self.decay_per_channel, self.low_rank_gate = bool(decay_per_channel), bool(low_rank_gate)
        self.low, self.low_is_free = (low, False) if low is not None else (default_low, True)
        self.gate_low, self.gate_low_is_free = (gate_low, False) if gate_low is not None else (default_low, True)
        self.q_scale = float(dim) ** -0.5
        self.keys, self.values = kv_heads * dim, heads * value_dim
        self.channels = 2 * self.keys + self.values             # what the convolutions run over: q | k | v
        self.matrix_size = matrix_floats(heads, dim, value_dim)
        n = names
        # Everything that reads the mixer's input is one product: q | k | v | write strength | decay (or its inner
        # rows) | gate (or its inner rows).
        self.decay_in = n.decay + "1" if self.decay_per_channel else n.decay
        self.gate_in = n.gate + "1" if self.low_rank_gate else n.gate
        self._pieces = (n.q, n.k, n.v, n.strength, self.decay_in, self.gate_in)
        self.proj = Linear(width, self._pieces, self._piece_sizes(), bare_names=True)
        self.decay_up = Linear(self.low, (n.decay + "2",), (heads * dim,), out_float32=True, bare_names=True) if self.decay_per_channel else None
        self.gate_up = Linear(self.gate_low, (n.gate + "2",), (self.values,), bare_names=True) if self.low_rank_gate else None
        self.o = Linear(self.values, (n.out,), (width,), bare_names=True)
        self._taps = {}
        self.conv_weight = None         # float32 [channels, taps]
        self.norm_weight = self.decay_scale = self.decay_bias = None

    def _piece_sizes(self):
        return (self.keys, self.keys, self.values, self.heads, self.low if self.decay_per_channel else self.heads,
                self.gate_low if self.low_rank_gate else self.values)

    def cache_spec(self):
        # (a multiple of four numbers, so that every slot's matrices start at a multiple of 16 bytes)
        return StateSpec((-(-(self.matrix_size + (self.taps - 1) * self.channels) // 4) * 4,), "float32")

    def param_specs(self):
        n = self.names
        specs = {**self.proj.param_specs(), **self.o.param_specs()}
        for part in (self.decay_up, self.gate_up):
            if part is not None:
                specs.update(part.param_specs())
        if self.decay_per_channel and self.low_is_free:
            specs[self.decay_in] = dataclasses.replace(specs[self.decay_in], free_dims=(0,))
            specs[n.decay + "2"] = dataclasses.replace(specs[n.decay + "2"], free_dims=(1,))
        if self.low_rank_gate and self.gate_low_is_free:
            specs[self.gate_in] = dataclasses.replace(specs[self.gate_in], free_dims=(0,))
            specs[n.gate + "2"] = dataclasses.replace(specs[n.gate + "2"], free_dims=(1,))
        for name, size in ((n.q, self.keys), (n.k, self.keys), (n.v, self.values)):
            specs[name + n.conv_suffix] = ParamSpec((size, self.taps), VECTOR, "normal")
        specs[n.norm] = ParamSpec((self.value_dim,), VECTOR, "norm")
        specs[n.decay_scale] = ParamSpec((self.heads,), VECTOR, "bias")
        specs[n.decay_bias] = ParamSpec((self.heads * self.dim if self.decay_per_channel else self.heads,), VECTOR, "bias")
        return specs

    def assign(self, name, tensor):
        n = self.names
        if name.endswith(n.conv_suffix) and name[:-len(n.conv_suffix)] in (n.q, n.k, n.v):
            self._taps[name[:-len(n.conv_suffix)]] = tensor
        elif name == n.norm:
            self.norm_weight = tensor
        elif name == n.decay_scale:
            self.decay_scale = tensor
        elif name == n.decay_bias:
            self.decay_bias = tensor
        elif self.decay_up is not None and self.decay_up.owns(name):
            self.decay_up.assign(name, tensor)
        elif self.gate_up is not None and self.gate_up.owns(name):
            self.gate_up.assign(name, tensor)
        elif self.o.owns(name):
            self.o.assign(name, tensor)
        elif name in self._pieces:
            if self.decay_per_channel and name == self.decay_in:        # (where the size was free, the checkpoint says it)
                self.low = int(tensor.shape[0])
            if self.low_rank_gate and name == self.gate_in:
                self.gate_low = int(tensor.shape[0])
            self.proj.piece_out = self._piece_sizes()
            self.proj.out_features = sum(self.proj.piece_out)
            self.proj.assign(name, tensor)
        else:
            raise KeyError(name)

    def finalize(self):
        n = self.names
        self.conv_weight = torch.cat([self._taps[name] for name in (n.q, n.k, n.v)], dim=0).contiguous()
        self._taps.clear()
        for part, inner in ((self.decay_up, self.low), (self.gate_up, self.gate_low)):
            if part is not None:
                part.in_features = inner
                part.finalize()
                if part.weight.shape[1] != inner:
                    raise ValueError(f"the two matrices of a low-rank map disagree about their inner size: {inner} and {part.weight.shape[1]}")
        self.proj.finalize()
        self.o.finalize()

    def mixing_flops(self, new_tokens: int, context: int) -> float:
        """Per token, head and state element: the decay, what the state returns for the key, the write and the read-out."""
        return 7.0 * new_tokens * self.heads * self.dim * self.value_dim

    def forward(self, x, ctx, cache):
        ops = ctx.ops
        n = x.shape[0]
        proj = self.proj.forward(x, ctx)
        at = self.channels
        strength = proj[:, at:at + self.heads]
        at += self.heads
        decay_width = self.low if self.decay_per_channel else self.heads
        decay = proj[:, at:at + decay_width]
        gate = proj[:, at + decay_width:]
        if self.decay_per_channel:
            decay = self.decay_up.forward(decay.contiguous(), ctx)                  # float32 [T, heads * dim]
        if self.low_rank_gate:
            gate = self.gate_up.forward(gate.contiguous(), ctx)
        single = ctx.n_tokens == ctx.n_rows         # one token a row: the workgroup that reads a row's last inputs also moves them on
        prepared = ctx.empty((n, self.channels), dtype=torch.float32)
        strengths = ctx.empty((n, self.heads), dtype=torch.float32)
        decays = ctx.empty((n, self.heads * self.dim if self.decay_per_channel else self.heads), dtype=torch.float32)
        ops.delta_prepare(proj, self.conv_weight, cache.state, self.matrix_size, ctx.state_slots, ctx.token_row, ctx.positions,
                          ctx.row_start, prepared, self.kv_heads, self.heads, self.dim, self.value_dim, self.q_scale, UNIT_EPS,
                          strength, decay, self.decay_scale, self.decay_bias, self.decay_per_channel, strengths, decays, keep=single)
        if not single and self.taps > 1:
            ops.delta_conv_keep(proj, self.channels, self.taps, cache.state, self.matrix_size, ctx.state_slots, ctx.row_start,
                                ctx.row_len, ctx.row_ctx)
        mixed = ctx.empty((n, self.values), dtype=torch.float32)
        ops.delta_rule(prepared, strengths, decays, self.decay_per_channel, cache.state, 0, ctx.state_slots, ctx.row_start, ctx.row_len,
                       ctx.row_ctx, mixed, self.heads, self.kv_heads, self.dim, self.value_dim)
        gated = ctx.empty((n, self.values))
        ops.heads_norm_gate(mixed, self.norm_weight, False, self.norm_eps, gate, gated, self.heads, self.value_dim,
                            gate_activation="sigmoid" if self.low_rank_gate else "silu")
        return self.o.forward(gated, ctx)
