"""Causal attention whose keys and values are linear maps of one low-rank latent per token.

Per token: ``c = rmsnorm(W_dkv h)[:rank] * w`` (the latent) and ``r = rotate(W_dkv h)[rank:]`` (a small rotated key
part shared by all heads).  Head ``a`` has the key ``[U_a c, r]`` and the value ``V_a c``; its query is
``[q_a, rotate(p_a)]``.  Since ``q_a . (U_a c) = (U_a^T q_a) . c``, the score is one dot product of
``[U_a^T q_a, rotate(p_a)]`` with the cached row ``[c, r]``, and the weighted sum of values is ``V_a`` applied to the
weighted sum of latents: the cache holds ``rank + rot_dim`` numbers a token, whatever the number of heads, and the
attention kernel sees one key-value head that all query heads share, with the cached row as key and as value.  The
row is padded with zeros to the next head size the attention kernels take.

The softmax's denominator may hold one more term per head (``exp(sink)``, no key, no value), and every head's output
may pass a sigmoid gate computed from the mixer's input: one gate a head, or one for every channel of every head.  A
window bounds the keys a query sees to the last ``window`` positions; pages behind it go back to the pool.
"""
from __future__ import annotations

import dataclasses
from typing import Optional

import torch

from .attention import SHORT_CONTEXT, stage_attention_plan
from .base import VECTOR, Mixer, PagedKVSpec, ParamSpec, PositionEncoding
from .linear import Linear


@dataclasses.dataclass(frozen=True)
class LatentAttentionNames:
    """Checkpoint names of the mixer's tensors (each is the tensor's whole name below the mixer's)."""
    q: str = "q"
    down: str = "dkv"
    down_norm: str = "dkv.norm"
    up_keys: str = "uk"
    up_values: str = "uv"
    out: str = "o"
    sink: Optional[str] = "sink"
    gate: Optional[str] = "g"


def padded_head(size: int, step: int = 16) -> int:
    return -(-size // step) * step


class LatentAttention(Mixer):
    graph_safe = True

    def __init__(self, width: int, n_heads: int, dim: int, rot_dim: int, value_dim: int, rank: int, position: PositionEncoding,
                 scale: float, norm_eps: float, names: LatentAttentionNames = LatentAttentionNames(), window: Optional[int] = None,
                 gate_per_channel: bool = False):
        """``window``: a query sees itself and the ``window - 1`` positions before it (None: all).  ``gate_per_channel``:
        the gate's projection has a row for every channel of every head's values instead of one a head."""
        if getattr(position, "pairing", None) != "neighbours":
            raise ValueError("this mixer's kernels turn neighbouring dimensions together; it takes a PairedRotaryPosition")
        if position.rotary_dim is None or position.rotary_dim > rot_dim or position.rotary_dim % 2:
            raise ValueError(f"the position encoding turns {position.rotary_dim} dimensions, the rotated part has {rot_dim}")
        self.width, self.n_heads, self.dim, self.rot_dim, self.value_dim, self.rank = width, n_heads, dim, rot_dim, value_dim, rank
        self.position, self.scale, self.norm_eps, self.names = position, float(scale), float(norm_eps), names
        self.window = int(window) if window else None
        self.gate_per_channel = bool(gate_per_channel) and names.gate is not None
        self.row = padded_head(rank + rot_dim)       # the cached row, as wide as a head of the attention kernels
        self.q_width = n_heads * (dim + rot_dim)
        pieces, sizes = [names.q, names.down], [self.q_width, rank + rot_dim]
        if names.gate is not None:
            pieces.append(names.gate)
            sizes.append(n_heads * value_dim if self.gate_per_channel else n_heads)
        self.proj = Linear(width, pieces, sizes, bare_names=True)      # queries, latent and shared key part, gates: one product
        self.o = Linear(n_heads * value_dim, (names.out,), (width,), bare_names=True)
        self.down_norm_weight = None
        self.sinks = None
        self._up_keys = self._up_values = None
        self.up_keys = None        # [heads, dim, rank]: q_latent = q @ up_keys[head]
        self.up_values = None      # [heads, rank, value_dim]: out = latent_sum @ up_values[head]

    def cache_spec(self):
        return PagedKVSpec(1, self.row, self.window)

    def param_specs(self):
        specs = {**self.proj.param_specs(), **self.o.param_specs()}
        specs[self.names.down_norm] = ParamSpec((self.rank,), VECTOR, "norm")
        share = 1.0
        specs[self.names.up_keys] = ParamSpec((self.n_heads * self.dim, self.rank), share_per_token=share)
        specs[self.names.up_values] = ParamSpec((self.n_heads * self.value_dim, self.rank), share_per_token=share)
        if self.names.sink is not None:
            specs[self.names.sink] = ParamSpec((self.n_heads,), VECTOR, "normal")
        return specs

    def assign(self, name, tensor):
        if name == self.names.down_norm:
            self.down_norm_weight = tensor
        elif name == self.names.sink:
            self.sinks = tensor
        elif name == self.names.up_keys:
            self._up_keys = tensor
        elif name == self.names.up_values:
            self._up_values = tensor
        elif name == self.names.out:
            self.o.assign(name, tensor)
        elif name in self.proj.pieces:
            self.proj.assign(name, tensor)
        else:
            raise KeyError(name)

    def finalize(self):
        self.proj.finalize()
        self.o.finalize()
        self.up_keys = self._up_keys.view(self.n_heads, self.dim, self.rank).contiguous()
        self.up_values = self._up_values.view(self.n_heads, self.value_dim, self.rank).transpose(1, 2).contiguous()
        self._up_keys = self._up_values = None

    def plan_key(self):
        # (the row's width is part of it: the plan is cut for the kernels of that head size)
        return ("paged_attention", self.n_heads, 1, self.window, self.row)

    def graph_shape(self, rows: int, longest_context: int):
        return "short contexts" if longest_context <= SHORT_CONTEXT else None

    def graph_shape_edges(self):
        return (SHORT_CONTEXT,)

    def mixing_flops(self, new_tokens: int, context: int) -> float:
        """Scores over ``rank + rot_dim`` and weighted latents over ``rank`` dimensions per head, query and visible key."""
        first = context - new_tokens
        if self.window is None:
            pairs = new_tokens * first + new_tokens * (new_tokens + 1) // 2
        else:
            pairs = sum(min(position + 1, self.window) for position in range(first, context))
        return 2.0 * self.n_heads * (2 * self.rank + self.rot_dim) * pairs

    def prepare(self, ctx):
        stage_attention_plan(ctx, self.plan_key(), self.n_heads, 1, self.row, self.window, self.graph_shape)

    def forward(self, x, ctx, cache):
        ops = ctx.ops
        n = x.shape[0]
        proj = self.proj.forward(x, ctx)                                        # [T, q | latent, key part | gates]
        per_head = self.dim + self.rot_dim
        inside = ops.latent_products_inside(n)      # few tokens: the per-head products are made inside the kernels around attention
        q_latent = None
        if not inside:
            q_plain = proj[:, :self.q_width].view(n, self.n_heads, per_head)[:, :, :self.dim].transpose(0, 1)
            q_latent = torch.bmm(q_plain, self.up_keys)                        # [heads, T, rank]
        table = ctx.block_table(cache.group)
        q = ctx.empty((n, self.n_heads * self.row))
        ops.latent_prepare(proj, q_latent, self.down_norm_weight, self.norm_eps, self.position.cos_sin(ctx), cache.keys, cache.values,
                           table, ctx.token_row, ctx.positions, cache.page_size, q, self.n_heads, self.dim, self.rot_dim, self.rank,
                           cache.writable, **({"up_keys": self.up_keys} if inside else {}))
        mixed = ctx.empty((n, self.n_heads * self.row))
        extra = {"sinks": self.sinks} if self.sinks is not None else {}
        ops.paged_attention(q, mixed, cache.keys, cache.values, table, ctx.row_start, ctx.row_len, ctx.row_ctx,
                            ctx.get_plan(self.plan_key()), self.scale, self.window, cache.page_size, self.n_heads, 1, self.row, ctx, **extra)
        gated = ctx.empty((n, self.n_heads * self.value_dim))
        # (without gates the same kernel only brings the heads back beside each other: a gate column of -1 says so)
        gate_column = self.q_width + self.rank + self.rot_dim if self.names.gate is not None else -1
        wide = {"per_channel": True} if self.gate_per_channel else {}
        if inside:
            ops.gate_heads(None, proj, gate_column, gated, mixed=mixed, up_values=self.up_values, **wide)
        else:
            latent = mixed.view(n, self.n_heads, self.row)[:, :, :self.rank].transpose(0, 1)
            ops.gate_heads(torch.bmm(latent, self.up_values), proj, gate_column, gated, **wide)      # [heads, T, value_dim]
        return self.o.forward(gated, ctx)
