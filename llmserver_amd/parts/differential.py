"""Differential attention over the paged cache: every head forms two softmax maps over the same values and returns their
weighted difference.

Per head ``q = [q1, q2]`` and per key/value head ``k = [k1, k2]`` (``dim`` numbers each) and ``v`` (``vdim``); map ``m`` is
``softmax(q_m . k_m * scale)`` over the keys the head sees (causal, possibly the last ``window`` only), ``a_m`` its
weighted sum of values; with one number ``lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff`` for the layer the head returns
``(a1 - lambda a2) / rms(a1 - lambda a2) * (1 - diff)``; the heads side by side go through the output projection.

The paged attention kernels see each map as a head of its own: ``2 * kv_heads`` key heads ``(g, m)`` and ``2 * heads`` query
heads, the queries of key head ``(g, m)`` lying side by side (the query matrix's rows are put in that order once, when
the tensors have been loaded, so the product leaves them so).  Both maps of a key/value head read the same value rows:
the pages hold them under either key head.  A kernel behind attention forms the difference and the norm.

A layer may have no keys and values of its own and read the pages that another layer of equal heads writes
(``shares_cache``); the pages then outlive the longer of the windows of all that read them (``cache_window``).
"""
from __future__ import annotations

import dataclasses
import math
from typing import Optional

import torch

from .attention import SHORT_CONTEXT, stage_attention_plan
from .base import VECTOR, Mixer, PagedKVSpec, ParamSpec
from .linear import Linear


@dataclasses.dataclass(frozen=True)
class DifferentialNames:
    q: str = "q"
    k: str = "k"
    v: str = "v"
    out: str = "o"
    lambdas: tuple = ("lq1", "lk1", "lq2", "lk2")


class DifferentialAttention(Mixer):
    graph_safe = True
    MAPS = 2

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, value_dim: int, scale: float, diff: float, norm_eps: float,
                 window: Optional[int] = None, shares_cache: bool = False, cache_window="own", names: DifferentialNames = DifferentialNames()):
        """``shares_cache``: no key and value projections; the layer reads the pages of the call whose cache it is given.
        ``cache_window``: how long the pages are kept (None: for ever), if that is not this layer's own window."""
        if heads % kv_heads:
            raise ValueError(f"{heads} query heads are no multiple of {kv_heads} key/value heads")
        self.width, self.heads, self.kv_heads, self.dim, self.value_dim = width, heads, kv_heads, dim, value_dim
        self.group_size = heads // kv_heads
        self.scale, self.diff, self.norm_eps = float(scale), float(diff), float(norm_eps)
        self.window = window
        self.cache_window = window if cache_window == "own" else cache_window
        self.shares_cache = bool(shares_cache)
        self.names = names
        self.row = -(-max(dim, value_dim) // 16) * 16            # a head as the attention kernels and the pages see it
        q_rows, k_rows, v_rows = heads * self.MAPS * dim, kv_heads * self.MAPS * dim, kv_heads * value_dim
        if shares_cache:
            self.qkv = Linear(width, (names.q,), (q_rows,), bare_names=True)
        else:
            self.qkv = Linear(width, (names.q, names.k, names.v), (q_rows, k_rows, v_rows), bare_names=True)
        self.o = Linear(heads * value_dim, (names.out,), (width,), bare_names=True)
        self._lambdas = {}
        self.lam = None             # the layer's lambda, a number

    @property
    def n_q(self):
        return self.MAPS * self.heads

    @property
    def n_kv(self):
        return self.MAPS * self.kv_heads

    def cache_spec(self):
        return PagedKVSpec(self.n_kv, self.row, self.cache_window)

    def param_specs(self):
        specs = {**self.qkv.param_specs(), **self.o.param_specs()}
        for name in self.names.lambdas:
            specs[name] = ParamSpec((self.dim,), VECTOR, "bias")
        return specs

    def assign(self, name, tensor):
        if name in self.names.lambdas:
            self._lambdas[name] = tensor
        elif self.o.owns(name):
            self.o.assign(name, tensor)
        elif self.qkv.owns(name):
            self.qkv.assign(name, tensor)
        else:
            raise KeyError(name)

    def finalize(self):
        self.qkv.finalize()
        self.o.finalize()
        lq1, lk1, lq2, lk2 = (self._lambdas[name].float() for name in self.names.lambdas)
        self.lam = math.exp(float((lq1 * lk1).sum())) - math.exp(float((lq2 * lk2).sum())) + self.diff
        self._lambdas.clear()
        # The query rows in the order the attention kernels group them: key head (g, m) is followed by the queries
        # (g * group + r, m) of its group, r = 0 ..; the checkpoint has them head by head, [map 1, map 2].
        order = torch.arange(self.heads * self.MAPS * self.dim, device=self.qkv.weight.device)
        order = order.view(self.kv_heads, self.group_size, self.MAPS, self.dim).permute(0, 2, 1, 3).reshape(-1)
        weight = self.qkv.weight
        q_rows = order.numel()
        self.qkv.weight = torch.cat([weight[:q_rows][order], weight[q_rows:]], dim=0).contiguous()

    def plan_key(self):
        return ("paged_attention", self.group_size, self.n_kv, self.window, self.row)

    def graph_shape(self, rows: int, longest_context: int):
        return "short contexts" if longest_context <= SHORT_CONTEXT else None

    def graph_shape_edges(self):
        return (SHORT_CONTEXT,)

    def mixing_flops(self, new_tokens: int, context: int) -> float:
        first = context - new_tokens
        if self.window is None:
            pairs = new_tokens * first + new_tokens * (new_tokens + 1) // 2
        else:
            pairs = sum(min(position + 1, self.window) for position in range(first, context))
        return 2.0 * self.n_q * (self.dim + self.value_dim) * pairs

    def prepare(self, ctx):
        stage_attention_plan(ctx, self.plan_key(), self.group_size, self.n_kv, self.row, self.window, self.graph_shape)

    def forward(self, x, ctx, cache):
        qkv = self.qkv.forward(x, ctx)
        table = ctx.block_table(cache.group)
        n = qkv.shape[0]
        if self.shares_cache == cache.writable:
            raise ValueError("a layer with keys and values of its own writes its pages; one without reads another's")
        q = ctx.empty((n, self.n_q * self.row))
        # (each key head's values are those of its key/value head: the two maps share them)
        ctx.ops.qkv_prepare(qkv, cache.keys, cache.values, table, ctx.token_row, ctx.positions, None, None, 0.0, None, cache.page_size,
                            self.n_q, self.n_kv, self.dim, self.value_dim, q, cache.writable, value_share=self.MAPS)
        attended = ctx.empty((n, self.n_q * self.row))
        ctx.ops.paged_attention(q, attended, cache.keys, cache.values, table, ctx.row_start, ctx.row_len, ctx.row_ctx,
                                ctx.get_plan(self.plan_key()), self.scale, self.window, cache.page_size, self.n_q, self.n_kv, self.row, ctx)
        out = ctx.empty((n, self.heads * self.value_dim))
        ctx.ops.differential_heads(attended, self.lam, 1.0 - self.diff, self.norm_eps, out, self.kv_heads, self.group_size, self.value_dim, self.row)
        return self.o.forward(out, ctx)
