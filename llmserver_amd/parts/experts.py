"""Routed experts: every token's feed-forward is a weighted sum of ``top`` of ``experts`` small gated feed-forwards.

Router logits ``z = R h`` (plus a bias per expert, where the checkpoint has one) in 32-bit.  ``scoring="softmax"``: the ``top`` largest logits are chosen (the first of equal
ones) and weighted by the softmax over the chosen logits only.  ``scoring="sigmoid"``: scores ``sigmoid(z)``; with
``groups=(count, keep)`` the experts form ``count`` equal groups of neighbours, a group's score is the sum of its two
largest scores, and only experts of the ``keep`` best groups can be chosen; the ``top`` largest scores are chosen and
are the weights as they are.  Expert: ``D (act(G h) * (U h))`` with ``act = silu``, or, with ``activation="clamped"``,
``g = min(G h, limit)``, ``u = clamp(U h, -limit, limit)``, ``D (g * sigmoid(1.702 g) * (u + 1))``; no biases.  The experts' matrices
are stacked (``[experts, 2F, W]`` gate rows then up rows, ``[experts, W, F]``), and the kernels pick each token's from
the list of chosen experts on the device: nothing of the routing is read on the host.
"""
from __future__ import annotations

import torch

from .base import VECTOR, FeedForward, ParamSpec


class RoutedExperts(FeedForward):
    reads_stream = True       # forward takes ``stream=``: the 32-bit rows that ``x`` was rounded from, for the router

    SCORINGS = ("softmax", "sigmoid")
    ACTIVATIONS = ("silu", "clamped")

    def __init__(self, width: int, intermediate: int, experts: int, top: int, router: str = "router", expert: str = "e{}",
                 pieces=("gate", "up", "down"), scoring: str = "softmax", groups=None, activation: str = "silu", limit: float = 0.0,
                 reads_stream: bool = True, router_bias: str = None):
        if not 1 <= top <= experts:
            raise ValueError(f"a token uses {top} of {experts} experts")
        if scoring not in self.SCORINGS or activation not in self.ACTIVATIONS:
            raise ValueError(f"scoring {scoring!r} / activation {activation!r}: built are {self.SCORINGS} and {self.ACTIVATIONS}")
        if groups is not None:
            count, keep = groups
            if scoring != "sigmoid" or experts % count or not 1 <= keep <= count or top > keep * (experts // count):
                raise ValueError(f"{experts} experts in {count} groups of which {keep} are kept, {top} chosen, scoring {scoring!r}")
        if activation == "clamped" and not limit > 0.0:
            raise ValueError("the clamped activation needs its limit")
        self.scoring, self.groups, self.activation, self.limit = scoring, tuple(groups) if groups is not None else None, activation, float(limit)
        self.reads_stream = reads_stream
        self.width, self.intermediate, self.experts, self.top = width, intermediate, experts, top
        self.router_name, self.expert_name, self.pieces = router, expert, tuple(pieces)
        self._parts = {}
        self.router_bias_name = router_bias       # the name of a vector that is added to the router's logits, or None
        self.router_bias = None   # float32 [experts]
        self.router = None        # float32 [experts, W]
        self.gate_up = None       # [experts, 2F, W]
        self.down = None          # [experts, W, F]

    def _names(self):
        gate, up, down = self.pieces
        for index in range(self.experts):
            prefix = self.expert_name.format(index)
            yield index, f"{prefix}.{gate}", f"{prefix}.{up}", f"{prefix}.{down}"

    def param_specs(self):
        share = self.top / self.experts
        specs = {self.router_name: ParamSpec((self.experts, self.width), VECTOR, "normal")}
        if self.router_bias_name is not None:
            specs[self.router_bias_name] = ParamSpec((self.experts,), VECTOR, "bias")
        for _, gate, up, down in self._names():
            specs[gate] = ParamSpec((self.intermediate, self.width), share_per_token=share)
            specs[up] = ParamSpec((self.intermediate, self.width), share_per_token=share)
            specs[down] = ParamSpec((self.width, self.intermediate), share_per_token=share)
        return specs

    def assign(self, name, tensor):
        if name == self.router_name:
            self.router = tensor
        elif name == self.router_bias_name:
            self.router_bias = tensor
        else:
            self._parts[name] = tensor

    def finalize(self):
        names = list(self._names())
        self.gate_up = torch.stack([torch.cat([self._parts[gate], self._parts[up]], dim=0) for _, gate, up, _ in names]).contiguous()
        self.down = torch.stack([self._parts[down] for _, _, _, down in names]).contiguous()
        self._parts.clear()

    def forward(self, x, ctx, stream=None):
        """``x [T, W]`` in the compute type -> float32 ``[T, W]``.  ``stream``: the same rows in 32-bit, if the caller
        has them (the router's logits are 32-bit either way; from these they need no widening first)."""
        ops = ctx.ops
        n = x.shape[0]
        chosen = ctx.empty((n, self.top), dtype=torch.int32)
        weights = ctx.empty((n, self.top), dtype=torch.float32)
        extra = {} if self.scoring == "softmax" else {"scoring": self.scoring, "groups": self.groups}
        if self.router_bias is not None:
            extra["bias"] = self.router_bias
        ops.route_experts(x if stream is None else stream, self.router, self.top, chosen, weights, **extra)
        out = ctx.empty((n, self.width), dtype=torch.float32)
        extra = {} if self.activation == "silu" else {"activation": self.activation, "limit": self.limit}
        if ops.experts_sorted(x, self.gate_up, self.down, chosen, weights, out, **extra):       # many tokens: pairs sorted by expert
            return out
        hidden = ctx.empty((n * self.top, self.intermediate))
        ops.experts_gate_up(x, self.gate_up, chosen, hidden, **extra)
        ops.experts_down(hidden, self.down, chosen, weights, out)
        return out
