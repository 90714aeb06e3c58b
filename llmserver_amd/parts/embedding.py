"""Token embedding lookup ``h0 = E[ids]`` (utils/model.py:56-59,110), optionally times a constant and into several
residual streams at once."""
from __future__ import annotations

import torch

from .base import MATRIX, ParamSpec, Part


class TokenEmbedding(Part):
    """``tensor``: the table's name below the part's own ("" if the part's name is the tensor's).  ``wide``: the rows
    start a residual stream that is kept in 32-bit whatever the type of the table.  ``scale``: what a wide row is
    multiplied by (in 32-bit; the table itself stays as stored, so a head that shares it reads it unscaled).
    ``streams``: a wide stream starts as this many equal copies ``[streams, T, W]`` (0: one stream ``[T, W]``)."""

    def __init__(self, vocab: int, width: int, tensor: str = "weight", wide: bool = False, scale: float = 1.0, streams: int = 0):
        if (scale != 1.0 or streams) and not wide:
            raise ValueError("a scaled embedding, and one that starts several streams, starts a 32-bit stream (wide=True)")
        self.vocab, self.width, self.tensor, self.wide = vocab, width, tensor, wide
        self.scale, self.streams = float(scale), int(streams)
        self.weight = None

    def param_specs(self):
        return {self.tensor: ParamSpec((self.vocab, self.width), MATRIX, "normal", share_per_token=0.0)}

    def assign(self, name, tensor):
        assert name == self.tensor
        self.weight = tensor

    def forward(self, token_ids, ctx):
        if self.wide:
            shape = (token_ids.shape[0], self.width)
            out = ctx.empty((self.streams, *shape) if self.streams else shape, dtype=torch.float32)
            if self.scale != 1.0 or self.streams:
                ctx.ops.embedding_wide(self.weight, token_ids, out, scale=self.scale)
            else:
                ctx.ops.embedding_wide(self.weight, token_ids, out)
            return out
        out = ctx.empty((token_ids.shape[0], self.width))
        ctx.ops.embedding(self.weight, token_ids, out)
        return out


class NormedTokenEmbedding(Part):
    """Lookup followed by a norm, as one kernel, into a 32-bit residual stream: ``x = norm(E[ids])``.  The table's
    tensor has the part's own name, the norm's weight the name ``norm`` below it."""

    def __init__(self, vocab: int, width: int, norm, table: str = "", norm_name: str = "norm"):
        self.vocab, self.width, self.norm = vocab, width, norm
        self.table_name, self.norm_name = table, norm_name
        self.weight = None

    def param_specs(self):
        specs = {self.table_name: ParamSpec((self.vocab, self.width), MATRIX, "normal", share_per_token=0.0)}
        for name, spec in self.norm.param_specs().items():
            specs[f"{self.norm_name}.{name}" if name else self.norm_name] = spec
        return specs

    def assign(self, name, tensor):
        if name == self.table_name:
            self.weight = tensor
        elif name == self.norm_name:
            self.norm.assign("", tensor)
        else:
            self.norm.assign(name[len(self.norm_name) + 1:], tensor)

    def forward(self, token_ids, ctx):
        out = ctx.empty((token_ids.shape[0], self.width), dtype=torch.float32)
        ctx.ops.embedding_norm(self.weight, token_ids, self.norm.weight, self.norm.eps, out)
        return out
