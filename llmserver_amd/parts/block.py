"""Pre-norm residual block: ``h += mixer(norm_in(h)); h += ffn(norm_post(h))``.

Order of the parts as in utils/model.py:15-35.  The block keeps the reference's
fused dataflow (utils/model.py:87-100): the residual stream and the update that
is still to be added travel as a pair, so every "add, then normalise" is one kernel.
"""
from __future__ import annotations

import torch

from .base import (VECTOR, Block, FeedForward, Mixer, Norm, PagedAndStateSpec, PagedKVSpec, ParamSpec, Part, ResidualSink,
                   StreamUpdate)


class PreNormBlock(Block):
    takes_following = True

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm, ffn: FeedForward,
                 names=("input_layernorm", "self_attn", "post_attention_layernorm", "mlp")):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn
        self.names = tuple(names)

    def _parts(self):
        return dict(zip(self.names, (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)))

    def param_specs(self):
        return {f"{prefix}.{name}": spec for prefix, part in self._parts().items() for name, spec in part.param_specs().items()}

    def assign(self, name, tensor):
        prefix, rest = name.split(".", 1)
        self._parts()[prefix].assign(rest, tensor)

    def finalize(self):
        for part in self._parts().values():
            part.finalize()

    @staticmethod
    def _feed(norm, consumer, resid, delta, ctx, *args, following=None):
        """Run ``consumer`` on ``norm(resid + delta)``; returns ``(resid + delta, consumer's output)``.

        A consumer that starts with a projection gets the normalisation still pending, so that the
        projection may apply a norm that the previous projection prepared (``delta`` is then a
        :class:`StreamUpdate`); otherwise the norm runs first, in its own kernel.  A consumer that
        ends with a projection is told the norm that follows its output (``following``), so that
        this projection may in turn add its result to the stream and prepare that norm."""
        if consumer.accepts_pending_norm:
            pending = norm.defer(resid, delta, ctx)
            kwargs = {}
            if following is not None and consumer.takes_sink:
                kwargs["sink"] = ResidualSink(pending, following)
            out = consumer.forward(pending, ctx, *args, **kwargs)
            if pending.delta is not None:          # nobody used it: the update must still be added
                pending.tensor()
            return pending.resid, out
        if isinstance(delta, StreamUpdate):
            resid, delta = delta.resid, None
        return resid, consumer.forward(norm.add_norm(resid, delta, ctx), ctx, *args)

    def entry_norm(self):
        return self.mixer_norm

    def forward(self, resid, delta, ctx, cache, following=None):
        """``following``: the norm that will be applied to this block's output, if the caller knows it."""
        resid, mixed = self._feed(self.mixer_norm, self.mixer, resid, delta, ctx, cache, following=self.ffn_norm)
        return self._feed(self.ffn_norm, self.ffn, resid, mixed, ctx, following=following)


class DepthAverage(Part):
    """What a layer hands on is a weighted sum of the embedding's output and the results of all layers so far:
    ``sum_{j <= i + 1} w[j] * X_j`` behind layer ``i`` (``X_0`` the embedding's output, ``X_(j+1)`` layer ``j``'s own
    result).  The results of a step's tokens are kept for the length of the step, in 32-bit; ``states`` is how many a
    model has (its layers and one).  Layer ``i``'s weights are a vector of ``i + 2`` numbers."""

    def __init__(self, index: int, states: int, tensor: str = "dwa"):
        self.index, self.states, self.tensor = index, states, tensor
        self.weights = None     # float32 [index + 2]

    def param_specs(self):
        return {self.tensor: ParamSpec((self.index + 2,), VECTOR, "norm")}

    def assign(self, name, tensor):
        assert name == self.tensor
        self.weights = tensor

    def history(self, x, ctx):
        """The step's kept results ``[states, T, W]``; the first layer puts the embedding's output there."""
        kept = ctx.computed(("depth average", self.states), lambda: ctx.empty((self.states, *x.shape), dtype=torch.float32))
        if self.index == 0:
            kept[0].copy_(x)
        return kept


class PostNormBlock(Block):
    """Sublayers that read the stream itself and are normalised on their way out:
    ``x <- x + s1 * n1(mixer(x + conv(x)))``, then ``x <- x + s2 * n2(ffn(x))``, the stream in 32-bit throughout.

    ``conv`` (a :class:`~llmserver_amd.parts.conv.ShortConvolution` or None) stands in front of the mixer and keeps a
    per-request state beside the mixer's cache; ``scales`` says whether per-channel scales ``ls1`` / ``ls2`` multiply the
    normalised results; ``ffn`` may be None; ``average`` (a :class:`DepthAverage` or None) mixes the layer's result with
    the results before it.  The sum, the norm, the scale and the average behind a sublayer are one kernel."""

    def __init__(self, mixer: Mixer, mixer_norm: Norm, ffn, ffn_norm, conv=None, scales: bool = True, average=None,
                 names=("mix", "norm1", "mlp", "norm2", "canon1", "ls1", "ls2")):
        self.mixer, self.mixer_norm, self.ffn, self.ffn_norm, self.conv, self.average = mixer, mixer_norm, ffn, ffn_norm, conv, average
        self.names = tuple(names)
        self.scales = scales
        self.scale1 = self.scale2 = None
        self.width = mixer_norm.width

    def _parts(self):
        mix, norm1, mlp, norm2, conv = self.names[:5]
        parts = {mix: self.mixer, norm1: self.mixer_norm}
        if self.ffn is not None:
            parts.update({mlp: self.ffn, norm2: self.ffn_norm})
        if self.conv is not None:
            parts[conv] = self.conv
        return parts

    def param_specs(self):
        specs = {f"{prefix}.{name}" if name else prefix: spec for prefix, part in self._parts().items()
                 for name, spec in part.param_specs().items()}
        if self.scales:
            specs[self.names[5]] = ParamSpec((self.width,), VECTOR, "norm")
            if self.ffn is not None:
                specs[self.names[6]] = ParamSpec((self.width,), VECTOR, "norm")
        if self.average is not None:
            specs.update(self.average.param_specs())
        return specs

    def assign(self, name, tensor):
        if self.scales and name in self.names[5:7]:
            if name == self.names[5]:
                self.scale1 = tensor
            else:
                self.scale2 = tensor
            return
        if self.average is not None and name in self.average.param_specs():
            self.average.assign(name, tensor)
            return
        parts = self._parts()
        if name in parts:                                   # the part's name is the tensor's
            parts[name].assign("", tensor)
            return
        prefix, rest = name.split(".", 1)
        parts[prefix].assign(rest, tensor)

    def finalize(self):
        for part in self._parts().values():
            part.finalize()

    def cache_spec(self):
        spec = self.mixer.cache_spec()
        state = self.conv.state_spec() if self.conv is not None else None
        if state is None:
            return spec
        if not isinstance(spec, PagedKVSpec):
            raise ValueError("a convolution in front of the mixer keeps its state beside a paged cache only")
        return PagedAndStateSpec(spec, state)

    def forward(self, resid, delta, ctx, cache):
        if delta is not None:
            raise ValueError("this block takes a stream to which everything has been added")
        x = resid
        ops = ctx.ops
        wide = ctx.dtype == torch.float32
        h = self.conv.forward(x, ctx, cache.state) if self.conv is not None else (x if wide else x.to(ctx.dtype))
        mixed = self.mixer.forward(h, ctx, cache)
        last = self.ffn is None
        history = self.average.history(x, ctx) if self.average is not None else None
        after = {"history": history, "before": self.average.index + 1, "mix": self.average.weights} if history is not None else {}
        out = ctx.empty(x.shape, dtype=torch.float32)
        if last:
            ops.scaled_norm_add(x, mixed, self.mixer_norm.weight, self.scale1, self.mixer_norm.eps, out, **after)
            return out, None
        rounded = None if wide else ctx.empty(x.shape)
        ops.scaled_norm_add(x, mixed, self.mixer_norm.weight, self.scale1, self.mixer_norm.eps, out, rounded=rounded)
        if getattr(self.ffn, "reads_stream", False):
            fed = self.ffn.forward(out if wide else rounded, ctx, stream=out)
        else:
            fed = self.ffn.forward(out if wide else rounded, ctx)
        result = ctx.empty(x.shape, dtype=torch.float32)
        ops.scaled_norm_add(out, fed, self.ffn_norm.weight, self.scale2, self.ffn_norm.eps, result, **after)
        return result, None


class SandwichBlock(Block):
    """A norm in front of every sublayer and one behind it: ``x <- x + n1b(mixer(n1(x)))``, then
    ``x <- x + n2b(ffn(n2(x)))``, the stream in 32-bit throughout; ``ffn`` may be None.  The norm behind a sublayer, the
    sum with the stream and the norm in front of the next sublayer are one kernel (``ops.norm_add_norm``); a mixer that
    returns two results with scales (:class:`~llmserver_amd.parts.parallel.ScaledPair`) has them added up there too."""
    takes_following = True

    def __init__(self, mixer_norm: Norm, mixer: Mixer, mixer_out_norm: Norm, ffn_norm=None, ffn=None, ffn_out_norm=None,
                 names=("norm1", "mix", "norm1b", "norm2", "mlp", "norm2b")):
        self.mixer_norm, self.mixer, self.mixer_out_norm = mixer_norm, mixer, mixer_out_norm
        self.ffn_norm, self.ffn, self.ffn_out_norm = ffn_norm, ffn, ffn_out_norm
        self.names = tuple(names)

    def _parts(self):
        parts = dict(zip(self.names[:3], (self.mixer_norm, self.mixer, self.mixer_out_norm)))
        if self.ffn is not None:
            parts.update(zip(self.names[3:], (self.ffn_norm, self.ffn, self.ffn_out_norm)))
        return parts

    def param_specs(self):
        return {f"{prefix}.{name}" if name else prefix: spec for prefix, part in self._parts().items()
                for name, spec in part.param_specs().items()}

    def assign(self, name, tensor):
        parts = self._parts()
        if name in parts:                                   # the part's name is the tensor's
            parts[name].assign("", tensor)
            return
        prefix, rest = name.split(".", 1)
        parts[prefix].assign(rest, tensor)

    def finalize(self):
        for part in self._parts().values():
            part.finalize()

    def entry_norm(self):
        return self.mixer_norm

    @staticmethod
    def _update(ctx, x, result, norm, following):
        """``x + norm(result)`` and, if ``following`` is given, that norm of the sum in the compute type."""
        from .parallel import ScaledPair
        second, scales = None, None
        if isinstance(result, ScaledPair):
            result, second, scales = result.left, result.right, (result.left_scale, result.right_scale)
        out = ctx.empty(x.shape, dtype=torch.float32)
        normed = ctx.empty(x.shape) if following is not None else None
        ctx.ops.norm_add_norm(x, result, norm.weight, norm.eps, out, following.weight if following is not None else None,
                              following.eps if following is not None else 0.0, normed, second, scales)
        return out, normed

    def forward(self, resid, delta, ctx, cache, following=None):
        """``delta``: None, or a :class:`StreamUpdate` whose ``normed`` rows are the stream under this block's first norm
        (the block before was told that norm as its ``following`` and has carried it out)."""
        x, h = resid, None
        if isinstance(delta, StreamUpdate):
            x = delta.resid
            h = delta.normed if delta.norm is self.mixer_norm else None
        elif delta is not None:
            raise ValueError("this block takes a stream to which everything has been added")
        if h is None:
            h = ctx.empty(x.shape)
            ctx.ops.norm_rows(x, None, self.mixer_norm.weight, self.mixer_norm.eps, h)
        mixed = self.mixer.forward(h, ctx, cache)
        if self.ffn is None:
            return self._handed_on(*self._update(ctx, x, mixed, self.mixer_out_norm, self._same_kind(following)), following)
        x, h = self._update(ctx, x, mixed, self.mixer_out_norm, self.ffn_norm)
        fed = self.ffn.forward(h, ctx)
        return self._handed_on(*self._update(ctx, x, fed, self.ffn_out_norm, self._same_kind(following)), following)

    @staticmethod
    def _handed_on(x, normed, following):
        return x, (StreamUpdate(following, x, normed=normed) if normed is not None else None)

    @staticmethod
    def _same_kind(following):
        """The next block's first norm, if its kernel can be folded in here (a plain RMS norm of the stream)."""
        return following if following is not None and hasattr(following, "weight") and hasattr(following, "eps") else None


class HyperConnection(Part):
    """How one sublayer is connected to ``streams`` residual streams ``x_1 .. x_S``.  It reads ``sum_s read[s] * x_s``; its
    result ``y`` goes into every stream, each new stream formed from the streams as they stood before: ``x_t <- sum_s mix[s, t] * x_s + mult * write[t] * y``
    (``mix`` indexed [from, to]).  ``learned``: ``read``, ``write`` and ``mix`` are checkpoint tensors (``names``); not
    learned, they are ones and the identity, which is the plain residual sum ``x <- x + mult * y`` on one stream."""

    def __init__(self, streams: int, mult: float = 1.0, learned: bool = True, names=("in", "out", "mix")):
        self.streams, self.mult, self.learned, self.names = int(streams), float(mult), bool(learned), tuple(names)
        self.read = self.write = self.mix = None        # float32 [S], [S] (times mult), [S, S]

    def param_specs(self):
        if not self.learned:
            return {}
        read, write, mix = self.names
        return {read: ParamSpec((self.streams,), VECTOR, "norm"), write: ParamSpec((self.streams,), VECTOR, "norm"),
                mix: ParamSpec((self.streams, self.streams), VECTOR, "identity")}

    def assign(self, name, tensor):
        read, write, mix = self.names
        if name == read:
            self.read = tensor
        elif name == write:
            self.write = tensor
        elif name == mix:
            self.mix = tensor
        else:
            raise KeyError(name)

    def settle(self, like: torch.Tensor) -> None:
        """Once all tensors are there (``like``: any float32 tensor of the block, for its device)."""
        if not self.learned:
            self.read, self.write = like.new_ones((self.streams,)), like.new_ones((self.streams,))
            self.mix = torch.eye(self.streams, device=like.device, dtype=like.dtype)
        self.write = (self.write * self.mult).contiguous()
        self.read, self.mix = self.read.contiguous(), self.mix.contiguous()


class MultiStreamBlock(Block):
    """Pre-norm sublayers over several residual streams kept in 32-bit, ``[streams, T, W]``: each sublayer reads a
    weighted sum of the streams under its norm and writes its result, times a constant, back into all of them through
    its :class:`HyperConnection`; ``ffn`` may be None.  With one stream and connections that are not learned this is
    the plain ``x <- x + mult * sublayer(norm(x))``.  The update behind a sublayer and the read and norm in front of the
    next one (the next block's, if it is of this kind) are one kernel (``ops.streams_update``).

    ``mixer_norm`` / ``ffn_norm``: :class:`~llmserver_amd.parts.norm.StreamReadNorm`; ``names``: the checkpoint's names of
    the mixer's norm, the mixer, the feed-forward's norm, the feed-forward and the two connections."""
    takes_following = True

    def __init__(self, mixer_norm, mixer: Mixer, mixer_connection: HyperConnection, ffn_norm=None, ffn=None, ffn_connection=None,
                 names=("norm1", "mix", "norm2", "mlp", "hc1", "hc2")):
        self.mixer_norm, self.mixer, self.mixer_connection = mixer_norm, mixer, mixer_connection
        self.ffn_norm, self.ffn, self.ffn_connection = ffn_norm, ffn, ffn_connection
        self.names = tuple(names)
        self.streams = mixer_connection.streams

    def _parts(self):
        norm1, mix, norm2, mlp, hc1, hc2 = self.names
        parts = {norm1: self.mixer_norm, mix: self.mixer, hc1: self.mixer_connection}
        if self.ffn is not None:
            parts.update({norm2: self.ffn_norm, mlp: self.ffn, hc2: self.ffn_connection})
        return parts

    def param_specs(self):
        return {f"{prefix}.{name}" if name else prefix: spec for prefix, part in self._parts().items()
                for name, spec in part.param_specs().items()}

    def assign(self, name, tensor):
        parts = self._parts()
        if name in parts:                                   # the part's name is the tensor's
            parts[name].assign("", tensor)
            return
        prefix, rest = name.split(".", 1)
        parts[prefix].assign(rest, tensor)

    def finalize(self):
        self.mixer_connection.settle(self.mixer_norm.weight)
        self.mixer_norm.read_weights = self.mixer_connection.read
        if self.ffn is not None:
            self.ffn_connection.settle(self.ffn_norm.weight)
            self.ffn_norm.read_weights = self.ffn_connection.read
        for part in self._parts().values():
            part.finalize()

    def entry_norm(self):
        return self.mixer_norm

    def _update(self, ctx, streams, result, connection, following):
        """The streams behind a sublayer (updated where they lie) and, if ``following`` is given, what the next sublayer
        reads from them under its norm, in the compute type."""
        normed = ctx.empty(streams.shape[1:]) if following is not None else None
        ctx.ops.streams_update(streams, result, connection.mix, connection.write,
                               following.read_weights if following is not None else None,
                               following.weight if following is not None else None,
                               following.eps if following is not None else 0.0, normed)
        return streams, normed

    def _same_kind(self, following):
        """The next block's first norm, if it reads as many streams as this block keeps."""
        from .norm import StreamReadNorm
        return following if isinstance(following, StreamReadNorm) and following.streams == self.streams \
            and following.read_weights is not None else None

    def forward(self, resid, delta, ctx, cache, following=None):
        """``delta``: None, or a :class:`StreamUpdate` whose ``normed`` rows are what this block's mixer reads (the block
        before was told this block's first norm as its ``following`` and has carried it out)."""
        streams, h = resid, None
        if isinstance(delta, StreamUpdate):
            streams = delta.resid
            h = delta.normed if delta.norm is self.mixer_norm else None
        elif delta is not None:
            raise ValueError("this block takes streams to which everything has been added")
        if h is None:
            h = self.mixer_norm.add_norm(streams, None, ctx)
        mixed = self.mixer.forward(h, ctx, cache)
        following = self._same_kind(following)
        if self.ffn is None:
            streams, normed = self._update(ctx, streams, mixed, self.mixer_connection, following)
        else:
            streams, h = self._update(ctx, streams, mixed, self.mixer_connection, self.ffn_norm)
            fed = self.ffn.forward(h, ctx)
            streams, normed = self._update(ctx, streams, fed, self.ffn_connection, following)
        return streams, (StreamUpdate(following, streams, normed=normed) if normed is not None else None)


class ParallelGatedBlock(Block):
    """Both sublayers read one norm of the stream and their results join it together:
    ``h = norm(x)``, ``x <- x + s1 * sigmoid(G1 h + b1) * mixer(h) + s2 * sigmoid(G2 h + b2) * ffn(h)``, the stream in
    32-bit throughout; ``ffn`` may be None.  ``s`` are per-channel scales, ``G``, ``b`` a gate per channel and sublayer
    (both gates are one product).  The gates' sigmoids, the scales, the sum with the stream and the norm in front of the
    next block are one kernel (``ops.gated_pair_update``).

    ``names``: the checkpoint's names of the norm, the mixer, the feed-forward, the two scales and the two gates (a
    gate's bias is its name with ``bias_suffix`` behind it)."""
    takes_following = True

    def __init__(self, norm: Norm, mixer: Mixer, ffn=None, names=("norm1", "mix", "mlp", "ls1", "ls2", "rg1", "rg2"), bias_suffix: str = ".b"):
        from .linear import Linear
        self.norm, self.mixer, self.ffn = norm, mixer, ffn
        self.names = tuple(names)
        self.width = norm.width
        gate_names = self.names[5:7] if ffn is not None else self.names[5:6]
        self.gates = Linear(self.width, gate_names, (self.width,) * len(gate_names), bias=True, bare_names=True, bias_suffix=bias_suffix)
        self.scale1 = self.scale2 = None

    def _parts(self):
        norm, mix, mlp = self.names[:3]
        parts = {norm: self.norm, mix: self.mixer}
        if self.ffn is not None:
            parts[mlp] = self.ffn
        return parts

    def _scale_names(self):
        return self.names[3:5] if self.ffn is not None else self.names[3:4]

    def param_specs(self):
        specs = {f"{prefix}.{name}" if name else prefix: spec for prefix, part in self._parts().items()
                 for name, spec in part.param_specs().items()}
        specs.update(self.gates.param_specs())
        for name in self._scale_names():
            specs[name] = ParamSpec((self.width,), VECTOR, "norm")
        return specs

    def assign(self, name, tensor):
        if name in self._scale_names():
            if name == self.names[3]:
                self.scale1 = tensor
            else:
                self.scale2 = tensor
            return
        if self.gates.owns(name):
            self.gates.assign(name, tensor)
            return
        parts = self._parts()
        if name in parts:                                   # the part's name is the tensor's
            parts[name].assign("", tensor)
            return
        prefix, rest = name.split(".", 1)
        parts[prefix].assign(rest, tensor)

    def finalize(self):
        self.gates.finalize()
        for part in self._parts().values():
            part.finalize()

    def entry_norm(self):
        return self.norm

    def forward(self, resid, delta, ctx, cache, following=None):
        """``delta``: None, or a :class:`StreamUpdate` whose ``normed`` rows are the stream under this block's norm (the
        block before was told that norm as its ``following`` and has carried it out).  The stream is updated where it lies."""
        x, h = resid, None
        if isinstance(delta, StreamUpdate):
            x = delta.resid
            h = delta.normed if delta.norm is self.norm else None
        elif delta is not None:
            raise ValueError("this block takes a stream to which everything has been added")
        if h is None:
            h = ctx.empty(x.shape)
            ctx.ops.norm_rows(x, None, self.norm.weight, self.norm.eps, h)
        gates = self.gates.forward(h, ctx)
        mixed = self.mixer.forward(h, ctx, cache)
        fed = self.ffn.forward(h, ctx) if self.ffn is not None else None
        following = SandwichBlock._same_kind(following)
        normed = ctx.empty(x.shape) if following is not None else None
        ctx.ops.gated_pair_update(x, gates, mixed, self.scale1, fed, self.scale2, following.weight if following is not None else None,
                                  following.eps if following is not None else 0.0, normed)
        return x, (StreamUpdate(following, x, normed=normed) if normed is not None else None)
