"""Arrangements of a layer's parts.

"prenorm" is the reference's: norm -> mixer -> add; norm -> feed-forward -> add
(runtime/backends/cuda/native/transformer_forward.cu:1805-1816, 2176-2241, 2260-2271,
2528-2610).  The adds are not done here: each sub-block's output is handed on as a pending
delta, and the norm that follows adds it to the float32 stream in the same kernel that
normalises (the reference's ResidualAddRmsNorm, cuda_kernels.cu:617-671).

With ``residual_scale`` m the adds are x <- x + m * sub-block(norm(x)) (the deltas are handed on with their factor,
``ScaledDelta``), and a layer may have no feed-forward (then no second norm either).

"outnorm" puts the norms on the sub-blocks' outputs instead: x <- x + norm1(mixer(x)), then
x <- x + norm2(ffn(x)); the sub-blocks read the stream itself (rounded to the activation type), and a layer may
have no feed-forward.  Its norms are parts with ``add_to(stream, delta, cast_dtype)``, which adds the normed delta
into the stream and returns the rounding that the next sub-block reads, all in one kernel.

"hyper" replaces the one stream by ``streams`` copies x_1 .. x_S (all equal to the embedding at the start).  Sub-block q
(1: the mixer, 2: the feed-forward) with its weights in_q [S], out_q [S], mix_q [S, S] reads u = sum_s in_q[s] x_s, computes
y = sub-block(norm(u)), and then all streams change at once from the old ones, x_t <- sum_s mix_q[s, t] x_s + out_q[t] y.
The update is not done where y is made: y travels on as ``HyperPending`` and the kernel that reads the streams for the
next sub-block (of this layer or the next) updates them first, so a sub-block costs one such kernel.  After the last layer
the model asks the block to ``close_stream``: the pending update, then the sum of the streams as the one stream that the
final norm reads.

For steps of few rows a sub-block that can do so adds its output to the stream in its last product's
epilogue and hands on the next norm's rows up to a factor per row (``ScaledRows``), which the sub-block
after it applies to its first product's sums: the norm between them then needs no kernel.  Parts that
do not declare this are given plain tensors, and a plain delta is taken from them.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..kernels.ops import ScaledDelta, ScaledRows
from .base import Block, MixerBinding, StreamSink, build_part, register_part
from .plan import LayerSpec, ParamSpec


def normed_for(norm, reader, residual, pending, ctx):
    """What ``reader`` is given: the norm of the stream plus ``pending``."""
    if getattr(pending, "in_stream", False):     # rows some other arrangement prepared for its like: the stream holds everything
        pending = None
    if isinstance(pending, ScaledRows):          # the delta is in the stream already
        accepts = getattr(reader, "accepts_scaled_rows", None)
        params = norm.rms_params()
        made_for_this_norm = params is not None and pending.norm_weight is params[0] and pending.eps == params[1]
        if made_for_this_norm and accepts is not None and accepts(pending.shape[0]):
            return pending
        pending = None                           # (rows prepared for another norm are of no use: the stream is)
    return norm.forward(residual, pending, ctx.act_dtype)


def _sink(part, residual, norm, mult=1.0):
    if norm is None or not getattr(part, "adds_to_stream", False):
        return None
    params = norm.rms_params()
    return StreamSink(residual, *params, mult) if params is not None else None


@register_part("block", "prenorm")
class PreNormBlock(Block):
    graph_safe = True

    def __init__(self, layer: LayerSpec, hidden_size: int, residual_scale: float = 1.0):
        if layer.norm_in is None or layer.extra or (layer.ffn is None) != (layer.norm_post is None):
            raise ValueError(f"layer {layer.prefix}: the prenorm block is a norm and a mixer, optionally a second norm with a feed-forward, no more and no less")
        self.prefix = layer.prefix
        self.residual_scale = float(residual_scale)
        self.norm_in = build_part("norm", layer.norm_in, hidden_size=hidden_size)
        self.mixer = build_part("mixer", layer.mixer, hidden_size=hidden_size)
        self.norm_post = build_part("norm", layer.norm_post, hidden_size=hidden_size) if layer.norm_post is not None else None
        self.ffn = build_part("ffn", layer.ffn, hidden_size=hidden_size) if layer.ffn is not None else None

    def children(self):
        return tuple(p for p in (self.norm_in, self.mixer, self.norm_post, self.ffn) if p is not None)

    def entry_norm(self):
        return self.norm_in

    def _scaled(self, delta):
        """A sub-block's output with the block's factor (what was added to the stream by the sub-block itself has it already)."""
        if self.residual_scale == 1.0 or isinstance(delta, ScaledRows):
            return delta
        return ScaledDelta(delta, self.residual_scale)

    def _mixer(self, h, ctx, binding, residual, following):
        sink = _sink(self.mixer, residual, self.norm_post if self.ffn is not None else following, self.residual_scale)
        out = self.mixer.forward(h, ctx, binding, sink=sink) if sink is not None else self.mixer.forward(h, ctx, binding)
        return self._scaled(out)

    def _ffn(self, h, ctx, residual, following):
        sink = _sink(self.ffn, residual, following, self.residual_scale)
        return self._scaled(self.ffn.forward(h, ctx, sink=sink) if sink is not None else self.ffn.forward(h, ctx))

    def forward(self, residual, pending, ctx, binding: MixerBinding, following=None):
        t = ctx.timer
        if t is None:
            h = normed_for(self.norm_in, self.mixer, residual, pending, ctx)
            delta = self._mixer(h, ctx, binding, residual, following)
            if self.ffn is None:
                return residual, delta
            h = normed_for(self.norm_post, self.ffn, residual, delta, ctx)
            return residual, self._ffn(h, ctx, residual, following)
        t.enter("norm"); h = normed_for(self.norm_in, self.mixer, residual, pending, ctx); t.mark("norm")
        t.enter("mixer"); delta = self._mixer(h, ctx, binding, residual, following); t.mark("mixer")
        if self.ffn is None:
            return residual, delta
        t.enter("norm"); h = normed_for(self.norm_post, self.ffn, residual, delta, ctx); t.mark("norm")
        t.enter("ffn"); out = self._ffn(h, ctx, residual, following); t.mark("ffn")
        return residual, out


@register_part("block", "outnorm")
class OutputNormBlock(Block):
    """x <- x + norm_in(mixer(x)); x <- x + norm_post(ffn(x)) (the second only if the layer has a feed-forward).  What
    a sub-block reads, the stream in the activation type, is handed from block to block as ``pending`` wrapped in
    ``StreamRows``, so that the kernel which adds a normed delta also writes the next reader's input."""
    graph_safe = True

    def __init__(self, layer: LayerSpec, hidden_size: int):
        if layer.norm_in is None or layer.extra or (layer.ffn is None) != (layer.norm_post is None):
            raise ValueError(f"layer {layer.prefix}: the outnorm block is a mixer with its norm and optionally a feed-forward with its norm")
        self.prefix = layer.prefix
        self.mixer = build_part("mixer", layer.mixer, hidden_size=hidden_size)
        self.norm_in = build_part("norm", layer.norm_in, hidden_size=hidden_size)
        self.ffn = build_part("ffn", layer.ffn, hidden_size=hidden_size) if layer.ffn is not None else None
        self.norm_post = build_part("norm", layer.norm_post, hidden_size=hidden_size) if layer.norm_post is not None else None
        for n in (self.norm_in, self.norm_post):
            if n is not None and not hasattr(n, "add_to"):
                raise ValueError(f"layer {layer.prefix}: the outnorm block needs norms that can add to the stream (add_to)")

    def children(self):
        return tuple(p for p in (self.mixer, self.norm_in, self.ffn, self.norm_post) if p is not None)

    def forward(self, residual, pending, ctx, binding: MixerBinding, following=None):
        t = ctx.timer
        if isinstance(pending, StreamRows) and pending.stream is residual:
            h = pending.rows
        else:
            if pending is not None:                       # a delta some other arrangement left: it belongs to the stream
                if isinstance(pending, ScaledDelta):
                    residual += pending.tensor()
                else:
                    residual += pending.sum(torch.float32) if hasattr(pending, "parts") else pending.float()
            h = residual if ctx.act_dtype == torch.float32 else ops.cast_rows(residual, ctx.act_dtype)
        if t is not None:
            t.enter("mixer")
        delta = self.mixer.forward(h, ctx, binding)
        if t is not None:
            t.mark("mixer"); t.enter("norm")
        h = self.norm_in.add_to(residual, delta, ctx.act_dtype)
        if t is not None:
            t.mark("norm")
        if self.ffn is not None:
            if t is not None:
                t.enter("ffn")
            delta = self.ffn.forward(h, ctx)
            if t is not None:
                t.mark("ffn"); t.enter("norm")
            h = self.norm_post.add_to(residual, delta, ctx.act_dtype)
            if t is not None:
                t.mark("norm")
        return residual, StreamRows(residual, h)


class StreamRows:
    """The stream rounded to the activation type (``rows``), valid for ``stream`` as it stands: what the next block
    that reads the stream itself takes as its input.  Anyone else ignores it (the stream already holds everything)."""
    __slots__ = ("stream", "rows")
    in_stream = True          # nothing is left to add: a reader that has no use for the rows drops them

    def __init__(self, stream, rows):
        self.stream, self.rows = stream, rows


class HyperStreams:
    """The S residual streams of a step's rows, float32 [T, S, H], as a "hyper" block hands them to the next."""
    __slots__ = ("data",)

    def __init__(self, data):
        self.data = data

    @property
    def device(self):
        return self.data.device


class HyperPending:
    """A sub-block's output y that has not changed the streams yet, with the weights that say how it will:
    x_t <- sum_s mix[s, t] x_s + out[t] y."""
    __slots__ = ("y", "mix", "out")

    def __init__(self, y, mix, out):
        self.y, self.mix, self.out = y, mix, out


_PARTIAL_SUMS_WELCOME = StreamSink(None, None, 0.0)


@register_part("block", "hyper")
class HyperConnectionBlock(Block):
    """Pre-norm sub-blocks over ``streams`` residual streams (see the module's text).  Tensors: ``<prefix>.hc1.in`` [S],
    ``.hc1.out`` [S], ``.hc1.mix`` [S, S] (indexed [from, to]) for the mixer and ``.hc2.*`` for the feed-forward; they are
    widened to float at load."""
    graph_safe = True

    def __init__(self, layer: LayerSpec, hidden_size: int, streams: int):
        if layer.norm_in is None or layer.extra or (layer.ffn is None) != (layer.norm_post is None):
            raise ValueError(f"layer {layer.prefix}: the hyper block is a norm and a mixer, optionally a second norm with a feed-forward")
        self.prefix, self.hidden_size, self.streams = layer.prefix, int(hidden_size), int(streams)
        if not 0 < self.streams <= ops.HYPER_MAX_STREAMS:
            raise ValueError(f"layer {layer.prefix}: {streams} streams (1 to {ops.HYPER_MAX_STREAMS})")
        self.norm_in = build_part("norm", layer.norm_in, hidden_size=hidden_size)
        self.mixer = build_part("mixer", layer.mixer, hidden_size=hidden_size)
        self.norm_post = build_part("norm", layer.norm_post, hidden_size=hidden_size) if layer.norm_post is not None else None
        self.ffn = build_part("ffn", layer.ffn, hidden_size=hidden_size) if layer.ffn is not None else None
        for n in (self.norm_in, self.norm_post):
            if n is not None and n.rms_params() is None and not hasattr(n, "weight"):
                raise ValueError(f"layer {layer.prefix}: the hyper block reads the streams through RMS norms")
        self.w = {}

    def children(self):
        return tuple(p for p in (self.norm_in, self.mixer, self.norm_post, self.ffn) if p is not None)

    def _subs(self):
        return ("hc1", "hc2") if self.ffn is not None else ("hc1",)

    def param_specs(self):
        S, out = self.streams, {}
        for q in self._subs():
            out[f"{self.prefix}.{q}.in"] = ParamSpec((S,), ("uniform", 0.1, 0.5))
            out[f"{self.prefix}.{q}.out"] = ParamSpec((S,), ("uniform", 0.5, 1.0))
            out[f"{self.prefix}.{q}.mix"] = ParamSpec((S, S), ("uniform", 0.0, 0.6))
        return out

    def load(self, tensors):
        for q in self._subs():
            for k in ("in", "out", "mix"):
                self.w[q, k] = tensors[f"{self.prefix}.{q}.{k}"].float().contiguous()
        self.ones = torch.ones(self.streams, dtype=torch.float32, device=self.w["hc1", "in"].device)

    def _read(self, streams, pending, sub, norm, ctx):
        """The streams after the pending update, and what sub-block ``sub`` reads from them through ``norm``."""
        weight, eps = norm.rms_params()
        src = streams.data if isinstance(streams, HyperStreams) else streams          # (one stream from the embedding: S copies)
        y = mix = out = None
        if isinstance(pending, HyperPending):
            y, mix, out = pending.y, pending.mix, pending.out
        elif pending is not None and not getattr(pending, "in_stream", False):
            raise ValueError(f"layer {self.prefix}: the hyper block was handed a delta of another arrangement")
        data, rows = ops.hyper_step(src, self.streams, y, mix, out, self.w[sub, "in"], weight, eps, ctx.act_dtype)
        return HyperStreams(data), rows

    @staticmethod
    def _run(part, h, ctx, *binding):
        """A sub-block's output; one that can leave its last product as partial sums is told that the kernel which updates
        the streams adds them up (nothing is added to a stream where it is made: every stream changes at once)."""
        if getattr(part, "adds_to_stream", False):
            return part.forward(h, ctx, *binding, sink=_PARTIAL_SUMS_WELCOME)
        return part.forward(h, ctx, *binding)

    def forward(self, residual, pending, ctx, binding: MixerBinding, following=None):
        t = ctx.timer
        if t is not None:
            t.enter("norm")
        streams, h = self._read(residual, pending, "hc1", self.norm_in, ctx)
        if t is not None:
            t.mark("norm"); t.enter("mixer")
        pending = HyperPending(self._run(self.mixer, h, ctx, binding), self.w["hc1", "mix"], self.w["hc1", "out"])
        if t is not None:
            t.mark("mixer")
        if self.ffn is None:
            return streams, pending
        if t is not None:
            t.enter("norm")
        streams, h = self._read(streams, pending, "hc2", self.norm_post, ctx)
        if t is not None:
            t.mark("norm"); t.enter("ffn")
        pending = HyperPending(self._run(self.ffn, h, ctx), self.w["hc2", "mix"], self.w["hc2", "out"])
        if t is not None:
            t.mark("ffn")
        return streams, pending

    def close_stream(self, residual, pending, ctx):
        """The one stream the final norm reads: the pending update, then the sum of the streams."""
        if not isinstance(residual, HyperStreams):
            return residual, pending
        y = mix = out = None
        if isinstance(pending, HyperPending):
            y, mix, out = pending.y, pending.mix, pending.out
        _, total = ops.hyper_step(residual.data, self.streams, y, mix, out, self.ones)
        return total, None
