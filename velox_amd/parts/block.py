"""Arrangements of one mixer and one feed-forward with their norms.

``PreNormBlock`` is the reference's ``DecoderLayer.forward`` (``src/decoder_layer.py:41-54``):
``h = h + mixer(norm1(h)); h = h + ff(norm2(h))``.  The residual ``h`` lives in a float32
tensor; what a sub-layer produced is carried as ``pending`` and added inside the next
norm's kernel, so each block hands its feed-forward output on to whoever normalises next.

``OutputNormBlock`` (not in the reference): ``h = h + m * norm1(mixer(h)); h = h + m * norm2(ff(h))``.  The sub-layers
read the residual stream itself and only their outputs are normed, so nothing is pending between blocks; what is handed
on is the updated residual in the run dtype (``ResidualCopy``), which the norm's kernel writes beside the float32 sum.

``ParallelBlock`` (not in the reference): ``n = norm(h); h = h + (mixer(n) + ff(n))``, one norm that both
sub-layers read.  It hands both outputs on as a ``SumOf``, which the next norm's kernel adds up in float32.

``HyperConnectionBlock`` (not in the reference): pre-norm sub-layers over several copies of the residual that are read
through learned weights and mixed by a learned matrix at every sub-layer.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .base import Block, FeedForward, Mixer, Norm, OutputNormSink, Part, ResidualCopy, ResidualSink, StreamUpdate, SumOf, register_arrangement


class PreNormBlock(Block):
    def __init__(self, prefix: str, mixer: Mixer, feed_forward: FeedForward, mixer_norm: Norm, ff_norm: Norm) -> None:
        super().__init__(prefix)
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.ff_norm = ff_norm
        self.has_feed_forward = type(feed_forward).__name__ != "NoFeedForward"

    def children(self) -> Tuple[Part, ...]:
        if not self.has_feed_forward:
            return (self.mixer_norm, self.mixer)  # (no second norm: its tensors do not exist)
        return (self.mixer_norm, self.mixer, self.ff_norm, self.feed_forward)

    def input_norm(self) -> Optional[Norm]:
        return self.mixer_norm

    def forward(self, residual: torch.Tensor, pending, ctx, cache, owns_cache: bool, next_norm: Optional[Norm] = None):
        """``next_norm``: the norm that will read this block's output (the next block's first norm), if the caller
        allows the feed-forward to add its output to the residual itself (see ``ResidualSink``)."""
        normed = self.mixer_norm.forward(residual, pending, ctx)
        if not getattr(self.mixer, "accepts_deferred", False):
            normed = ctx.ops.materialize(normed)  # (a DeferredNorm becomes a tensor; a tensor stays)
        if not self.has_feed_forward:
            return self.mixer.forward(normed, ctx, cache, owns_cache)  # (the mixer's output is what the next norm adds)
        if getattr(self.mixer, "accepts_sink", False):
            mixed = self.mixer.forward(normed, ctx, cache, owns_cache, sink=ResidualSink(residual, self.ff_norm))
        else:
            mixed = self.mixer.forward(normed, ctx, cache, owns_cache)
        normed = self.ff_norm.forward(residual, mixed, ctx)
        if not getattr(self.feed_forward, "accepts_deferred", False):
            normed = ctx.ops.materialize(normed)
        if next_norm is not None and getattr(self.feed_forward, "accepts_sink", False):
            return self.feed_forward.forward(normed, ctx, sink=ResidualSink(residual, next_norm))
        return self.feed_forward.forward(normed, ctx)


register_arrangement("pre_norm", PreNormBlock)


class ParallelBlock(Block):
    def __init__(self, prefix: str, mixer: Mixer, feed_forward: FeedForward, mixer_norm: Norm, ff_norm: Optional[Norm] = None) -> None:
        """``ff_norm`` is not used and owns no tensors here: there is one norm."""
        super().__init__(prefix)
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norm = mixer_norm

    def children(self) -> Tuple[Part, ...]:
        return (self.norm, self.mixer, self.feed_forward)

    def input_norm(self) -> Optional[Norm]:
        return self.norm

    def forward(self, residual: torch.Tensor, pending, ctx, cache, owns_cache: bool, next_norm: Optional[Norm] = None):
        normed = ctx.ops.materialize(self.norm.forward(residual, pending, ctx))
        mixed = self.mixer.forward(normed, ctx, cache, owns_cache)
        other = self.feed_forward.forward(normed, ctx)
        if other is None:
            return mixed
        if other.dim() == 3:
            mixed, other = other, mixed  # (the term that may be partial sums goes first)
        if other.dim() == 3:
            other = other.sum(0)
        return SumOf(mixed, other)


register_arrangement("parallel", ParallelBlock)


class OutputNormBlock(Block):
    def __init__(self, prefix: str, mixer: Mixer, feed_forward: FeedForward, mixer_norm: Norm, ff_norm: Norm, residual_mult: float = 1.0) -> None:
        """``residual_mult``: the factor ``m`` on both normed sub-layer outputs."""
        super().__init__(prefix)
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.ff_norm = ff_norm
        self.residual_mult = float(residual_mult)
        self.has_feed_forward = type(feed_forward).__name__ != "NoFeedForward"

    def children(self) -> Tuple[Part, ...]:
        if not self.has_feed_forward:
            return (self.mixer_norm, self.mixer)  # (no second norm: its tensor does not exist)
        return (self.mixer_norm, self.mixer, self.ff_norm, self.feed_forward)

    def input_norm(self) -> Optional[Norm]:
        return None  # (the block begins with its mixer)

    @staticmethod
    def _input(residual: torch.Tensor, pending, ctx) -> torch.Tensor:
        if isinstance(pending, ResidualCopy):
            return pending.copy
        if isinstance(pending, SumOf):
            first = pending.first.float().sum(0) if pending.first.dim() == 3 else pending.first.float()
            pending = first + pending.second.float()
        elif pending is not None and pending.dim() == 3:
            pending = pending.sum(0)
        return ctx.ops.add_cast(residual, pending, ctx.dtype)

    def forward(self, residual: torch.Tensor, pending, ctx, cache, owns_cache: bool, next_norm: Optional[Norm] = None):
        x = self._input(residual, pending, ctx)
        mixed = self.mixer.forward(x, ctx, cache, owns_cache)
        x = self.mixer_norm.add_normed(residual, mixed, self.residual_mult, ctx)
        if self.has_feed_forward:
            form = self.ff_norm.deferred_form()  # (weight, eps) of a weighted RMS norm, which a sub-layer's last kernel may take over
            if form is not None and getattr(self.feed_forward, "accepts_output_norm", False):
                out = self.feed_forward.forward(x, ctx, output_norm=OutputNormSink(residual, form[0], form[1], self.residual_mult))
            else:
                out = self.feed_forward.forward(x, ctx)
            if isinstance(out, ResidualCopy):
                return out
            x = self.ff_norm.add_normed(residual, out, self.residual_mult, ctx)
        return ResidualCopy(x)


register_arrangement("output_norm", OutputNormBlock)


class HyperConnectionBlock(Block):
    """Pre-norm sub-layers over ``streams`` copies of the residual (hyper-connections): for sub-layer ``q`` with learned
    ``in_q [S]``, ``out_q [S]`` and ``mix_q [S, S]`` (indexed [from, to]),

        ``u = sum_s in_q[s] x_s``;  ``y = sublayer(norm_q(u))``;  ``x_t <- sum_s mix_q[s, t] x_s + out_q[t] y``  (all ``t`` at once).

    The residual is float32 ``[T, S * H]``.  A sub-layer's output is not worked into the streams by a pass of its own:
    it is handed on as a ``StreamUpdate`` and the next norm's kernel (``StreamNorm``) applies it before it reads the
    streams, as the plain residual sum is folded into the next norm for the other arrangements.  The block's own tensors
    are ``<prefix>hc1.{in,out,mix}`` and ``<prefix>hc2.{in,out,mix}`` (``names`` replaces the two prefixes)."""

    def __init__(self, prefix: str, mixer: Mixer, feed_forward: FeedForward, mixer_norm: Norm, ff_norm: Norm, streams: int = 1,
                 names: Tuple[str, str] = ("hc1.", "hc2."), learned: bool = True) -> None:
        """``learned`` False: no tensors of the block's own; every stream is read with weight 1, keeps itself and takes
        the output with weight 1 (with one stream: the plain pre-norm block, which may also go without a feed-forward)."""
        super().__init__(prefix)
        self.learned = bool(learned)
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.ff_norm = ff_norm
        self.streams = int(streams)
        self.names = tuple(names)
        self.has_feed_forward = type(feed_forward).__name__ != "NoFeedForward"
        for norm in (mixer_norm, ff_norm):
            if getattr(norm, "streams", None) != self.streams or not hasattr(norm, "forward_streams"):
                raise ValueError(f"a block over {self.streams} streams needs norms over as many (the 'stream_norm' kind)")
        self.in1 = self.out1 = self.mix1 = self.in2 = self.out2 = self.mix2 = None

    def children(self) -> Tuple[Part, ...]:
        if not self.has_feed_forward:
            return (self.mixer_norm, self.mixer)  # (no second norm: its tensor does not exist)
        return (self.mixer_norm, self.mixer, self.ff_norm, self.feed_forward)

    def params(self):
        from .base import single

        s = self.streams
        out = {}
        if not self.learned:
            return out
        for number, name in ((1, self.names[0]), (2, self.names[1])):
            if number == 2 and not self.has_feed_forward:
                break
            out[f"in{number}"] = single(name + "in", (s,), role="vector", init="mean_plus_normal")
            out[f"out{number}"] = single(name + "out", (s,), role="vector", init="one_plus_normal")
            out[f"mix{number}"] = single(name + "mix", (s, s), role="vector", init="identity_plus_normal")
        return out

    def input_norm(self) -> Optional[Norm]:
        return self.mixer_norm

    def forward(self, residual: torch.Tensor, pending, ctx, cache, owns_cache: bool, next_norm: Optional[Norm] = None):
        normed = self.mixer_norm.forward_streams(residual, pending, self.in1, ctx)
        mixed = self.mixer.forward(normed, ctx, cache, owns_cache)
        update = StreamUpdate(mixed, self.mix1, self.out1)
        if not self.has_feed_forward:
            return update
        normed = self.ff_norm.forward_streams(residual, update, self.in2, ctx)
        return StreamUpdate(self.feed_forward.forward(normed, ctx), self.mix2, self.out2)


register_arrangement("hyper_connection", HyperConnectionBlock)
