"""Arrangements of a layer's parts around the residual stream.

Pre-norm with two residual additions, as the reference's block
(/root/reference/src/models/block.cpp:23-29): a = x + Mixer(N1(x)); y = a + FF(N2(a)).
The additions are made in float32 inside the following norm's kernel.
Parallel with one norm: x = N(h); y = h + Mixer(x) + FF(x).
"""
from __future__ import annotations

import torch

from .. import kernels
from .base import Block, PendingNorm, register_part


class PreNormBlock(Block):
    norm_slots = ("mixer", "feed_forward")

    def forward(self, h, delta, ctx, cache, state):
        pending = PendingNorm(h, delta, self.norms["mixer"])                  # x = N1(h + delta)
        x = pending if self.mixer.takes_pending_norm else pending.materialize()
        a = self.mixer.forward(x, ctx, cache, state)
        h = pending.h_after
        pending = PendingNorm(h, a, self.norms["feed_forward"])               # x = N2(h + a)
        x = pending if self.feed_forward.takes_pending_norm else pending.materialize()
        m = self.feed_forward.forward(x, ctx)
        return pending.h_after, m                                            # m is added by whoever comes next


class PreNormMixerOnlyBlock(Block):
    """The pre-norm arrangement of a layer that has no feed-forward: y = x + Mixer(N1(x))."""

    norm_slots = ("mixer",)
    uses_feed_forward = False

    def forward(self, h, delta, ctx, cache, state):
        pending = PendingNorm(h, delta, self.norms["mixer"])
        x = pending if self.mixer.takes_pending_norm else pending.materialize()
        a = self.mixer.forward(x, ctx, cache, state)
        return pending.h_after, a


class ParallelBlock(Block):
    """One norm whose output both branches read, both added to the stream: x = N(h); y = h + Mixer(x) + FF(x).
    The two branch outputs go on as one not-yet-added delta: float32 partial sums of both products side by side
    (the next norm's kernel adds them in float32), or, when a branch returns a rounded tensor, the mixer's output
    is added to the stream here and the feed-forward's goes on.

    Where the stream takes additions (fixed point, steps of few tokens) and nothing is pending, both branches are
    handed the norm unapplied: each may fold it into its own first product, and each adds its output into the stream
    itself.  Both must have read the stream before either adds to it, so the mixer runs in two phases (`project`
    reads, `finish` adds) around the feed-forward."""

    norm_slots = ("input",)

    def forward(self, h, delta, ctx, cache, state):
        pending = PendingNorm(h, delta, self.norms["input"])
        ff = self.feed_forward
        if (delta is None and h.dtype == torch.int64 and hasattr(self.mixer, "project") and self.mixer.takes_pending_norm
                and (ff is None or ff.takes_pending_norm)):
            projected = self.mixer.project(pending, ctx)
            m = ff.forward(_Reader(pending), ctx) if ff is not None else None
            a = self.mixer.finish(projected, ctx, cache, state)
            h = pending.h_after
        else:
            x = pending.materialize()
            h = pending.h_after
            a = self.mixer.forward(x, ctx, cache, state)
            m = ff.forward(x, ctx) if ff is not None else None
        if a is None or m is None:
            return h, (m if a is None else a)
        if a.dim() == 3 and m.dim() == 3 and a.dtype == m.dtype == torch.float32:
            return h, torch.cat([a, m], dim=0)
        kernels.backend().residual_add(h, a)
        return h, m


class _Reader(PendingNorm):
    """The same pending norm for a second part that reads the stream: nothing is pending on a complete stream, so the
    part may fold the norm or compute it again, and what it learns of the stream is passed on to the first."""

    def __init__(self, first: PendingNorm):
        super().__init__(first.h_after if first.h_after is not None else first.h, None, first.norm)
        self.first = first

    def applied(self, h_new) -> None:
        super().applied(h_new)
        self.first.h_after = h_new

    def materialize(self):
        x = super().materialize()
        self.first.h_after = self.h_after
        return x


class ParallelMixerOnlyBlock(ParallelBlock):
    """The parallel arrangement of a layer that has no feed-forward: y = h + Mixer(N(h))."""

    uses_feed_forward = False


register_part("block", "pre_norm", PreNormBlock)
register_part("block", "pre_norm_mixer_only", PreNormMixerOnlyBlock)
register_part("block", "parallel", ParallelBlock)
register_part("block", "parallel_mixer_only", ParallelMixerOnlyBlock)
