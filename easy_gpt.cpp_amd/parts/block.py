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


class SandwichBlock(Block):
    """A norm before and a norm behind each branch, and a constant factor on what a branch adds:
    a = h + m * N1b(Mixer(N1(h))); y = a + m * N2b(FF(N2(a))).  The norms behind the branches read the branches' products
    unrounded (float32 partial sums) and the additions are float32, in one kernel with the norm that follows them where
    there is one.  With a stream join that keeps the depth's results (`parts/depth_average.py`), y is stored among them
    and what the next layer reads is their weighted sum, written by the kernel of the layer's last addition.  The norms
    are the layer norm without bias (`layernorm`, whose weight and eps the fused kernel takes)."""

    norm_slots = ("mixer", "mixer_out", "feed_forward", "feed_forward_out")
    takes_stream_join = True

    def __init__(self, mixer, feed_forward, norms, residual_mult: float = 1.0, stream_join=None):
        super().__init__(mixer, feed_forward, norms)
        self.residual_mult = float(residual_mult)
        self.stream_join = stream_join
        for slot in self.norm_slots:
            n = self.norms[slot]
            if getattr(n, "bias_name", "") is not None or not hasattr(n, "eps"):
                raise ValueError(f"the sandwich arrangement's norm '{slot}' must be a layer norm without bias")

    def parts(self):
        return super().parts() + ([self.stream_join] if self.stream_join is not None else [])

    def _last_addition(self, h, y, norm, ctx):
        """h + m * norm(y), through the stream join if there is one: the stream that goes on."""
        k = kernels.backend()
        join = self.stream_join
        if join is None:
            k.post_norm_add(h, y, norm.weight, norm.eps, self.residual_mult)
            return h
        kept = join.results(ctx, h)
        k.post_norm_add(h, y, norm.weight, norm.eps, self.residual_mult, history=kept, n_history=join.index, mix=join.weights)
        return h

    def forward(self, h, delta, ctx, cache, state):
        if h.dtype != torch.float32:
            raise TypeError("the sandwich arrangement keeps its stream in float32")
        k = kernels.backend()
        if self.stream_join is not None:
            self.stream_join.results(ctx, h)                              # (the first layer keeps the embedding's output)
        x = self.norms["mixer"].forward(h, delta)                         # adds what is pending, if anything
        y = self.mixer.forward(x, ctx, cache, state)
        if self.feed_forward is None:
            return self._last_addition(h, y, self.norms["mixer_out"], ctx), None
        post, pre = self.norms["mixer_out"], self.norms["feed_forward"]
        if pre.eps == post.eps:
            x = k.post_norm_add(h, y, post.weight, post.eps, self.residual_mult, next_weight=pre.weight)
        else:
            k.post_norm_add(h, y, post.weight, post.eps, self.residual_mult)
            x = pre.forward(h, None)
        z = self.feed_forward.forward(x, ctx)
        return self._last_addition(h, z, self.norms["feed_forward_out"], ctx), None


class SandwichMixerOnlyBlock(SandwichBlock):
    """The sandwich arrangement of a layer that has no feed-forward: y = h + m * N1b(Mixer(N1(h)))."""

    norm_slots = ("mixer", "mixer_out")
    uses_feed_forward = False


register_part("block", "sandwich", SandwichBlock)
register_part("block", "sandwich_mixer_only", SandwichMixerOnlyBlock)
