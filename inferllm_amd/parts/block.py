"""Arrangements of mixer, feed-forward and norms around the residual stream."""
from __future__ import annotations

from ..kernels import ops
from .base import Block, StepContext, register_part


@register_part("block", "pre_norm")
class PreNormBlock(Block):
    """x1 = x + mixer(norm(x)); x2 = x1 + feed_forward(norm(x1)).

    src/graph/llama_like.cpp:66-105.  The residual stream stays float32; each add is
    fused into the norm that follows it, so the block returns its feed-forward
    output for the next norm (the next block's, or the model's last) to add.  For steps of
    few rows, parts that say so (`Part.adds_residual`, `takes_normed_rows`) shorten this: a
    part adds its output to the stream in its last kernel, which also prepares the norm that
    follows for the next part's first kernel; what the block hands on is then None (nothing
    left to add) or `ops.NormedRows`.
    """

    graph_safe_prompts = True

    takes_next_norm = True
    takes_prepared_rows = True

    @staticmethod
    def _enter(norm, part, x, pending, ctx):
        """The input of `part`: the normed rows of x (+ pending), by a kernel or prepared."""
        if isinstance(pending, ops.NormedRows):
            params = norm.rms_params()
            if params is not None and pending.made_for(*params):
                return pending if part.takes_normed_rows else pending.rows()
            pending = None                       # the sum is in x already; another norm follows
        return norm.forward(x, pending, ctx)

    def forward(self, x, pending, ctx: StepContext, line, writes_cache, next_norm=None):
        h = self._enter(self.mixer_norm, self.mixer, x, pending, ctx)
        if self.mixer.adds_residual:
            d = self.mixer.forward(h, ctx, line, writes_cache, self.position, residual=x,
                                   next_norm=self.feed_forward_norm)
        else:
            d = self.mixer.forward(h, ctx, line, writes_cache, self.position)
        h2 = self._enter(self.feed_forward_norm, self.feed_forward, x, d, ctx)
        if self.feed_forward.adds_residual:
            return self.feed_forward.forward(h2, ctx, residual=x, next_norm=next_norm)
        return self.feed_forward.forward(h2, ctx)


@register_part("block", "parallel")
class ParallelBlock(Block):
    """x <- x + (mixer(h) + feed_forward(h)) with h = norm(x): one norm, both parts read its rows.

    The two outputs are left for the next norm to add to the stream as (mixer + feed-forward) in
    float32: as a pair, if that norm says it adds pairs in its own kernel (`Norm.adds_pairs`), else
    as their float32 sum (`ops.sum_rows`).  A feed-forward that returns None (a layer without one)
    leaves the mixer's output alone.
    """

    graph_safe_prompts = True

    takes_next_norm = True           # to know whether the norm that follows adds a pair itself
    takes_prepared_rows = True       # (prepared rows mean: the sum is in x already)

    def forward(self, x, pending, ctx: StepContext, line, writes_cache, next_norm=None):
        if isinstance(pending, ops.NormedRows):
            pending = None                       # its sum is in x already
        if isinstance(pending, tuple) and not getattr(self.mixer_norm, "adds_pairs", False):
            pending = ops.sum_rows(*pending)
        h = self.mixer_norm.forward(x, pending, ctx)
        a = self.mixer.forward(h, ctx, line, writes_cache, self.position)
        f = self.feed_forward.forward(h, ctx)
        if f is None:
            return a
        if next_norm is not None and getattr(next_norm, "adds_pairs", False):
            return (a, f)
        return ops.sum_rows(a, f)
