"""Pre-norm arrangement: ``r += mixer(norm(r)); r += feed_forward(norm(r))``; a layer
without a feed-forward has the first sub-layer only.  The sandwich arrangement has a second
norm behind each sub-layer, applied to its output before the add.

The add of each sub-layer's output is carried forward as ``delta`` and happens inside the
next norm kernel, as the reference threads ``(hidden, residual)`` through its layers
(rapid_llm/models/base.py:231-266,:363-375).
"""

from __future__ import annotations

from .base import BLOCKS, Block
from .lazy import NormedDelta, SummedDeltas, plain, run_norm


class PreNormBlock(Block):
    replayable = True
    accepts_deferred = True  # the incoming delta may be a DeferredProduct

    def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm) -> None:
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.feed_forward_norm = feed_forward_norm

    def parts(self):
        if self.feed_forward is None:
            return (self.mixer_norm, self.mixer)
        return (self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward)

    def forward(self, residual, delta, ctx, cache):
        x = run_norm(self.mixer_norm, residual, delta, ctx, consumer=self.mixer)
        a = self.mixer.forward(x, ctx, cache)
        if self.feed_forward is None:
            return a
        x = run_norm(self.feed_forward_norm, residual, a, ctx, consumer=self.feed_forward)
        return self.feed_forward.forward(x, ctx)


class SandwichBlock(Block):
    """A norm before and after each sub-layer: ``r += post1(mixer(pre1(r)))``, then
    ``r += post2(feed_forward(pre2(r)))``.  A sub-layer's output travels on as a
    :class:`~rapid_llm_amd.parts.lazy.NormedDelta`: the norm that runs next applies the pending
    post-norm, adds the result to the stream and computes its own rows in one kernel."""

    replayable = True
    accepts_deferred = True

    def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm, mixer_post_norm,
                 feed_forward_post_norm=None) -> None:
        if (feed_forward is None) != (feed_forward_post_norm is None):
            raise ValueError("a feed-forward and the norm behind it come together or not at all")
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.feed_forward_norm = feed_forward_norm
        self.mixer_post_norm = mixer_post_norm
        self.feed_forward_post_norm = feed_forward_post_norm

    def parts(self):
        if self.feed_forward is None:
            return (self.mixer_norm, self.mixer, self.mixer_post_norm)
        return (self.mixer_norm, self.mixer, self.mixer_post_norm,
                self.feed_forward_norm, self.feed_forward, self.feed_forward_post_norm)

    @staticmethod
    def _pending(norm, y):
        return NormedDelta(plain(y), norm.weight, norm.eps)

    def forward(self, residual, delta, ctx, cache):
        x = run_norm(self.mixer_norm, residual, delta, ctx)
        a = self._pending(self.mixer_post_norm, self.mixer.forward(x, ctx, cache))
        if self.feed_forward is None:
            return a
        x = run_norm(self.feed_forward_norm, residual, a, ctx)
        return self._pending(self.feed_forward_post_norm, self.feed_forward.forward(x, ctx))


class ParallelBlock(Block):
    """Both sub-layers read the same stream: ``r += mixer(norm1(r)) + feed_forward(norm2(r))``.
    Their outputs travel on as one pending :class:`~rapid_llm_amd.parts.lazy.SummedDeltas`; where
    the two norms can share their statistics (``pairs_with``) one kernel adds what is pending
    and writes both sub-layers' inputs."""

    replayable = True
    accepts_deferred = True

    def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm) -> None:
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.feed_forward_norm = feed_forward_norm

    def parts(self):
        if self.feed_forward is None:
            return (self.mixer_norm, self.mixer)
        return (self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward)

    def forward(self, residual, delta, ctx, cache):
        if self.feed_forward is None:
            x = run_norm(self.mixer_norm, residual, delta, ctx)
            return self.mixer.forward(x, ctx, cache)
        pairs = getattr(self.mixer_norm, "pairs_with", None)
        if pairs is not None and pairs(self.feed_forward_norm):
            x1, x2 = self.mixer_norm.forward(residual, delta, ctx, second=self.feed_forward_norm)
        else:
            x1 = plain(run_norm(self.mixer_norm, residual, delta, ctx))
            x2 = plain(run_norm(self.feed_forward_norm, residual, None, ctx))
        a = self.mixer.forward(x1, ctx, cache)
        b = self.feed_forward.forward(x2, ctx)
        return SummedDeltas(a, b)


BLOCKS.register("parallel", ParallelBlock)
BLOCKS.register("prenorm", PreNormBlock)
BLOCKS.register("sandwich", SandwichBlock)
