"""Block arrangements.  "prenorm": h += mixer(norm(h)); h += feed_forward(norm(h))
(src/arch/llama.rs:152-170).  Another arrangement (one norm for two parallel
halves, norms after the parts) is another subclass of `Block`, registered under
its own name; the parts it needs beyond these four come under the names the
layer's spec gives them in `extra`.  "sandwich": a norm before and after each half.
"parallel": both halves read the stream as it was, each through a norm of its own or both through the one norm the
layer has."""
from __future__ import annotations

import torch

from .base import Block, register_block


class PreNormBlock(Block):
    def __init__(self, named):
        super().__init__(named)
        if self.feed_forward is not None and self.feed_forward_norm is None:
            raise ValueError("block arrangement PreNormBlock needs the parts feed_forward_norm")

    needs = ("mixer", "mixer_norm")      # a layer may have no feed-forward; one that has needs its norm too
    keeps_left_current = True       # `normed_input` drops what was left before each part; the feed-forward runs last

    def first_norm(self):
        return self.mixer_norm

    def forward(self, ctx, h, cache):
        after = ctx.norm_after_block
        if self.feed_forward is None:
            self.mixer.forward(ctx, self.normed_input(ctx, h, self.mixer_norm, self.mixer, after), h, cache)
            ctx.upcoming_norm = None
            return
        self.mixer.forward(ctx, self.normed_input(ctx, h, self.mixer_norm, self.mixer, self.feed_forward_norm), h, cache)
        self.feed_forward.forward(ctx, self.normed_input(ctx, h, self.feed_forward_norm, self.feed_forward, after), h)
        ctx.upcoming_norm = None


register_block("prenorm", PreNormBlock)


class SandwichBlock(Block):
    """A norm before and after each sublayer: h += post_mixer_norm(mixer(mixer_norm(h))), then, where the layer has a
    feed-forward, h += post_feed_forward_norm(feed_forward(feed_forward_norm(h))).  The sublayer adds its result into
    a cleared 32-bit buffer of the stream's shape; the norm after it reads that and adds into the stream, in 32-bit."""
    needs = ("mixer", "mixer_norm", "post_mixer_norm")

    def __init__(self, named):
        super().__init__(named)
        self.post_mixer_norm = self.named["post_mixer_norm"]
        self.post_feed_forward_norm = self.named.get("post_feed_forward_norm")
        if self.feed_forward is not None and (self.feed_forward_norm is None or self.post_feed_forward_norm is None):
            raise ValueError("a feed-forward between two norms needs both of them")

    def _half(self, ctx, h, norm, post, run) -> None:
        T, D = h.shape
        x = ctx.workspace("block.x", (T, D), self.mixer.dtype)
        y = ctx.workspace("block.y", (T, D), torch.float32)
        ctx.note_left(h, None)
        ctx.upcoming_norm = None
        norm.forward_clearing(ctx, h, x, y)
        run(x, y)
        post.add_normed(ctx, y, h)

    def forward(self, ctx, h, cache):
        self._half(ctx, h, self.mixer_norm, self.post_mixer_norm, lambda x, y: self.mixer.forward(ctx, x, y, cache))
        if self.feed_forward is not None:
            self._half(ctx, h, self.feed_forward_norm, self.post_feed_forward_norm, lambda x, y: self.feed_forward.forward(ctx, x, y))
        ctx.note_left(h, None)
        ctx.upcoming_norm = None


register_block("sandwich", SandwichBlock)


class ParallelBlock(Block):
    """Both halves read the same stream and both add into it: h <- h + mixer(mixer_norm(h)) + feed_forward(n(h)), where
    n is the feed-forward's own norm or, for a layer that has one norm only, the mixer's: then both halves read the same
    normed rows.  The norms run before either half touches the stream (two in one launch where the norms can:
    `forward_with`); the sums are 32-bit.  A layer may have no feed-forward."""
    needs = ("mixer", "mixer_norm")

    def forward(self, ctx, h, cache):
        T, D = h.shape
        ctx.note_left(h, None)
        ctx.upcoming_norm = None
        x = ctx.workspace("block.x", (T, D), self.mixer.dtype)
        if self.feed_forward is None or self.feed_forward_norm is None:
            self.mixer_norm.forward(ctx, h, x)
            self.mixer.forward(ctx, x, h, cache)
            if self.feed_forward is not None:
                self.feed_forward.forward(ctx, x, h)
        else:
            x2 = ctx.workspace("block.x2", (T, D), self.feed_forward.dtype)
            together = getattr(self.mixer_norm, "forward_with", None)
            if together is None or not together(ctx, h, x, self.feed_forward_norm, x2):
                self.mixer_norm.forward(ctx, h, x)
                self.feed_forward_norm.forward(ctx, h, x2)
            self.mixer.forward(ctx, x, h, cache)
            self.feed_forward.forward(ctx, x2, h)
        ctx.note_left(h, None)
        ctx.upcoming_norm = None


register_block("parallel", ParallelBlock)
