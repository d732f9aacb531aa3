"""Arrangements of a layer's parts around the residual stream."""
from .. import debug
from .base import Block, Stream, register_block


@register_block("pre_norm")
class PreNormBlock(Block):
    """`x = x + mixer(norm(x))`, `x = x + feed_forward(norm(x))`
    (reference: opt/model.py:351-375). The sums are made in float32 by the
    last matrix product of each part."""

    recordable = True

    def forward(self, stream: Stream, ctx, cache) -> Stream:
        _, h = self.mixer_norm.forward(stream.x, False, True)
        x = debug.tap("after_mixer", self.mixer.forward(h, ctx, cache, stream.x))
        _, h = self.feed_forward_norm.forward(x, False, True)
        x = self.feed_forward.forward(h, ctx, x)
        return Stream(x, None)


@register_block("post_norm")
class PostNormBlock(Block):
    """`x = norm(x + mixer(x))`, `x = norm(x + feed_forward(x))`: the norm follows
    each sum, and its output is the stream."""

    recordable = True

    reads_compute_copy = True      # the mixer reads the stream itself, in the compute dtype

    def forward(self, stream: Stream, ctx, cache) -> Stream:
        h = stream.compute if stream.compute is not None else self.mixer_norm.ops.cast(stream.x, self.mixer_norm.dtype)
        t = self.mixer.forward(h, ctx, cache, stream.x)
        x, h = self.mixer_norm.forward(t, True, True)
        debug.tap("after_mixer", x)
        t = self.feed_forward.forward(h, ctx, x)
        x, h = self.feed_forward_norm.forward(t, True, True)
        return Stream(x, h)
