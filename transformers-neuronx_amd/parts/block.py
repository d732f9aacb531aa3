"""Arrangements of a layer's parts around the residual stream."""
from .. import debug
from .base import Block, Stream, register_block


@register_block("pre_norm")
class PreNormBlock(Block):
    """`x = x + mixer(norm(x))`, `x = x + feed_forward(norm(x))`
    (reference: opt/model.py:351-375). The sums are made in float32 by the
    last matrix product of each part."""

    recordable = True

    fold_mixer_norm = fold_feed_forward_norm = False

    def after_load(self) -> None:
        # Each norm's output goes to one part only; where that part does nothing with it but one matrix
        # product, the backend may do the norm inside the product (the few-rows products of decode steps:
        # one launch less for each half of a layer).
        w = self.mixer.first_weight()
        self.fold_mixer_norm = w is not None and self.mixer_norm.fold_into(w)
        w = self.feed_forward.first_weight()
        self.fold_feed_forward_norm = w is not None and self.feed_forward_norm.fold_into(w)

    def forward(self, stream: Stream, ctx, cache) -> Stream:
        h = (self.mixer_norm.deferred(stream.x) if self.fold_mixer_norm
             else self.mixer_norm.forward(stream.x, False, True)[1])
        x = debug.tap("after_mixer", self.mixer.forward(h, ctx, cache, stream.x))
        h = (self.feed_forward_norm.deferred(x) if self.fold_feed_forward_norm
             else self.feed_forward_norm.forward(x, False, True)[1])
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
