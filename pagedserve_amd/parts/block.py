"""Arrangements of parts in a block."""

from .registry import register_arrangement


@register_arrangement("pre_norm")
class PreNormBlock:
    """``h += mixer(norm1(h))`` then ``h += feed_forward(norm2(h))``
    (src/model/paged_decoder.py:181-189,210-228)."""

    def __init__(self, width, dtype, norm1, mixer, norm2, feed_forward):
        self.width = width
        self.dtype = dtype
        self.norm1 = norm1
        self.mixer = mixer
        self.norm2 = norm2
        self.feed_forward = feed_forward

    def parts(self):
        return {"norm1": self.norm1, "mixer": self.mixer, "norm2": self.norm2,
                "feed_forward": self.feed_forward}

    def forward(self, h, ctx, cache):
        normed = ctx.workspace.rows("normed", self.width, self.dtype)[:ctx.tokens]
        self.norm1.forward(h, normed)
        self.mixer.forward(normed, h, ctx, cache)
        self.norm2.forward(h, normed)
        self.feed_forward.forward(normed, h, ctx)
        return h
