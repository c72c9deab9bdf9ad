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

    @property
    def graph_safe(self):
        """The arrangement itself looks at no host value of the step; its parts decide."""
        return all(getattr(part, "graph_safe", False) for part in self.parts().values())

    def parts(self):
        return {"norm1": self.norm1, "mixer": self.mixer, "norm2": self.norm2,
                "feed_forward": self.feed_forward}

    def _normed(self, norm, part, h, ctx):
        """Input of ``part``: the norm as a pending object if the part takes one, else rows."""
        scratch = ctx.workspace.rows("normed", self.width, self.dtype)[:ctx.tokens]
        if getattr(part, "accepts_pending_norm", False):
            pending = norm.pending(h, scratch)
            if pending is not None:
                return pending
        return norm.forward(h, scratch)

    def forward(self, h, ctx, cache):
        self.mixer.forward(self._normed(self.norm1, self.mixer, h, ctx), h, ctx, cache)
        self.feed_forward.forward(self._normed(self.norm2, self.feed_forward, h, ctx), h, ctx)
        return h
