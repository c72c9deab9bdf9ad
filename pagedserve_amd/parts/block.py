"""Arrangements of parts in a block.

An arrangement says which named parts it is made of and what each is (``roles``: name ->
``"norm"``, ``"mixer"`` or ``"feed_forward"``, the registry its kind is looked up in), and in
which order they run; ``mixer`` is the part whose ``cache_spec`` decides what the block's cache
entry holds.  The model builds the parts that the block's spec names and hands them
over as a dict; an arrangement with another number of parts declares other roles."""

from .registry import register_arrangement


@register_arrangement("pre_norm")
class PreNormBlock:
    """``h += mixer(norm1(h))`` then ``h += feed_forward(norm2(h))``
    (src/model/paged_decoder.py:181-189,210-228)."""

    roles = {"norm1": "norm", "mixer": "mixer", "norm2": "norm", "feed_forward": "feed_forward"}

    def __init__(self, width, dtype, parts):
        self.width = width
        self.dtype = dtype
        self._parts = dict(parts)
        self.norm1 = parts["norm1"]
        self.mixer = parts["mixer"]
        self.norm2 = parts["norm2"]
        self.feed_forward = parts["feed_forward"]

    @property
    def graph_safe(self):
        """The arrangement itself looks at no host value of the step; its parts decide."""
        return all(getattr(part, "graph_safe", False) for part in self.parts().values())

    def parts(self):
        return dict(self._parts)

    def _normed(self, norm, part, h, ctx):
        """Input of ``part``: the norm as a pending object if the part takes one, else rows."""
        scratch = ctx.workspace.first_rows("normed", self.width, self.dtype, ctx.tokens)
        if getattr(part, "accepts_pending_norm", False):
            pending = norm.pending(h, scratch)
            if pending is not None:
                return pending
        return norm.forward(h, scratch)

    def forward(self, h, ctx, cache):
        self.mixer.forward(self._normed(self.norm1, self.mixer, h, ctx), h, ctx, cache)
        self.feed_forward.forward(self._normed(self.norm2, self.feed_forward, h, ctx), h, ctx)
        return h
