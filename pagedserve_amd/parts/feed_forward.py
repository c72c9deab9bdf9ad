"""Feed-forward parts."""

from ..ops import kernels
from ..weights.loader import MATRIX, VECTOR, ParamSpec
from .base import FeedForward, site_memo
from .registry import register_feed_forward

ACTIVATIONS = ("gelu_tanh", "gelu_erf")


@register_feed_forward("dense")
class DenseFeedForward(FeedForward):
    """``residual += act(x W_up + b_up) W_down + b_down``
    (src/model/paged_decoder.py:178-179,224-228; activations ``:273-280``)."""

    graph_safe = True

    accepts_pending_norm = True

    def __init__(self, width: int, dtype, inner: int, activation: str, bias: bool = True):
        if activation not in ACTIVATIONS:
            raise ValueError(f"unknown activation {activation!r}; known: {', '.join(ACTIVATIONS)}")
        self.width = width
        self.dtype = dtype
        self.inner = inner
        self.activation = activation
        self.bias = bias
        self._memo_up, self._memo_down = {}, {}

    def parameters(self):
        params = {
            "up.weight": ParamSpec((self.inner, self.width), MATRIX),
            "down.weight": ParamSpec((self.width, self.inner), MATRIX),
        }
        if self.bias:
            params["up.bias"] = ParamSpec((self.inner,), VECTOR)
            params["down.bias"] = ParamSpec((self.width,), VECTOR)
        return params

    def bind(self, tensors):
        self.up_weight = tensors["up.weight"]
        self.down_weight = tensors["down.weight"]
        self.up_bias = tensors.get("up.bias")
        self.down_bias = tensors.get("down.bias")
        # copies in the layout that the products of few rows (decode steps) read fastest
        self.up_packed = kernels.pack_decode_weight(self.up_weight)
        self.down_packed = kernels.pack_decode_weight(self.down_weight)
        self._memo_up.clear()
        self._memo_down.clear()

    def forward(self, x, residual, ctx):
        hidden = ctx.workspace.first_rows("ffn", self.inner, self.dtype, ctx.tokens)
        # (the hidden rows belong to these two calls alone: at 17 to 64 rows the first may leave
        # them in the order in which the second reads them)
        _, hidden_packed = kernels.linear(x, self.up_weight, self.up_bias, hidden,
                                          epilogue=self.activation, packed=self.up_packed,
                                          packed_out=True, memo=site_memo(self._memo_up, ctx.workspace),
                                          shared=ctx.shared_calls)
        kernels.linear(hidden, self.down_weight, self.down_bias, residual, epilogue="residual",
                       packed=self.down_packed, a_packed=hidden_packed, memo=site_memo(self._memo_down, ctx.workspace),
                       shared=ctx.shared_calls)
