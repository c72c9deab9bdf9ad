"""Norms over the float residual stream; statistics are always 32-bit."""

from ..ops import kernels
from ..weights.loader import VECTOR, ParamSpec
from .base import Norm
from .registry import register_norm


@register_norm("layernorm")
class LayerNorm(Norm):
    """(h - mean) / sqrt(var + eps) * gamma + beta with the biased variance
    (src/model/paged_decoder.py:170-177; src/kernels/triton_residual_layernorm.py:25-39)."""

    graph_safe = True

    def __init__(self, width: int, dtype, eps: float):
        self.width = width
        self.dtype = dtype
        self.eps = float(eps)

    def parameters(self):
        return {"gamma": ParamSpec((self.width,), VECTOR), "beta": ParamSpec((self.width,), VECTOR)}

    def forward(self, h, out, rows=None):
        return kernels.norm(h, self.gamma, self.beta, self.eps, out, rows=rows, rms=False)

    def pending(self, h, scratch, rows=None):
        return kernels.PendingNorm(h, self.gamma, self.beta, self.eps, False, scratch, rows)


@register_norm("rmsnorm")
class RMSNorm(Norm):
    """h / sqrt(mean(h^2) + eps) * gamma.  Not used by GPT-2; the kernel's second mode."""

    graph_safe = True

    def __init__(self, width: int, dtype, eps: float):
        self.width = width
        self.dtype = dtype
        self.eps = float(eps)

    def parameters(self):
        return {"gamma": ParamSpec((self.width,), VECTOR)}

    def forward(self, h, out, rows=None):
        return kernels.norm(h, self.gamma, None, self.eps, out, rows=rows, rms=True)

    def pending(self, h, scratch, rows=None):
        return kernels.PendingNorm(h, self.gamma, None, self.eps, True, scratch, rows)
