"""How token ids become rows of the residual stream, and how rows become logits."""

from ..ops import kernels
from ..weights.loader import MATRIX, TABLE, VECTOR, ParamSpec
from .base import Embedding, Head
from .registry import register_embedding, register_head


@register_embedding("lookup")
class TokenLookup(Embedding):
    """``h[t] = scale * table[id[t]] + position_table[pos[t]]`` in float
    (src/model/paged_decoder.py:306-314, where the scale is 1).  A token id may be "what the
    last step chose for row r", which the kernel reads from the device."""

    graph_safe = True

    def __init__(self, width: int, dtype, vocab_size: int, scale: float = 1.0):
        self.width = width
        self.dtype = dtype
        self.vocab_size = vocab_size
        self.scale = float(scale)

    def parameters(self):
        return {"table": ParamSpec((self.vocab_size, self.width), TABLE)}

    def forward(self, ctx, position_table, out):
        return kernels.embed(self.table, position_table, ctx.token_ids, ctx.positions, out,
                             token_src=ctx.token_src, carried=ctx.carried_tokens, scale=self.scale)


@register_head("linear")
class LinearHead(Head):
    """``logits = f W^T (+ b)`` in float.  Tied: ``W`` is the token table itself, not a copy,
    and there is no bias (src/model/paged_decoder.py:295-301,605)."""

    graph_safe = True

    def __init__(self, width: int, dtype, vocab_size: int, tied: bool = True, bias: bool = False):
        if tied and bias:
            raise ValueError("a head tied to the token table has no bias of its own")
        self.width = width
        self.dtype = dtype
        self.vocab_size = vocab_size
        self.tied = tied
        self.bias = bias
        self.weight = None
        self.packed = None
        self.bias_vector = None

    def parameters(self):
        params = {}
        if not self.tied:
            params["weight"] = ParamSpec((self.vocab_size, self.width), MATRIX)
        if self.bias:
            params["bias"] = ParamSpec((self.vocab_size,), VECTOR)
        return params

    def bind(self, tensors, embedding_table=None):
        self.weight = embedding_table if self.tied else tensors["weight"]
        if self.weight is None:
            raise ValueError("a tied head needs the token table")
        self.bias_vector = tensors.get("bias")
        self.packed = kernels.pack_decode_weight(self.weight)

    chooses_tokens = True

    def forward(self, x, logits, choose=None):
        if choose is None:
            kernels.linear(x, self.weight, self.bias_vector, logits, packed=self.packed)
            return False
        _, chosen = kernels.linear(x, self.weight, self.bias_vector, logits, packed=self.packed,
                                   choose=choose)
        return chosen
