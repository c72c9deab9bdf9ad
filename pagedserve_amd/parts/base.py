"""Interfaces of the parts that a layer is put together from.

A part is built from sizes and constants only, declares the parameters it needs
(``parameters``), receives them once (``bind``) and is then called with the step's
tensors.  It never sees the model's configuration.

* ``Norm.forward(h, out, rows=None)``: ``h`` is the float residual stream ``[T, d]``;
  writes the normed rows in the engine dtype.
* ``Norm.pending(h, scratch, rows=None)``: the same norm as an object that has not run
  yet (``ops.kernels.PendingNorm``); a part that sets ``accepts_pending_norm = True`` gets
  this instead of normed rows and may hand it to ``kernels.linear``, which runs norm and
  product as one launch where it can.  Other parts get the tensor.
* ``Mixer.forward(x, residual, ctx, cache)``: ``x`` is ``[T, d]`` in the engine dtype;
  the mixer ADDS its output to the float ``residual`` in place.  ``cache`` is the
  ``CacheView`` of this call of the layer: pools of a paged key/value entry, or the
  state tensor ``[max_slots, ...]`` of a mixer that declared a ``StateSpec``.
* ``FeedForward.forward(x, residual, ctx)``: same contract without a cache.
* ``Embedding.forward(ctx, position_table, out)`` fills the float stream from token ids;
  ``Head.forward(x, logits)`` turns the (normed) wanted rows into float logits.
* ``PositionEncoding``: ``embedding_table()`` is added to the token embedding when it
  is not ``None``; ``apply_to_qk(q, k, ctx)`` may transform queries and keys in place
  before they are cached (the default does nothing).

Folding the residual sum into the part lets the last matrix product of a part add
in float in its own epilogue instead of a separate pass over the stream.
"""

import itertools
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch

from ..weights.loader import ParamSpec


@dataclass(frozen=True)
class PagedKVSpec:
    """A mixer that caches keys and values of every (or the last ``window``) positions."""

    kv_heads: int
    head_dim: int
    window: int = 0
    value_dim: int = 0     # head size of the cached values where it is not the keys' (0: the same)


@dataclass(frozen=True)
class SlotStateSpec:
    """A mixer that keeps a fixed-size state per request."""

    shape: tuple
    dtype: torch.dtype = torch.float32


@dataclass
class CacheView:
    """What one call of a layer may touch in the cache."""

    entry: int
    writes: bool
    group: Optional[int] = None                # index of the cache group (paged entries)
    k_pool: Optional[torch.Tensor] = None      # [pages, kv_heads, page, head_dim]
    v_pool: Optional[torch.Tensor] = None      # [pages, kv_heads, page, value head size]
    state: Optional[torch.Tensor] = None       # [max_slots, ...]


class Part:
    # True when ``forward`` issues the same launches with the same arguments for every step
    # of one layout (it reads what differs between steps from the step's device tensors
    # only): such a step may be recorded once and replayed as a graph.  A part that looks at
    # host values of the step (``ctx.items``, lengths) must leave this False.
    graph_safe = False

    def parameters(self) -> Dict[str, ParamSpec]:
        return {}

    def bind(self, tensors: Dict[str, torch.Tensor]):
        """Receive the tensors that ``parameters`` named.  A part may derive further tensors
        from them here (the built-in ones keep a second copy of their matrices in a layout for
        decode steps): whoever changes a weight afterwards binds again."""
        for name in self.parameters():
            setattr(self, name.replace(".", "_"), tensors[name])


class Norm(Part):
    def forward(self, h, out, rows=None):
        raise NotImplementedError

    def pending(self, h, scratch, rows=None):
        """This norm of ``h`` as a ``PendingNorm``, or ``None`` if it can only run on its own."""
        return None


class PositionEncoding(Part):
    transforms_qk = False   # True when apply_to_qk changes queries or keys

    def embedding_table(self):
        return None

    def apply_to_qk(self, q, k, ctx):
        return None


class Embedding(Part):
    """``forward(ctx, position_table, out)`` fills the float stream ``out[T, d]`` from the
    step's token ids; ``table`` is the parameter that a tied head shares."""

    def forward(self, ctx, position_table, out):
        raise NotImplementedError


class Head(Part):
    """``forward(x, logits)`` writes float logits of the rows ``x`` (normed rows, or a pending
    norm if ``accepts_pending_norm``).  ``bind`` also receives the token table, which a tied
    head uses as its matrix."""

    accepts_pending_norm = True
    # True: ``forward`` takes ``choose=(kernels.TopChoice, tokens)`` and returns whether it
    # also wrote each row's most likely token into ``tokens`` (greedy decoding without a
    # sampling launch); the caller samples from the logits where it did not.
    chooses_tokens = False

    def bind(self, tensors, embedding_table=None):
        super().bind(tensors)

    def forward(self, x, logits):
        raise NotImplementedError


class Mixer(Part):
    accepts_pending_norm = False

    def cache_spec(self):
        """``PagedKVSpec``, ``SlotStateSpec`` or ``None``."""
        return None

    def set_position(self, position: PositionEncoding):
        self.position = position

    def forward(self, x, residual, ctx, cache: CacheView):
        raise NotImplementedError


class FeedForward(Part):
    accepts_pending_norm = False

    def forward(self, x, residual, ctx):
        raise NotImplementedError


_WORKSPACE_SERIALS = itertools.count(1)


def site_memo(store: dict, workspace) -> dict:
    """The memo of one call site of ``kernels.linear`` for the buffers of one workspace.  A
    memo holds addresses and the room behind them; another workspace may get the same
    addresses with other room (the allocator hands freed memory out again), so every workspace
    has memos of its own, told apart by a serial number that is never used twice."""
    memo = store.get(workspace.serial)
    if memo is None:
        if len(store) >= 8:
            store.clear()
        memo = store[workspace.serial] = {}
    return memo


class Workspace:
    """Activation buffers that live as long as the engine.

    ``rows(name, columns, dtype)`` returns a ``[max_rows, columns]`` tensor that is
    allocated on first use and never moves afterwards, so kernels captured in a HIP
    graph keep valid addresses.  Buffers are shared by all layers (they run one after
    the other)."""

    def __init__(self, max_rows: int, device):
        self.max_rows = max_rows
        self.device = torch.device(device)
        self._buffers: Dict[tuple, torch.Tensor] = {}
        # counts the buffers that were replaced by larger ones: whoever holds addresses
        # (recorded graphs) compares it with the value at the time of recording
        self.moved = 0
        self.serial = next(_WORKSPACE_SERIALS)
        self._views: Dict[tuple, torch.Tensor] = {}

    def rows(self, name: str, columns: int, dtype: torch.dtype, max_rows: Optional[int] = None):
        key = (name, columns, dtype, max_rows or self.max_rows)
        buffer = self._buffers.get(key)
        if buffer is None:
            buffer = torch.empty((max_rows or self.max_rows, columns), dtype=dtype, device=self.device)
            self._buffers[key] = buffer
        return buffer

    def first_rows(self, name: str, columns: int, dtype: torch.dtype, count: int):
        """``rows(name, columns, dtype)[:count]``, the same tensor object every time: a step of a
        layer asks for a handful of such views, and making a view costs the host as much as
        half a kernel launch."""
        key = (name, columns, dtype, count)
        view = self._views.get(key)
        if view is None:
            if len(self._views) > 4096:
                self._views.clear()
            view = self._views[key] = self.rows(name, columns, dtype)[:count]
        return view

    def column_views(self, name: str, columns: int, dtype: torch.dtype, count: int, cuts: tuple):
        """``first_rows(name, columns, dtype, count)`` and its pieces along the columns (``cuts``:
        the widths of the pieces), the same tensor objects every time and for every layer that
        asks with the same sizes."""
        key = (name, columns, dtype, count, cuts)
        views = self._views.get(key)
        if views is None:
            if len(self._views) > 4096:
                self._views.clear()
            whole = self.first_rows(name, columns, dtype, count)
            pieces, begin = [whole], 0
            for width in cuts:
                pieces.append(whole[:, begin:begin + width])
                begin += width
            views = self._views[key] = tuple(pieces)
        return views

    def flat(self, name: str, numel: int, dtype: torch.dtype):
        """A 1-D scratch buffer of at least ``numel`` elements; callers ask for their worst
        case so that it is allocated once."""
        key = (name, dtype)
        buffer = self._buffers.get(key)
        if buffer is None or buffer.numel() < numel:
            if buffer is not None:
                self.moved += 1
            buffer = torch.empty(numel, dtype=dtype, device=self.device)
            self._buffers[key] = buffer
        return buffer

    def bytes(self) -> int:
        return sum(buffer.numel() * buffer.element_size() for buffer in self._buffers.values())


@dataclass
class StepItem:
    """One request's share of a step (host side)."""

    request_id: object
    slot: int
    start: int      # position of its first token in the request
    count: int      # tokens in this step
    offset: int     # index of its first token in the step's flat token list


@dataclass
class StepContext:
    """Everything a part may read about the running step."""

    tokens: int
    dtype: torch.dtype
    device: torch.device
    items: List[StepItem]
    token_ids: torch.Tensor     # int32 [T]
    positions: torch.Tensor     # int32 [T]   position of each token in its request
    tok_item: torch.Tensor      # int32 [T]   index into ``items``
    cu_tokens: torch.Tensor     # int32 [items + 1]
    kv_lens: torch.Tensor       # int32 [items]  cached length after this step
    slots: torch.Tensor         # int32 [items]
    tables: List[torch.Tensor]  # per cache group: int32 [items, pages per request]
    page_size: int
    workspace: Workspace
    decode_only: bool = False   # every item brings exactly one token
    max_kv_len: int = 0         # longest cached length after this step (host value)
    single_tokens: Optional[torch.Tensor] = None   # int32: step indices of one-token items
    portion_tokens: Optional[torch.Tensor] = None  # int32: step indices of all other tokens
    max_positions: int = 0
    # For every tile size that a mixer asked for (``Mixer.query_tile``, one size or several):
    # the queries of the items with several tokens, cut into tiles of that many.  size -> (int32 item of each tile,
    # int32 first query of the tile within its item), the tiles that see the most keys first.
    query_tiles: Optional[Dict[int, tuple]] = None
    token_src: Optional[torch.Tensor] = None       # int32 [T]: >= 0: the token is carried_tokens[src]
    carried_tokens: Optional[torch.Tensor] = None  # int32: tokens that the last step chose
    extra: Optional[dict] = None
    # what ``kernels.linear`` and the attention calls leave for the same call of the next layer
    # (their ``shared``): lives for this step only
    shared_calls: dict = field(default_factory=dict)
