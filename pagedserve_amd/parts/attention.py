"""Multi-head attention over the paged cache."""

import torch

from ..ops import kernels
from ..weights.loader import MATRIX, VECTOR, ParamSpec
from .base import Mixer, PagedKVSpec, site_memo
from .registry import register_mixer


@register_mixer("attention")
class Attention(Mixer):
    """Packed QKV projection, cache write, attention over the request's cached keys,
    output projection added to the residual stream.

    One product gives ``[q | k | v]`` (src/model/paged_decoder.py:47-53); head ``j`` owns
    columns ``j*head_dim`` onward of each part (``:63-69``).  Keys and values of the
    step's tokens are stored before attention runs, so a token attends to itself and a
    prompt portion, a whole prompt and a decoded token are one case: every query at
    position p reads keys ``0..p`` (the last ``window`` of them) from the pages.
    ``scale`` multiplies the scores (``head_dim**-0.5`` in src/model/paged_attention.py:27).
    """

    graph_safe = True

    accepts_pending_norm = True

    # decoded tokens and prompt portions of one step in one attention launch where the kernel
    # takes the shape (``kernels.attention_mixed``)
    fuse_mixed = True

    # the step's index arrays list the queries of a prompt portion in tiles of these sizes (the
    # tiled kernel's three; ``kernels.attention_prefill`` checks them against the library's)
    query_tile = (kernels.PREFILL_TILE, kernels.PREFILL_SMALL_TILE, kernels.PREFILL_LARGE_TILE)

    def __init__(self, width: int, dtype, heads: int, kv_heads: int, head_dim: int, scale: float,
                 window: int = 0, bias: bool = True):
        if heads % kv_heads != 0:
            raise ValueError(f"heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
        if not 0 < head_dim <= 256:
            raise ValueError(f"head_dim {head_dim} must lie in 1..256")
        self.width = width
        self.dtype = dtype
        self.heads = heads
        self.kv_heads = kv_heads
        self.head_dim = head_dim
        self.scale = float(scale)
        self.window = int(window)
        self.bias = bias
        self.q_cols = heads * head_dim
        self.kv_cols = kv_heads * head_dim
        self.position = None
        # what ``kernels.linear`` keeps per call site and step shape (its ``memo``), per workspace
        self._memo_qkv, self._memo_out, self._memo_attention = {}, {}, {}

    def parameters(self):
        total = self.q_cols + 2 * self.kv_cols
        params = {
            "qkv.weight": ParamSpec((total, self.width), MATRIX),
            "out.weight": ParamSpec((self.width, self.q_cols), MATRIX),
        }
        if self.bias:
            params["qkv.bias"] = ParamSpec((total,), VECTOR)
            params["out.bias"] = ParamSpec((self.width,), VECTOR)
        return params

    def bind(self, tensors):
        self.qkv_weight = tensors["qkv.weight"]
        self.out_weight = tensors["out.weight"]
        self.qkv_bias = tensors.get("qkv.bias")
        self.out_bias = tensors.get("out.bias")
        # copies in the layout that the products of few rows (decode steps) read fastest
        self.qkv_packed = kernels.pack_decode_weight(self.qkv_weight)
        self.out_packed = kernels.pack_decode_weight(self.out_weight)
        self._memo_qkv.clear()
        self._memo_out.clear()
        self._memo_attention.clear()

    def cache_spec(self):
        return PagedKVSpec(self.kv_heads, self.head_dim, self.window)

    def forward(self, x, residual, ctx, cache):
        tokens = ctx.tokens
        total = self.q_cols + 2 * self.kv_cols
        # (the step's rows and their three column views, made once per row count for all layers)
        qkv, q, k, v = ctx.workspace.column_views("qkv", total, self.dtype, tokens,
                                                  (self.q_cols, self.kv_cols, self.kv_cols))
        tables = ctx.tables[cache.group]
        rotates = self.position is not None and self.position.transforms_qk
        if cache.writes and not rotates:
            # keys and values go to their pages from the product's own epilogue
            kernels.linear(x, self.qkv_weight, self.qkv_bias, qkv,
                           scatter=(cache.k_pool, cache.v_pool, ctx.tok_item, ctx.positions, tables,
                                    self.q_cols, self.kv_cols), packed=self.qkv_packed,
                           scatter_only=True, memo=site_memo(self._memo_qkv, ctx.workspace),
                           shared=ctx.shared_calls)
        else:
            kernels.linear(x, self.qkv_weight, self.qkv_bias, qkv, packed=self.qkv_packed,
                           memo=site_memo(self._memo_qkv, ctx.workspace),
                           shared=ctx.shared_calls)
            if rotates:
                self.position.apply_to_qk(q, k, ctx)
            if cache.writes:
                kernels.kv_write(k, v, cache.k_pool, cache.v_pool, ctx.tok_item, ctx.positions,
                                 tables)
        context = ctx.workspace.first_rows("attn", self.q_cols, self.dtype, tokens)
        singles = ctx.single_tokens.numel() if ctx.single_tokens is not None else 0
        if not kernels.decode_supported(self.head_dim):
            # a head size that the split-KV kernel does not take: every token, decoded ones
            # too, goes to the kernel that takes all sizes
            singles = 0
        merged_splits = 0
        if singles == tokens and kernels.merge_linear_supported(self.dtype, tokens, self.head_dim,
                                                                 self.out_packed):
            merged_splits = self._merged_splits(singles, ctx.max_kv_len)
        if merged_splits:
            # a decode step of few tokens over long contexts: the key ranges are merged inside
            # the output projection, which is split over the heads: no launch for the merge
            splits = merged_splits
            partial = self._range_records(ctx)
            kernels.attention_decode_partial(q, cache.k_pool, cache.v_pool, partial, ctx.tok_item,
                                             ctx.positions, tables, self.heads, self.scale, splits,
                                             window=self.window, waves=4)
            kernels.attention_merge_linear(partial, singles, self.heads, self.head_dim, splits,
                                           self.out_weight, self.out_packed, self.out_bias, residual)
            return
        tiled = singles < tokens and kernels.prefill_supported(self.dtype, self.head_dim, tables.shape[1])
        if singles and tiled and self._one_launch(singles, ctx, tables):
            # decoded tokens beside prompt portions: one launch whose blocks are of both kinds
            tile_item, tile_q0 = ctx.query_tiles[kernels.PREFILL_TILE]
            kernels.attention_mixed(q, cache.k_pool, cache.v_pool, context, ctx.single_tokens,
                                    ctx.tok_item, ctx.positions, tile_item, tile_q0, ctx.cu_tokens,
                                    ctx.kv_lens, tables, self.heads, self.scale, self.window,
                                    memo=site_memo(self._memo_attention, ctx.workspace),
                                    shared=ctx.shared_calls)
            kernels.linear(context, self.out_weight, self.out_bias, residual, epilogue="residual",
                           packed=self.out_packed, memo=site_memo(self._memo_out, ctx.workspace),
                       shared=ctx.shared_calls)
            return
        if singles:
            # one-token items: keys of a request are cut into ranges so that few requests
            # still fill the chip
            splits, waves = self._splits(singles, ctx.max_kv_len)
            partial = None
            if splits > 1:
                partial = self._range_records(ctx)
            # in a step of single tokens only, token t is item t: without the index the kernel
            # asks for its block table a trip to memory earlier (64 requests of 12 heads: 1.6 %
            # of the step).  The path above, of few blocks with one or two pages each, measured
            # 0.6 % slower with it, and so did a grid of more than four blocks per compute unit,
            # which waits for bytes and not for a trip (64 requests of 25 heads: 1 us a launch):
            # both keep the index.
            direct = (singles == tokens
                      and singles * self.heads * splits <= 4 * kernels.compute_units())
            kernels.attention_decode(q, cache.k_pool, cache.v_pool, context,
                                     None if direct else ctx.tok_item,
                                     ctx.positions, tables, self.heads, self.scale, splits,
                                     partial=partial, window=self.window, waves=waves,
                                     tok_list=None if singles == tokens else ctx.single_tokens)
        whole = singles == 0
        if tiled:
            size = kernels.PREFILL_TILE
            tile_item, tile_q0 = ctx.query_tiles[size]
            if kernels.prefill_small_tile_pays(self.heads, self.head_dim, tile_item.numel()):
                size = kernels.PREFILL_SMALL_TILE
                tile_item, tile_q0 = ctx.query_tiles[size]
            elif kernels.prefill_large_tile_pays(self.heads, self.head_dim,
                                                 ctx.query_tiles[kernels.PREFILL_LARGE_TILE][0].numel(),
                                                 ctx.max_kv_len):
                size = kernels.PREFILL_LARGE_TILE
                tile_item, tile_q0 = ctx.query_tiles[size]
            kernels.attention_prefill(q, cache.k_pool, cache.v_pool, context, tile_item,
                                      tile_q0, ctx.cu_tokens, ctx.kv_lens, tables,
                                      self.heads, self.scale, self.window,
                                      max_kv_len=ctx.max_kv_len, query_tile=size,
                                      memo=site_memo(self._memo_attention, ctx.workspace),
                                      shared=ctx.shared_calls)
        elif singles < tokens and kernels.tiled_f32_supported(self.dtype, self.head_dim):
            # 32-bit: tiles of queries too, on plain float arithmetic.  The tiles hold the items
            # of several tokens; one-token items that the split-KV kernel did not take (a head
            # size that it refuses) go to the kernel that takes all sizes
            tile_item, tile_q0 = ctx.query_tiles[kernels.PREFILL_TILE]
            if tile_item.numel():
                kernels.attention_tiled_f32(q, cache.k_pool, cache.v_pool, context, tile_item, tile_q0,
                                            ctx.cu_tokens, ctx.kv_lens, tables, self.heads, self.scale,
                                            self.window)
            if not singles and ctx.single_tokens is not None and ctx.single_tokens.numel():
                kernels.attention_rowwise(q, cache.k_pool, cache.v_pool, context, ctx.tok_item,
                                          ctx.positions, tables, self.heads, self.scale, self.window,
                                          tok_list=None if ctx.single_tokens.numel() == tokens
                                          else ctx.single_tokens)
        elif singles < tokens:
            kernels.attention_rowwise(q, cache.k_pool, cache.v_pool, context, ctx.tok_item,
                                      ctx.positions, tables, self.heads, self.scale, self.window,
                                      tok_list=None if whole else ctx.portion_tokens)
        kernels.linear(context, self.out_weight, self.out_bias, residual, epilogue="residual",
                       packed=self.out_packed, memo=site_memo(self._memo_out, ctx.workspace),
                       shared=ctx.shared_calls)

    def _one_launch(self, singles: int, ctx, tables) -> bool:
        """Whether a step's one-token items and its items of several tokens go to the kernel
        that runs both kinds of block in one grid: where it takes the shape, where the prompts
        are not so long that tiles of 128 queries are the better cut, and not where a handful
        of tokens is decoded over long contexts.  Its decode blocks are of four waves over all
        keys of a request, also where the decode kernel alone would run ranges or blocks of
        sixteen waves: beside the tiles' blocks they are not what the launch waits for (a
        portion of 512 beside 8 tokens over 900 keys: the step 0.978 against 1.005 ms at GPT-2
        small shape, 16 over 300 keys 0.90 against 0.99, 24 over 600 keys 0.97 against 1.08; at
        medium shape 16 over 900 keys 2.24 against 2.34), unless they are so few that their
        eight rounds of loads are (2 and 4 tokens over 900 keys: 0.956 against 0.946 and 0.974
        against 0.958 ms)."""
        if not (self.fuse_mixed and kernels.mixed_supported(self.dtype, self.head_dim, tables.shape[1])):
            return False
        visible = ctx.max_kv_len if self.window <= 0 else min(ctx.max_kv_len, self.window)
        if 4 * singles * self.heads < kernels.compute_units() and visible > 512:
            return False
        large_tiles = ctx.query_tiles[kernels.PREFILL_LARGE_TILE][0].numel()
        return not kernels.prefill_large_tile_pays(self.heads, self.head_dim, large_tiles, ctx.max_kv_len)

    def _range_records(self, ctx):
        """Scratch for one record per (token, head, key range): always asked for at its largest
        (both rules below keep tokens x heads x ranges under six blocks per compute unit beside
        one per pair), so that it never moves under the launches that recorded steps hold.
        Layers of equal heads and head size share one buffer; a layer of other sizes has its
        own, so that no layer makes another's grow."""
        worst = ((6 * kernels.compute_units() + ctx.workspace.max_rows * self.heads)
                 * (self.head_dim + 2))
        return ctx.workspace.flat(f"attn_partial_{self.heads}x{self.head_dim}", worst, torch.float32)

    def _merged_splits(self, count: int, max_kv_len: int) -> int:
        """Ranges per request for the path that merges them inside the output projection, or 0
        where the other path is as fast or faster: more (token, head) pairs than three quarters
        of the compute units (16 requests of 12 heads still gain 2 %), and, from half a pair
        per unit on, contexts that feed fewer than three ranges (16 requests over 100 keys:
        3 % slower).  Fewer pairs take this path at every length, also with a single range:
        the other path would cut 130 to 250 keys into two ranges and merge them with a launch
        of its own (1 to 4 requests over 20 to 250 keys: 5 % of the step, 8 requests 2 %).
        About three blocks of four waves per compute unit, never more ranges than the keys of
        the longest request can feed; and not where the projection's blocks would read more
        than 12 MB of records between them (wide models)."""
        visible = max_kv_len if self.window <= 0 else min(max_kv_len, self.window)
        pairs = count * self.heads
        units = kernels.compute_units()
        most = max(1, -(-visible // kernels.decode_keys_per_block(self.head_dim, 4)))
        if pairs > units * 3 // 4 or (most < 3 and 2 * pairs > units):
            return 0
        wanted = max(1, -(-3 * units // pairs))
        splits = min(most, wanted, 64)
        # Every block of 16 output columns merges the records of its head again: together they
        # read the records as often as the projection has column tiles, which grows with the
        # square of the heads.  Beyond some 12 MB of that the other path is ahead (decode steps
        # over 1,024 keys, merged against not: 8 requests of 16 heads, 12.3 MB, 0.837 against
        # 0.821 ms; 4 of 25 heads, 21 MB, 2.089 against 1.995; under it 4 requests of 16 heads
        # 0.724 against 0.771, 2 of 25 heads 1.903 against 1.951, 16 of 12 heads 2 % ahead).
        tiles = -(-self.width // 16)
        if tiles * pairs * splits * (self.head_dim + 2) * 4 > 12_000_000:
            return 0
        return splits

    def _splits(self, count: int, max_kv_len: int):
        """(ranges per request, waves per block) of the decode kernel, by the number of (token,
        head) pairs per compute unit and the keys that a query sees:

        * from three and a half pairs per unit: one block of 4 waves per pair fills the chip;
        * from one and a half: the same at short contexts; from 2,048 keys on a handful of long
          blocks per unit would leave units idle towards the end, so the keys are cut into
          ranges until six blocks come to a unit;
        * between one and one and a half: blocks of 16 waves would come two to some units and
          one to the others, and the kernel would last as long as the units with two (24
          requests of 12 heads at 1,000 keys: 22.3 us): ranges of 4-wave blocks, four blocks to a
          unit (19.0 us with the launch that merges them), six over thousands of keys;
        * up to one pair per unit: one block of 16 waves takes a whole request's keys and no
          second launch is needed (two or three such blocks per request while each still has
          a unit of its own); just under a pair per unit and from 4,096 keys on, ranges of
          4-wave blocks are ahead again;
        * few pairs: ranges of 4-wave blocks until four blocks come to a unit.

        Never more ranges than the keys of the longest request can feed, and never more than
        six blocks per unit beside one per pair (the scratch for the records is sized for
        that)."""
        visible = max_kv_len if self.window <= 0 else min(max_kv_len, self.window)
        pairs = count * self.heads
        units = kernels.compute_units()
        if 2 * pairs >= 7 * units:
            return 1, 4
        if pairs >= units + units // 2:
            # One block of 4 waves per pair fills the chip at short contexts.  At long ones a
            # handful of blocks per unit, each walking thousands of keys, leaves units idle
            # towards the end: ranges until six blocks come to a unit (32 requests of 12 heads
            # at 8,192 keys: 126 instead of 172 us), none under 2,048 keys.
            return max(1, min(-(-6 * units // pairs), visible // 1024)), 4
        if pairs > units:
            # (four blocks to a unit, six over thousands of keys)
            blocks = (6 if visible >= 4096 else 4) * units
            return max(1, min(-(-blocks // pairs), visible // 256)), 4
        if 4 * pairs >= 3 * units and visible >= 4096:
            # nearly a pair per unit over thousands of keys: six blocks of 4 waves to a unit are
            # ahead of one block of 16 waves per pair (17 requests of 12 heads at 4,096 keys:
            # 41.4 against 44.2 us, at 16,384 keys 141 against 155)
            return min(-(-6 * units // pairs), 64), 4
        if pairs >= units // 4 and visible > kernels.decode_keys_per_block(self.head_dim, 4):
            # contexts of several thousand keys: two or three such blocks per request, as
            # long as every block still has a compute unit of its own
            return max(1, min(units // pairs, visible // 1024)), 16
        most = max(1, -(-visible // kernels.decode_keys_per_block(self.head_dim, 4)))
        wanted = max(1, -(-4 * units // pairs))
        return min(most, wanted, 64), 4
