"""Each kernel of a decode step and of a prefill step alone, timed the way the step meets it.

A kernel is launched ``copies`` times inside one HIP graph, each launch on its own copy of the
weights (so many copies that neither the L2 caches nor the memory-side cache hold the next
one: a model step walks through all layers' matrices and finds none of them in a cache), the
graph is replayed until at least 100 launches have been timed after at least 25 untimed ones,
and the mean time of a launch is reported with the bytes it has to move, its flops, and both
as fractions of the published and of the measured peak.  (Timing method after the reference's
benchmark_paged_attention.py:33-44 and benchmark.py:63-89: warm-up, then events around the
timed iterations.)

Launch shapes (key ranges of decode attention, the merge inside the output projection) are
chosen by the same rules as in the engine: the attention part is asked.
"""

import math

import torch

from ..ops import kernels
from ..parts.attention import Attention

HBM_GBPS = 8000.0          # MI355X, published
PEAK_TFLOPS = 2500.0       # dense bf16 MFMA, published
ROTATE_BYTES = 600e6       # weights that the copies of one kernel cover together


def graph_time(launch, copies, timed_launches=100, warm_launches=25):
    """Mean microseconds of ``launch(i)`` over a graph of ``copies`` launches (i = 0 ..)."""
    for i in range(max(copies, warm_launches)):
        launch(i % copies)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with kernels.on_stream(side):
            with torch.cuda.graph(graph, stream=side):
                for i in range(copies):
                    launch(i)
    graph.replay()
    torch.cuda.synchronize()
    rounds = max(1, -(-timed_launches // copies))
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(rounds):
        graph.replay()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) * 1e3 / (rounds * copies)


def measured_peaks():
    """What this device gives to the simplest programs: a copy of 1 GiB (read + write) and a
    bfloat16 product of 4096 cubed by the vendor library."""
    source = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
    target = torch.empty_like(source)
    copy_us = graph_time(lambda i: target.copy_(source), 4, timed_launches=20, warm_launches=4)
    a = torch.randn(4096, 4096, device="cuda").bfloat16()
    b = torch.randn(4096, 4096, device="cuda").bfloat16()
    c = torch.empty(4096, 4096, device="cuda", dtype=torch.bfloat16)
    product_us = graph_time(lambda i: torch.matmul(a, b, out=c), 10, timed_launches=50, warm_launches=10)
    del source, target
    torch.cuda.empty_cache()
    return {"copy_GBps": round(2 * 4 * (1 << 28) / copy_us / 1e3, 1),
            "product_4096_TFLOPs": round(2 * 4096 ** 3 / product_us / 1e6, 1)}


class _Shape:
    def __init__(self, raw):
        self.d = raw["n_embd"]
        self.heads = raw["n_head"]
        self.head_dim = self.d // self.heads
        self.inner = raw["n_inner"]
        self.vocab = raw["vocab_size"]
        self.positions = raw["n_positions"]
        self.eps = raw["layer_norm_epsilon"]
        self.activation = "gelu_tanh" if raw["activation_function"] != "gelu" else "gelu_erf"


def _copies(bytes_each, least=4, most=96):
    return int(max(least, min(most, math.ceil(ROTATE_BYTES / max(bytes_each, 1)))))


def _matrices(n, k, copies, seed):
    generator = torch.Generator(device="cuda").manual_seed(seed)
    weights, packed = [], []
    for _ in range(copies):
        w = (torch.randn(n, k, device="cuda", generator=generator) * k ** -0.5).bfloat16()
        weights.append(w)
        packed.append(kernels.pack_decode_weight(w))
    return weights, packed


def _row(name, us, bytes_moved, flops, peaks, launches=1):
    gbps = bytes_moved / us / 1e3
    tflops = flops / us / 1e6
    return {"kernel": name, "us": round(us, 2), "launches": launches, "MB": round(bytes_moved / 1e6, 3),
            "GFLOP": round(flops / 1e9, 3), "GBps": round(gbps, 1), "TFLOPs": round(tflops, 1),
            "of_hbm": round(gbps / HBM_GBPS, 4), "of_mfma": round(tflops / PEAK_TFLOPS, 4),
            "of_measured_copy": round(gbps / peaks["copy_GBps"], 4),
            "of_measured_product": round(tflops / peaks["product_4096_TFLOPs"], 4)}


def decode_table(raw, rows, context, peaks, page_size=16, only=None):
    """The kernels of one layer of a decode step of ``rows`` requests over ``context`` keys,
    and of the step's ends (embedding, final norm + head, token choice), bfloat16."""
    shape = _Shape(raw)
    d, inner, heads, head_dim = shape.d, shape.inner, shape.heads, shape.head_dim
    dtype = torch.bfloat16
    generator = torch.Generator(device="cuda").manual_seed(1)

    def randn(*size, scale=1.0, kind=torch.float32):
        return (torch.randn(*size, device="cuda", generator=generator) * scale).to(kind)

    h = randn(rows, d)
    gamma, beta = randn(d) * 0.1 + 1, randn(d) * 0.1
    normed = torch.empty(max(rows, 64), d, dtype=dtype, device="cuda")
    qkv = torch.empty(rows, 3 * d, dtype=dtype, device="cuda")
    context_rows = torch.empty(rows, d, dtype=dtype, device="cuda")
    hidden = torch.empty(max(rows, 64), inner, dtype=dtype, device="cuda")
    pages_each = -(-context // page_size)
    table_width = -(-shape.positions // page_size)
    tables = torch.zeros(rows, table_width, dtype=torch.int32, device="cuda")
    tables[:, :pages_each] = torch.arange(rows * pages_each, dtype=torch.int32, device="cuda").view(rows, pages_each)
    positions = torch.full((rows,), context - 1, dtype=torch.int32, device="cuda")
    tok_item = torch.arange(rows, dtype=torch.int32, device="cuda")
    cache_copies = _copies(2 * rows * pages_each * page_size * d * 2, least=2, most=24)
    pools = [(randn(rows * pages_each, heads, page_size, head_dim, kind=dtype),
              randn(rows * pages_each, heads, page_size, head_dim, kind=dtype)) for _ in range(cache_copies)]
    part = Attention(width=d, dtype=dtype, heads=heads, kv_heads=heads, head_dim=head_dim,
                     scale=head_dim ** -0.5)
    out = []

    def wanted(name):
        return only is None or any(piece in name for piece in only)

    def product(name, n, k, call, seed, extra_bytes=0):
        if not wanted(name):
            return
        copies = _copies(n * k * 2)
        weights, packed = _matrices(n, k, copies, seed)
        bias = randn(n) * 0.1
        us = graph_time(lambda i: call(weights[i], packed[i], bias, i), copies)
        out.append(_row(name, us, n * k * 2 + extra_bytes, 2 * rows * n * k, peaks))
        del weights, packed
        torch.cuda.empty_cache()

    # norm + QKV + cache write
    def qkv_call(w, wp, bias, i):
        k_pool, v_pool = pools[i % cache_copies]
        kernels.linear(kernels.PendingNorm(h, gamma, beta, shape.eps, False, normed), w, bias, qkv,
                       scatter=(k_pool, v_pool, tok_item, positions, tables, d, d), packed=wp,
                       scatter_only=True)
    product("norm+qkv+cache_write", 3 * d, d, qkv_call, 11, extra_bytes=rows * d * 4)

    # attention over the cache (+ output projection where the merge runs inside it)
    merged = 0
    if kernels.merge_linear_supported(dtype, rows, head_dim, True):
        merged = part._merged_splits(rows, context)
    cache_bytes = 2 * rows * context * d * 2
    worst = (6 * kernels.compute_units() + rows * heads) * (head_dim + 2)
    partial = torch.empty(worst, dtype=torch.float32, device="cuda")
    q = qkv[:, :d]
    q.copy_(randn(rows, d, kind=dtype))
    if merged:
        if wanted("attention"):
            us = graph_time(lambda i: kernels.attention_decode_partial(
                q, pools[i % cache_copies][0], pools[i % cache_copies][1], partial, tok_item, positions,
                tables, heads, part.scale, merged, waves=4), cache_copies)
            out.append(_row(f"attention (records of {merged} key ranges)", us, cache_bytes,
                            4 * rows * context * d, peaks))

        def merge_call(w, wp, bias, i):
            kernels.attention_merge_linear(partial, rows, heads, head_dim, merged, w, wp, bias, h)
        product("merge+out_proj+residual", d, d, merge_call, 12,
                extra_bytes=rows * heads * merged * (head_dim + 2) * 4)
    else:
        splits, waves = part._splits(rows, context)
        direct = rows * heads * splits <= 4 * kernels.compute_units()
        if wanted("attention"):
            us = graph_time(lambda i: kernels.attention_decode(
                q, pools[i % cache_copies][0], pools[i % cache_copies][1], context_rows,
                None if direct else tok_item, positions, tables, heads, part.scale, splits,
                partial=partial if splits > 1 else None, waves=waves), cache_copies)
            out.append(_row(f"attention ({splits} key ranges, {waves} waves)", us, cache_bytes,
                            4 * rows * context * d, peaks, launches=2 if splits > 1 else 1))

        def out_call(w, wp, bias, i):
            kernels.linear(context_rows, w, bias, h, epilogue="residual", packed=wp)
        product("out_proj+residual", d, d, out_call, 12)

    # norm + FC + activation, projection + residual
    state = {}

    def fc_call(w, wp, bias, i):
        _, state["packed"] = kernels.linear(kernels.PendingNorm(h, gamma, beta, shape.eps, False, normed),
                                            w, bias, hidden[:rows], epilogue=shape.activation, packed=wp,
                                            packed_out=True)
    product("norm+fc+gelu", inner, d, fc_call, 13, extra_bytes=rows * d * 4)
    if "packed" not in state:
        fc_w, fc_p = _matrices(inner, d, 1, 13)
        fc_call(fc_w[0], fc_p[0], randn(inner), 0)

    def proj_call(w, wp, bias, i):
        kernels.linear(hidden[:rows], w, bias, h, epilogue="residual", packed=wp, a_packed=state["packed"])
    product("proj+residual", d, inner, proj_call, 14)

    # the ends of the step
    if wanted("embed"):
        table = randn(shape.vocab, d, kind=dtype)
        pos_table = randn(shape.positions, d, kind=dtype)
        ids = torch.randint(0, shape.vocab, (rows,), device="cuda", dtype=torch.int32)
        us = graph_time(lambda i: kernels.embed(table, pos_table, ids, positions, h), 8)
        out.append(_row("embed", us, rows * d * 8, 0, peaks))
        del table, pos_table
    if wanted("head"):
        logits = torch.empty(rows, -(-shape.vocab // 8) * 8, dtype=torch.float32, device="cuda")[:, :shape.vocab]
        tokens = torch.zeros(rows, dtype=torch.int32, device="cuda")
        top = kernels.TopChoice(64, "cuda")
        final = torch.empty(rows, d, dtype=dtype, device="cuda")
        chose = {}

        def head_call(w, wp, bias, i):
            _, chose["head"] = kernels.linear(kernels.PendingNorm(h, gamma, beta, shape.eps, False, final),
                                              w, None, logits, packed=wp, choose=(top, tokens))
        product("final_norm+head" , shape.vocab, d, head_call, 15, extra_bytes=rows * shape.vocab * 4)
        if out and not chose.get("head", True):
            out[-1]["kernel"] += " (tokens chosen by the sampling kernel)"
        if wanted("sample"):
            us = graph_time(lambda i: kernels.sample(logits, None, None, tokens), 8)
            out.append(_row("sample (greedy)", us, rows * shape.vocab * 4, 0, peaks))
    torch.cuda.empty_cache()
    return out


def prefill_table(raw, prompts, length, peaks, page_size=16, only=None):
    """The kernels of one layer of a prefill step of ``prompts`` whole prompts of ``length``."""
    shape = _Shape(raw)
    d, inner, heads, head_dim = shape.d, shape.inner, shape.heads, shape.head_dim
    dtype = torch.bfloat16
    rows = prompts * length
    generator = torch.Generator(device="cuda").manual_seed(2)

    def randn(*size, scale=1.0, kind=torch.float32):
        return (torch.randn(*size, device="cuda", generator=generator) * scale).to(kind)

    h = randn(rows, d)
    gamma, beta = randn(d) * 0.1 + 1, randn(d) * 0.1
    normed = torch.empty(rows, d, dtype=dtype, device="cuda")
    qkv = torch.empty(rows, 3 * d, dtype=dtype, device="cuda")
    context_rows = torch.empty(rows, d, dtype=dtype, device="cuda")
    hidden = torch.empty(rows, inner, dtype=dtype, device="cuda")
    pages_each = -(-length // page_size)
    table_width = max(pages_each, -(-shape.positions // page_size))
    tables = torch.zeros(prompts, table_width, dtype=torch.int32, device="cuda")
    tables[:, :pages_each] = torch.arange(prompts * pages_each, dtype=torch.int32, device="cuda").view(prompts, pages_each)
    positions = torch.arange(length, dtype=torch.int32, device="cuda").repeat(prompts)
    tok_item = torch.arange(prompts, dtype=torch.int32, device="cuda").repeat_interleave(length)
    cu_tokens = torch.arange(prompts + 1, dtype=torch.int32, device="cuda") * length
    kv_lens = torch.full((prompts,), length, dtype=torch.int32, device="cuda")
    tile = kernels.PREFILL_TILE
    if kernels.prefill_large_tile_pays(heads, head_dim, prompts * -(-length // kernels.PREFILL_LARGE_TILE), length):
        tile = kernels.PREFILL_LARGE_TILE   # as the attention part chooses
    starts = list(range(0, length, tile))
    order = sorted(((item, q0) for item in range(prompts) for q0 in starts), key=lambda t: -t[1])
    tile_item = torch.tensor([t[0] for t in order], dtype=torch.int32, device="cuda")
    tile_q0 = torch.tensor([t[1] for t in order], dtype=torch.int32, device="cuda")
    k_pool = randn(prompts * pages_each, heads, page_size, head_dim, kind=dtype)
    v_pool = randn(prompts * pages_each, heads, page_size, head_dim, kind=dtype)
    out = []

    def wanted(name):
        return only is None or any(piece in name for piece in only)

    def product(name, n, k, call, seed, extra_bytes=0):
        if not wanted(name):
            return
        copies = _copies(n * k * 2, least=8, most=48)
        weights, packed = _matrices(n, k, copies, seed)
        bias = randn(n) * 0.1
        us = graph_time(lambda i: call(weights[i], packed[i], bias), copies)
        out.append(_row(name, us, n * k * 2 + extra_bytes, 2 * rows * n * k, peaks))
        del weights, packed
        torch.cuda.empty_cache()

    if wanted("norm"):
        us = graph_time(lambda i: kernels.norm(h, gamma, beta, shape.eps, normed), 8)
        out.append(_row("norm", us, rows * d * 6, 0, peaks))
    product("qkv+cache_write", 3 * d, d,
            lambda w, wp, bias: kernels.linear(normed, w, bias, qkv, packed=wp, scatter_only=True,
                                               scatter=(k_pool, v_pool, tok_item, positions, tables, d, d)),
            21, extra_bytes=rows * d * 2 * 4)
    if wanted("attention") and kernels.prefill_supported(dtype, head_dim, table_width):
        q = qkv[:, :d]
        us = graph_time(lambda i: kernels.attention_prefill(
            q, k_pool, v_pool, context_rows, tile_item, tile_q0, cu_tokens, kv_lens, tables, heads,
            head_dim ** -0.5, max_kv_len=length, query_tile=tile), 8)
        flops = prompts * 4 * d * (length * (length + 1) // 2)
        out.append(_row(f"attention (tiles of {tile}, causal)", us, rows * d * 2 * 4, flops, peaks))
    product("out_proj+residual", d, d,
            lambda w, wp, bias: kernels.linear(context_rows, w, bias, h, epilogue="residual", packed=wp),
            22, extra_bytes=rows * d * (2 + 8))
    product("fc+gelu", inner, d,
            lambda w, wp, bias: kernels.linear(normed, w, bias, hidden, epilogue=shape.activation, packed=wp),
            23, extra_bytes=rows * (d + inner) * 2)
    product("proj+residual", d, inner,
            lambda w, wp, bias: kernels.linear(hidden, w, bias, h, epilogue="residual", packed=wp),
            24, extra_bytes=rows * (inner * 2 + d * 8))
    torch.cuda.empty_cache()
    return out


def mixed_table(raw, decodes, context, portion, peaks, page_size=16):
    """The kernels of one layer of a mixed step: ``decodes`` decoded tokens over ``context`` keys
    each beside one prompt portion of ``portion`` tokens (a new request's first)."""
    shape = _Shape(raw)
    d, inner, heads, head_dim = shape.d, shape.inner, shape.heads, shape.head_dim
    dtype = torch.bfloat16
    rows = decodes + portion
    generator = torch.Generator(device="cuda").manual_seed(3)

    def randn(*size, scale=1.0, kind=torch.float32):
        return (torch.randn(*size, device="cuda", generator=generator) * scale).to(kind)

    h = randn(rows, d)
    gamma, beta = randn(d) * 0.1 + 1, randn(d) * 0.1
    normed = torch.empty(rows, d, dtype=dtype, device="cuda")
    qkv = randn(rows, 3 * d, kind=dtype)
    context_rows = torch.empty(rows, d, dtype=dtype, device="cuda")
    hidden = torch.empty(rows, inner, dtype=dtype, device="cuda")
    items = decodes + 1
    lengths = [context] * decodes + [portion]
    pages_each = [-(-length // page_size) for length in lengths]
    table_width = -(-shape.positions // page_size)
    tables = torch.zeros(items, table_width, dtype=torch.int32, device="cuda")
    first = 0
    for item, count in enumerate(pages_each):
        tables[item, :count] = torch.arange(first, first + count, dtype=torch.int32, device="cuda")
        first += count
    positions = torch.tensor([context - 1] * decodes + list(range(portion)), dtype=torch.int32, device="cuda")
    tok_item = torch.tensor(list(range(decodes)) + [decodes] * portion, dtype=torch.int32, device="cuda")
    cu_tokens = torch.tensor(list(range(decodes + 1)) + [rows], dtype=torch.int32, device="cuda")
    kv_lens = torch.tensor(lengths, dtype=torch.int32, device="cuda")
    single_tokens = torch.arange(decodes, dtype=torch.int32, device="cuda")
    tile = kernels.PREFILL_TILE
    if kernels.prefill_small_tile_pays(heads, head_dim, -(-portion // tile)):
        tile = kernels.PREFILL_SMALL_TILE   # as the attention part chooses
    starts = sorted(range(0, portion, tile), reverse=True)
    tile_item = torch.full((len(starts),), decodes, dtype=torch.int32, device="cuda")
    tile_q0 = torch.tensor(starts, dtype=torch.int32, device="cuda")
    k_pool = randn(first, heads, page_size, head_dim, kind=dtype)
    v_pool = randn(first, heads, page_size, head_dim, kind=dtype)
    part = Attention(width=d, dtype=dtype, heads=heads, kv_heads=heads, head_dim=head_dim, scale=head_dim ** -0.5)
    out = []

    def product(name, n, k, call, seed, extra_bytes=0):
        copies = _copies(n * k * 2, least=8, most=48)
        weights, packed = _matrices(n, k, copies, seed)
        bias = randn(n) * 0.1
        us = graph_time(lambda i: call(weights[i], packed[i], bias), copies)
        out.append(_row(name, us, n * k * 2 + extra_bytes, 2 * rows * n * k, peaks))
        del weights, packed
        torch.cuda.empty_cache()

    us = graph_time(lambda i: kernels.norm(h, gamma, beta, shape.eps, normed), 8)
    out.append(_row("norm", us, rows * d * 6, 0, peaks))
    product("qkv+cache_write", 3 * d, d,
            lambda w, wp, bias: kernels.linear(normed, w, bias, qkv, packed=wp, scatter_only=True,
                                               scatter=(k_pool, v_pool, tok_item, positions, tables, d, d)),
            31, extra_bytes=rows * d * 2 * 4)
    q = qkv[:, :d]
    splits, waves = part._splits(decodes, max(context, portion))
    worst = (6 * kernels.compute_units() + rows * heads) * (head_dim + 2)
    partial = torch.empty(worst, dtype=torch.float32, device="cuda")
    fused = (part.fuse_mixed and kernels.mixed_supported(dtype, head_dim, table_width)
             and not (4 * decodes * heads < kernels.compute_units() and max(context, portion) > 512))
    if fused:
        # as the attention part runs them: both kinds of block in one launch (tiles of 64)
        starts64 = sorted(range(0, portion, kernels.PREFILL_TILE), reverse=True)
        item64 = torch.full((len(starts64),), decodes, dtype=torch.int32, device="cuda")
        q064 = torch.tensor(starts64, dtype=torch.int32, device="cuda")
        us = graph_time(lambda i: kernels.attention_mixed(
            q, k_pool, v_pool, context_rows, single_tokens, tok_item, positions, item64, q064, cu_tokens,
            kv_lens, tables, heads, part.scale), 8)
        out.append(_row("attention (decoded tokens and portion in one launch)", us,
                        2 * decodes * context * d * 2 + portion * d * 2 * 4,
                        4 * decodes * context * d + 4 * d * (portion * (portion + 1) // 2), peaks))
    us = graph_time(lambda i: kernels.attention_decode(
        q, k_pool, v_pool, context_rows, tok_item, positions, tables, heads, part.scale, splits,
        partial=partial if splits > 1 else None, waves=waves, tok_list=single_tokens), 8)
    apart = " (apart: not part of the step)" if fused else ""
    out.append(_row(f"attention of the decoded tokens ({splits} key ranges, {waves} waves){apart}", us,
                    2 * decodes * context * d * 2, 4 * decodes * context * d, peaks,
                    launches=2 if splits > 1 else 1))
    if kernels.prefill_supported(dtype, head_dim, table_width):
        us = graph_time(lambda i: kernels.attention_prefill(
            q, k_pool, v_pool, context_rows, tile_item, tile_q0, cu_tokens, kv_lens, tables, heads,
            head_dim ** -0.5, max_kv_len=max(context, portion), query_tile=tile), 8)
        out.append(_row(f"attention of the portion (tiles of {tile}, causal){apart}", us, portion * d * 2 * 4,
                        4 * d * (portion * (portion + 1) // 2), peaks))
    product("out_proj+residual", d, d,
            lambda w, wp, bias: kernels.linear(context_rows, w, bias, h, epilogue="residual", packed=wp),
            32, extra_bytes=rows * d * (2 + 8))
    product("fc+gelu", inner, d,
            lambda w, wp, bias: kernels.linear(normed, w, bias, hidden, epilogue=shape.activation, packed=wp),
            33, extra_bytes=rows * (d + inner) * 2)
    product("proj+residual", d, inner,
            lambda w, wp, bias: kernels.linear(hidden, w, bias, h, epilogue="residual", packed=wp),
            34, extra_bytes=rows * (inner * 2 + d * 8))
    torch.cuda.empty_cache()
    return out


def format_table(title, rows):
    lines = [title,
             f"  {'kernel':<52} {'us':>8} {'MB':>9} {'GB/s':>8} {'of 8 TB/s':>9} {'GFLOP':>8} {'TFLOP/s':>8} {'of 2.5 PF':>9}"]
    for row in rows:
        lines.append(f"  {row['kernel']:<52} {row['us']:>8.2f} {row['MB']:>9.3f} {row['GBps']:>8.0f} "
                     f"{100 * row['of_hbm']:>8.1f}% {row['GFLOP']:>8.2f} {row['TFLOPs']:>8.1f} {100 * row['of_mfma']:>8.1f}%")
    return "\n".join(lines)
