"""Each HIP kernel alone against a plain float64 torch formula, at sizes that differ
from the engine's tiny models (ragged widths, odd row counts, head sizes 16..128)."""

import math

import pytest
import torch
from torch.nn import functional as F

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def _tol(dtype):
    """(atol, rtol).  bfloat16: a result stored in bfloat16 is off by up to 2^-9 of itself (half a
    unit in the last place), and inputs rounded the same way move a sum of k products by some
    2^-9 of its terms' size; measured, the kernels here stay within 9e-4 + 9e-4 |expected| at
    every shape of these tests, and the bound leaves five times that."""
    return (2e-5, 2e-5) if dtype == torch.float32 else (5e-3, 5e-3)


def _rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).cuda()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tokens,width,vocab,positions", [(1, 64, 50, 9), (37, 100, 257, 64), (300, 768, 1000, 128)])
def test_embed(dtype, tokens, width, vocab, positions):
    from pagedserve_amd.ops import kernels

    table = _rand((vocab, width), dtype, 0)
    pos_table = _rand((positions, width), dtype, 1)
    g = torch.Generator().manual_seed(2)
    ids = torch.randint(0, vocab, (tokens,), generator=g).int().cuda()
    pos = torch.randint(0, positions, (tokens,), generator=g).int().cuda()
    out = torch.full((tokens, width), float("nan"), device="cuda")
    kernels.embed(table, pos_table, ids, pos, out)
    expected = F.embedding(ids.long(), table.float()) + F.embedding(pos.long(), pos_table.float())
    torch.testing.assert_close(out, expected, atol=0, rtol=0)
    kernels.embed(table, None, ids, pos, out)
    torch.testing.assert_close(out, F.embedding(ids.long(), table.float()), atol=0, rtol=0)
    kernels.embed(table, pos_table, ids, pos, out, scale=8.0)
    torch.testing.assert_close(out, expected + 7.0 * F.embedding(ids.long(), table.float()), atol=1e-5, rtol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,width", [(1, 768), (8, 768), (32, 768), (5, 96), (3, 1600), (7, 50)])
def test_layernorm_matches_library(dtype, rows, width):
    # shapes (1, 8, 32) x 768 are those of testing/test_triton_residual_layernorm.py:7-35
    from pagedserve_amd.ops import kernels

    x = _rand((rows, width), torch.float32, 515)
    gamma = _rand((width,), torch.float32, 516)
    beta = _rand((width,), torch.float32, 517)
    out = torch.empty((rows, width), dtype=dtype, device="cuda")
    kernels.norm(x, gamma, beta, 1e-5, out)
    expected = F.layer_norm(x.double(), (width,), gamma.double(), beta.double(), 1e-5)
    atol, rtol = _tol(dtype)
    torch.testing.assert_close(out.double(), expected, atol=atol, rtol=rtol)


def test_layernorm_eps_and_gather():
    """A row of tiny variance tells eps 1e-5 from 1e-6; `rows` gathers and reorders."""
    from pagedserve_amd.ops import kernels

    width = 64
    x = torch.zeros(4, width, device="cuda")
    # tiny variance around zero (an offset would only add the float rounding of the mean)
    x[1] = _rand((width,), torch.float32, 3) * 1e-3
    x[3] = _rand((width,), torch.float32, 4)
    gamma = torch.ones(width, device="cuda")
    beta = torch.zeros(width, device="cuda")
    rows = torch.tensor([3, 1], dtype=torch.int32, device="cuda")
    for eps in (1e-5, 1e-6):
        out = torch.empty(2, width, device="cuda")
        kernels.norm(x, gamma, beta, eps, out, rows=rows)
        expected = F.layer_norm(x[[3, 1]].double(), (width,), None, None, eps)
        torch.testing.assert_close(out.double(), expected, atol=1e-5, rtol=1e-5)
    a = torch.empty(2, width, device="cuda")
    b = torch.empty(2, width, device="cuda")
    kernels.norm(x, gamma, beta, 1e-5, a, rows=rows)
    kernels.norm(x, gamma, beta, 1e-6, b, rows=rows)
    assert (a[1] - b[1]).abs().max() > 1e-2          # the tiny-variance row feels eps
    # a constant row maps to beta
    const = torch.full((1, width), 3.0, device="cuda")
    out = torch.empty(1, width, device="cuda")
    kernels.norm(const, gamma, beta + 0.25, 1e-5, out)
    torch.testing.assert_close(out, torch.full_like(out, 0.25), atol=1e-6, rtol=0)


def test_rmsnorm():
    from pagedserve_amd.ops import kernels

    x = _rand((6, 80), torch.float32, 5)
    gamma = _rand((80,), torch.float32, 6)
    out = torch.empty(6, 80, device="cuda")
    kernels.norm(x, gamma, None, 1e-6, out, rms=True)
    xd = x.double()
    expected = xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + 1e-6) * gamma.double()
    torch.testing.assert_close(out.double(), expected, atol=2e-5, rtol=2e-5)


# rows 1..64 take the skinny kernel in bfloat16, more rows the tiled one; k = 100 and 66 are
# not multiples of 8 and fall to the plain kernel
GEMM_SHAPES = [(1, 50, 64), (5, 1000, 96), (64, 2304, 768), (130, 70, 320), (33, 257, 100),
               (256, 768, 3072), (2, 50257, 64), (17, 768, 768), (48, 100, 3072), (65, 192, 96),
               (300, 1000, 320), (129, 257, 66), (8, 768, 3072), (512, 2304, 768),
               # enough tiles for the larger tile shapes of the bfloat16 tiled kernel, with whole
               # and with ragged rows of eight columns
               (1100, 2800, 128), (1027, 2801, 192), (3500, 3530, 64),
               # 17 to 64 rows: rows spread over blocks where the columns give few of them, and
               # the tiled kernel for a k beyond one round of the skinny kernel's loads
               (64, 768, 768), (40, 400, 1600), (50, 4800, 1600), (33, 330, 2112), (64, 1600, 6400),
               # so many blocks that two column tiles go to a block (residual epilogue), with a
               # ragged last tile and a last k range of one step
               (33, 1290, 5184), (20, 1600, 6400),
               # few rows and very many columns: two tiles of columns per block, ragged end
               (9, 16411, 320), (16, 20000, 768),
               # few rows in float: a k shorter than one pass of a wave's lanes, a k that is a
               # multiple of 4 only, columns that end inside a wave's share
               (13, 41, 16), (3, 333, 60), (4, 101, 100), (16, 7, 1028)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", GEMM_SHAPES)
@pytest.mark.parametrize("epilogue", ["none", "gelu_tanh", "gelu_erf", "residual"])
def test_gemm_nt(dtype, m, n, k, epilogue):
    from pagedserve_amd.ops import kernels

    if epilogue != "none" and n > 5000:
        pytest.skip("one epilogue is enough at the vocabulary size")
    if epilogue == "gelu_erf" and m > 1000:
        pytest.skip("one activation is enough at the large shapes")
    a = _rand((m, k), dtype, 10, 1.0)
    w = _rand((n, k), dtype, 11, 1.0 / math.sqrt(k))
    bias = _rand((n,), torch.float32, 12)
    product = a.double() @ w.double().t() + bias.double()
    if epilogue == "residual":
        out = _rand((m, n), torch.float32, 13)
        expected = out.double() + product
    else:
        out_dtype = dtype
        out = torch.full((m, n), float("nan"), dtype=out_dtype, device="cuda")
        if epilogue == "gelu_tanh":
            expected = F.gelu(product, approximate="tanh")
        elif epilogue == "gelu_erf":
            expected = F.gelu(product)
        else:
            expected = product
    kernels.gemm_nt(a, w, bias, out, epilogue=epilogue)
    atol, rtol = _tol(dtype)
    torch.testing.assert_close(out.double(), expected, atol=atol * 2, rtol=rtol)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_float_logits_and_strided_views(dtype):
    """bfloat16 operands with float output (the head), inputs and outputs that are column
    slices of wider buffers, and no bias."""
    from pagedserve_amd.ops import kernels

    wide = _rand((9, 300), dtype, 20)
    a = wide[:, 100:196]
    w = _rand((77, 96), dtype, 21, 0.1)
    out_wide = torch.zeros((9, 200), dtype=torch.float32, device="cuda")
    out = out_wide[:, 50:127]
    kernels.gemm_nt(a, w, None, out)
    expected = a.double() @ w.double().t()
    atol, rtol = (2e-5, 2e-5) if dtype == torch.float32 else (2e-3, 2e-3)
    torch.testing.assert_close(out.double(), expected, atol=atol, rtol=rtol)
    assert float(out_wide[:, :50].abs().max()) == 0 and float(out_wide[:, 127:].abs().max()) == 0


def test_gemm_identity_and_one_hot():
    from pagedserve_amd.ops import kernels

    w = _rand((40, 40), torch.float32, 30)
    eye = torch.eye(40, device="cuda")
    out = torch.empty(40, 40, device="cuda")
    kernels.gemm_nt(eye, w, None, out)           # row m of out = column m of w^T... = w[:, m]
    torch.testing.assert_close(out, w.t().contiguous(), atol=0, rtol=0)
    kernels.gemm_nt(w, eye, None, out)
    torch.testing.assert_close(out, w, atol=0, rtol=0)


def _paged_fixture(dtype, batch_lens, kv_heads, head_dim, page_size, seed, extra_pages=5):
    """Fragmented pools and tables for requests of the given cached lengths.  Whatever no
    request owns holds NaN: page 0 and the other spare pages, and the slots behind each
    request's last key, so a kernel that lets a masked or clamped load reach its result fails."""
    g = torch.Generator().manual_seed(seed)
    pages_per = [-(-length // page_size) for length in batch_lens]
    width = max(pages_per) + 2
    total = sum(pages_per) + extra_pages
    order = (torch.randperm(total - 1, generator=g) + 1).tolist()     # page 0 stays unowned
    tables = torch.full((len(batch_lens), width), -1, dtype=torch.int32)
    owned = torch.zeros(total, page_size, dtype=torch.bool)
    cursor = 0
    for index, (count, length) in enumerate(zip(pages_per, batch_lens)):
        pages = order[cursor:cursor + count]
        tables[index, :count] = torch.tensor(pages, dtype=torch.int32)
        for logical, page in enumerate(pages):
            owned[page, :max(0, min(page_size, length - logical * page_size))] = True
        cursor += count
    k_pool = torch.randn((total, kv_heads, page_size, head_dim), generator=g)
    v_pool = torch.randn((total, kv_heads, page_size, head_dim), generator=g)
    hole = ~owned[:, None, :, None].expand_as(k_pool)
    k_pool[hole] = float("nan")
    v_pool[hole] = float("nan")
    return k_pool.to(dtype).cuda(), v_pool.to(dtype).cuda(), tables.cuda()


def _gather(pool, table, length, page_size):
    pages = table[: -(-length // page_size)].long()
    return pool[pages].permute(1, 0, 2, 3).reshape(pool.shape[1], -1, pool.shape[3])[:, :length]


def _attention_expected(q, k_pool, v_pool, tables, tok_item, tok_pos, heads, scale, window=0):
    """float64 attention of every token over the keys 0..position (the last ``window``) of its
    request, gathered page by page through the table: softmax(q K^T scale) V, nothing shared
    with any kernel."""
    kv_heads, page_size, head_dim = k_pool.shape[1], k_pool.shape[2], k_pool.shape[3]
    group = heads // kv_heads
    k_cpu, v_cpu, t_cpu = k_pool.double().cpu(), v_pool.double().cpu(), tables.cpu()
    q_cpu = q.double().cpu()
    out = torch.empty_like(q_cpu)
    for t, (item, pos) in enumerate(zip(torch.as_tensor(tok_item).tolist(), torch.as_tensor(tok_pos).tolist())):
        first = max(0, pos - window + 1) if window > 0 else 0
        keys = _gather(k_cpu, t_cpu[item], pos + 1, page_size)[:, first:].repeat_interleave(group, 0)
        values = _gather(v_cpu, t_cpu[item], pos + 1, page_size)[:, first:].repeat_interleave(group, 0)
        scores = torch.einsum("hd,hkd->hk", q_cpu[t].reshape(heads, head_dim), keys) * scale
        out[t] = torch.einsum("hk,hkd->hd", torch.softmax(scores, -1), values).reshape(-1)
    return out.cuda()


# head sizes: multiples of 16, of 8 only (8, 24, 40), and of neither (20, 7, 100); page sizes
# that are no power of two (12, 5)
ROWWISE_GEOMETRIES = [(1, 1, 32, 16), (4, 4, 16, 8), (6, 2, 48, 16), (3, 3, 128, 4), (12, 12, 64, 16),
                      (2, 2, 8, 4), (4, 2, 20, 12), (3, 1, 7, 5), (2, 2, 100, 16), (5, 5, 80, 12),
                      (2, 1, 256, 16), (6, 2, 24, 12)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,head_dim,page_size", ROWWISE_GEOMETRIES)
def test_attention_rowwise_decode_contexts(dtype, heads, kv_heads, head_dim, page_size):
    """Single-token queries over fragmented tables; contexts around page edges as in
    testing/test_triton_correctness_matrix.py:9 (1, 15, 16, 17, 31, 32, 33, 128, 512)."""
    from pagedserve_amd.ops import kernels

    contexts = [1, 15, 16, 17, 31, 32, 33, 128, 512]
    k_pool, v_pool, tables = _paged_fixture(dtype, contexts, kv_heads, head_dim, page_size, 17)
    q = _rand((len(contexts), heads * head_dim), dtype, 18)
    out = torch.empty_like(q)
    tok_item = torch.arange(len(contexts), dtype=torch.int32, device="cuda")
    tok_pos = torch.tensor([c - 1 for c in contexts], dtype=torch.int32, device="cuda")
    scale = head_dim ** -0.5
    kernels.attention_rowwise(q, k_pool, v_pool, out, tok_item, tok_pos, tables, heads, scale)
    group = heads // kv_heads
    for index, context in enumerate(contexts):
        keys = _gather(k_pool, tables[index], context, page_size).double()
        values = _gather(v_pool, tables[index], context, page_size).double()
        keys = keys.repeat_interleave(group, 0)
        values = values.repeat_interleave(group, 0)
        query = q[index].double().reshape(heads, 1, head_dim)
        expected = F.scaled_dot_product_attention(query, keys, values).reshape(-1)
        atol, rtol = (3e-5, 3e-5) if dtype == torch.float32 else (2e-2, 2e-2)
        torch.testing.assert_close(out[index].double(), expected, atol=atol, rtol=rtol)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,head_dim,page_size", [(6, 2, 48, 12), (4, 4, 20, 8), (2, 1, 256, 16)])
@pytest.mark.parametrize("window", [0, 7, 40])
def test_attention_rowwise_portions_grouped_heads_and_windows(dtype, heads, kv_heads, head_dim, page_size, window):
    """Portions of several requests in one launch (fresh, continued, a single token), grouped
    key/value heads with a window, a page size that is no power of two, head sizes 20 and
    256: against float64 attention over the gathered pages."""
    from pagedserve_amd.ops import kernels

    items = [(0, 9), (30, 23), (17, 1), (100, 37)]
    totals = [past + new for past, new in items]
    k_pool, v_pool, tables = _paged_fixture(dtype, totals, kv_heads, head_dim, page_size, 123)
    tok_item, tok_pos = [], []
    for index, (past, new) in enumerate(items):
        tok_item += [index] * new
        tok_pos += list(range(past, past + new))
    q = _rand((len(tok_item), heads * head_dim), dtype, 124)
    out = torch.full_like(q, float("nan"))
    scale = head_dim ** -0.5
    kernels.attention_rowwise(q, k_pool, v_pool, out, torch.tensor(tok_item, dtype=torch.int32, device="cuda"),
                              torch.tensor(tok_pos, dtype=torch.int32, device="cuda"), tables, heads, scale,
                              window=window)
    expected = _attention_expected(q, k_pool, v_pool, tables, tok_item, tok_pos, heads, scale, window)
    atol, rtol = (3e-5, 3e-5) if dtype == torch.float32 else (2e-2, 2e-2)
    torch.testing.assert_close(out.double(), expected, atol=atol, rtol=rtol)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [0, 5, 16, 40])
def test_attention_rowwise_portion_and_window(dtype, window):
    """A portion of 23 queries that continues 30 cached keys; with and without a window;
    page tails hold NaN to prove they are never read into the result."""
    from pagedserve_amd.ops import kernels
    import plain_gpt2

    heads, head_dim, page_size, past, new = 2, 32, 8, 30, 23
    total = past + new
    k_pool, v_pool, tables = _paged_fixture(dtype, [total], heads, head_dim, page_size, 23)
    pages = tables[0, : -(-total // page_size)].long()
    last = pages[-1]
    k_pool[last, :, total % page_size:] = float("nan")
    v_pool[last, :, total % page_size:] = float("nan")
    keys = _gather(k_pool, tables[0], total, page_size).double()
    values = _gather(v_pool, tables[0], total, page_size).double()
    g = torch.Generator().manual_seed(5)
    q_all = torch.randn((heads, total, head_dim), generator=g).to(dtype).cuda()
    expected = plain_gpt2.causal_attention(q_all.double().cpu(), keys.cpu(), values.cpu(),
                                           head_dim ** -0.5, window=window)[:, past:]
    q = q_all[:, past:].permute(1, 0, 2).reshape(new, heads * head_dim).contiguous()
    out = torch.empty_like(q)
    tok_item = torch.zeros(new, dtype=torch.int32, device="cuda")
    tok_pos = torch.arange(past, total, dtype=torch.int32, device="cuda")
    kernels.attention_rowwise(q, k_pool, v_pool, out, tok_item, tok_pos, tables, heads,
                              head_dim ** -0.5, window=window)
    got = out.double().cpu().reshape(new, heads, head_dim).permute(1, 0, 2)
    atol, rtol = (3e-5, 3e-5) if dtype == torch.float32 else (2e-2, 2e-2)
    torch.testing.assert_close(got, expected, atol=atol, rtol=rtol)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,head_dim,page_size", [(1, 1, 32, 16), (4, 4, 16, 8), (6, 2, 48, 16), (3, 3, 128, 4), (12, 12, 64, 16), (2, 1, 256, 16), (5, 5, 80, 12),
                                                                (2, 2, 8, 4), (6, 2, 24, 12), (3, 3, 40, 16), (4, 1, 200, 5)])
@pytest.mark.parametrize("splits", [1, 2, 5, 16, 40])
def test_attention_decode_split_kv(dtype, heads, kv_heads, head_dim, page_size, splits):
    """The split-KV kernel over fragmented tables at the contexts of
    testing/test_triton_correctness_matrix.py:9, for any number of splits (also more than the
    keys can feed), listed tokens in any order, and a window."""
    from pagedserve_amd.ops import kernels

    contexts = [1, 15, 16, 17, 31, 32, 33, 128, 512, 1024]
    k_pool, v_pool, tables = _paged_fixture(dtype, contexts, kv_heads, head_dim, page_size, 19)
    count = len(contexts)
    q = _rand((count, heads * head_dim), dtype, 20)
    tok_item = torch.arange(count, dtype=torch.int32, device="cuda")
    tok_pos = torch.tensor([c - 1 for c in contexts], dtype=torch.int32, device="cuda")
    scale = head_dim ** -0.5
    partial = torch.full((count * heads * splits * (head_dim + 2),), float("nan"), device="cuda")
    atol, rtol = (3e-5, 3e-5) if dtype == torch.float32 else (2e-2, 2e-2)
    for window in (0, 20):
        expected = _attention_expected(q, k_pool, v_pool, tables, tok_item, tok_pos, heads, scale, window)
        out = torch.full_like(q, float("nan"))
        kernels.attention_decode(q, k_pool, v_pool, out, tok_item, tok_pos, tables, heads, scale, splits,
                                 partial=partial, window=window)
        torch.testing.assert_close(out.double(), expected, atol=atol, rtol=rtol)
        # no item index: token t is item t (tables of 66 to 258 entries: short ones are held
        # in registers, over 64 in two, long ones are read as before); the same sums in the
        # same order, so not a bit differs
        direct = torch.full_like(q, float("nan"))
        kernels.attention_decode(q, k_pool, v_pool, direct, None, tok_pos, tables, heads, scale, splits,
                                 partial=partial, window=window)
        assert torch.equal(direct, out)
    # a list of tokens: only those rows are written
    chosen = torch.tensor([7, 2, 9], dtype=torch.int32, device="cuda")
    out = torch.full_like(q, 7.0)
    kernels.attention_decode(q, k_pool, v_pool, out, tok_item, tok_pos, tables, heads, scale, splits,
                             partial=partial, tok_list=chosen)
    expected = _attention_expected(q, k_pool, v_pool, tables, tok_item, tok_pos, heads, scale)
    for row in range(count):
        if row in (7, 2, 9):
            torch.testing.assert_close(out[row].double(), expected[row], atol=atol, rtol=rtol)
        else:
            assert float((out[row].float() - 7.0).abs().max()) == 0.0
    direct = torch.full_like(q, 7.0)
    kernels.attention_decode(q, k_pool, v_pool, direct, None, tok_pos, tables, heads, scale, splits,
                             partial=partial, tok_list=chosen)
    assert torch.equal(direct, out)

    with pytest.raises(kernels.KernelError, match="row per token"):
        kernels.attention_decode(q, k_pool, v_pool, direct, None, tok_pos, tables[:3], heads, scale, splits,
                                 partial=partial)


def test_attention_far_key_stands_out():
    """One key among 700 is made to dominate: the output must be its value.  A kernel that
    skips a page, mixes two requests' tables or misplaces an offset fails this."""
    from pagedserve_amd.ops import kernels

    heads, head_dim, page_size, context = 2, 64, 16, 700
    for dtype in DTYPES:
        k_pool, v_pool, tables = _paged_fixture(dtype, [context, context], heads, head_dim, page_size, 31)
        k_pool *= 0.1
        q = _rand((2, heads * head_dim), dtype, 32, 0.1)
        targets = [(0, 0, 3), (0, 1, 367), (1, 0, 688), (1, 1, 699)]
        for item, head, key in targets:
            page = int(tables[item, key // page_size])
            direction = q[item, head * head_dim:(head + 1) * head_dim].float()
            direction = direction / direction.norm()
            q[item, head * head_dim:(head + 1) * head_dim] = (direction * 8.0).to(dtype)
            k_pool[page, head, key % page_size] = (direction * 40.0).to(dtype)
        tok_item = torch.arange(2, dtype=torch.int32, device="cuda")
        tok_pos = torch.full((2,), context - 1, dtype=torch.int32, device="cuda")
        partial = torch.empty(2 * heads * 7 * (head_dim + 2), device="cuda")
        # "direct": without the item index, tables of 46 entries held in one register a lane
        for kernel in ("rowwise", "decode1", "decode7", "direct1", "direct7"):
            out = torch.empty_like(q)
            if kernel == "rowwise":
                kernels.attention_rowwise(q, k_pool, v_pool, out, tok_item, tok_pos, tables, heads, head_dim ** -0.5)
            else:
                kernels.attention_decode(q, k_pool, v_pool, out,
                                         tok_item if kernel.startswith("decode") else None, tok_pos,
                                         tables, heads, head_dim ** -0.5, int(kernel[6:]), partial=partial)
            for item, head, key in targets:
                page = int(tables[item, key // page_size])
                expected = v_pool[page, head, key % page_size].float()
                got = out[item, head * head_dim:(head + 1) * head_dim].float()
                torch.testing.assert_close(got, expected, atol=5e-3, rtol=5e-3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_kv_write_places_tokens(dtype):
    """Token t of a request lands at (table[t // page], t % page)
    (testing/test_project.py:66-88) and nothing else in the pool changes."""
    from pagedserve_amd.ops import kernels

    kv_heads, head_dim, page_size = 3, 16, 4
    lens = [5, 9]
    k_pool, v_pool, tables = _paged_fixture(dtype, lens, kv_heads, head_dim, page_size, 41)
    before_k, before_v = k_pool.clone(), v_pool.clone()
    starts = [2, 0]      # request 0 already holds 2 tokens
    tok_item, tok_pos = [], []
    for item, (start, length) in enumerate(zip(starts, lens)):
        for position in range(start, length):
            tok_item.append(item)
            tok_pos.append(position)
    tokens = len(tok_item)
    wide = _rand((tokens, 5 * kv_heads * head_dim), dtype, 42)
    k = wide[:, kv_heads * head_dim:2 * kv_heads * head_dim]
    v = wide[:, 3 * kv_heads * head_dim:4 * kv_heads * head_dim]
    kernels.kv_write(k, v, k_pool, v_pool, torch.tensor(tok_item, dtype=torch.int32, device="cuda"),
                     torch.tensor(tok_pos, dtype=torch.int32, device="cuda"), tables)
    touched = torch.zeros(k_pool.shape[:3], dtype=torch.bool)
    for t, (item, position) in enumerate(zip(tok_item, tok_pos)):
        page = int(tables[item, position // page_size])
        torch.testing.assert_close(k_pool[page, :, position % page_size], k[t].reshape(kv_heads, head_dim), atol=0, rtol=0)
        torch.testing.assert_close(v_pool[page, :, position % page_size], v[t].reshape(kv_heads, head_dim), atol=0, rtol=0)
        touched[page, :, position % page_size] = True
    untouched = ~touched.cuda()
    assert torch.equal(k_pool[untouched].view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                       before_k[untouched].view(torch.int16 if dtype == torch.bfloat16 else torch.int32))
    assert torch.equal(v_pool[untouched].view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                       before_v[untouched].view(torch.int16 if dtype == torch.bfloat16 else torch.int32))


def test_sample_argmax_and_ties():
    from pagedserve_amd.ops import kernels

    for vocab in (7, 257, 1000, 16385, 50257, 53249, 65537):
        logits = _rand((5, vocab), torch.float32, vocab)
        logits[2, vocab // 2] = 50.0
        logits[3, 1] = 60.0
        logits[3, vocab - 1] = 60.0      # tie: the lowest id wins
        out = torch.empty(5, dtype=torch.int32, device="cuda")
        kernels.sample(logits, None, None, out)
        assert out.tolist() == torch.argmax(logits, dim=-1).tolist()
        assert out[3].item() == 1


@pytest.mark.parametrize("vocab,rows", [(1000, 64), (5, 16), (16384, 12), (16385, 12), (50257, 24), (53249, 8),
                                        (65536, 8), (70001, 8)])
def test_sample_temperature_inverse_cdf(vocab, rows):
    """The token drawn is the one whose share of the cumulative distribution (in id order) holds
    the row's uniform number; rows of up to 16,384, 53,248 and 65,536 ids take the kernels that
    keep the row in registers (16, 52 and 64 ids a lane), longer ones the kernel that reads the
    row three times.  Uniform numbers at and near 0 and 1 are among them."""
    from pagedserve_amd.ops import kernels

    logits = _rand((rows, vocab), torch.float32, 77, 2.0)
    g = torch.Generator().manual_seed(78)
    uniform = torch.rand(rows, generator=g)
    uniform[1], uniform[2], uniform[3] = 0.0, 0.999999, 1e-7
    uniform = uniform.cuda()
    temperature = 0.8
    inv_t = torch.full((rows,), 1.0 / temperature, device="cuda")
    inv_t[0] = 0.0   # greedy row inside a sampling batch
    out = torch.empty(rows, dtype=torch.int32, device="cuda")
    kernels.sample(logits, inv_t, uniform, out)
    probs = torch.softmax(logits.double() / temperature, dim=-1)
    cdf = probs.cumsum(-1)
    assert out[0].item() == int(torch.argmax(logits[0]))
    for row in range(1, rows):
        token = out[row].item()
        assert 0 <= token < vocab
        upper = float(cdf[row, token])
        lower = float(cdf[row, token - 1]) if token > 0 else 0.0
        assert lower - 1e-5 <= float(uniform[row]) <= upper + 1e-5, (row, token)
    if vocab != 1000:
        return
    # frequencies follow the probabilities on a small vocabulary
    small = torch.tensor([[0.0, 1.0, 2.0, -1.0, 0.5]], device="cuda").repeat(4000, 1)
    u = torch.rand(4000, generator=g).cuda()
    toks = torch.empty(4000, dtype=torch.int32, device="cuda")
    kernels.sample(small, torch.ones(4000, device="cuda"), u, toks)
    freq = torch.bincount(toks.long().cpu(), minlength=5).double() / 4000
    assert (freq - torch.softmax(small[0].double().cpu(), -1)).abs().max() < 0.03


def test_kernels_refuse_bad_sizes():
    from pagedserve_amd.ops import kernels

    q = torch.zeros((1, 20), device="cuda")
    pool = torch.zeros((2, 1, 4, 20), device="cuda")
    idx = torch.zeros(1, dtype=torch.int32, device="cuda")
    tables = torch.zeros((1, 2), dtype=torch.int32, device="cuda")
    with pytest.raises(kernels.KernelError, match="multiple of 8"):
        kernels.attention_decode(q, pool, pool.clone(), q.clone(), idx, idx, tables, 1, 1.0, 1)
    assert not kernels.decode_supported(20) and kernels.decode_supported(24)
    wide = torch.zeros((1, 264), device="cuda")
    wide_pool = torch.zeros((2, 1, 4, 264), device="cuda")
    with pytest.raises(kernels.KernelError, match="1..256"):
        kernels.attention_rowwise(wide, wide_pool, wide_pool.clone(), wide.clone(), idx, idx, tables, 1, 1.0)
    with pytest.raises(kernels.KernelError, match="GPU"):
        kernels.norm(torch.zeros(2, 4), torch.ones(4), None, 1e-5, torch.zeros(2, 4))
    with pytest.raises(kernels.KernelError):
        kernels.gemm_nt(torch.zeros(2, 8, device="cuda"), torch.zeros(3, 9, device="cuda"), None,
                        torch.zeros(2, 3, device="cuda"))


@pytest.mark.parametrize("heads,kv_heads,head_dim,page_size", [(1, 1, 32, 16), (4, 4, 16, 8), (6, 2, 48, 16), (2, 2, 128, 4), (12, 12, 64, 16), (3, 1, 80, 12),
                                                                # more than 256 blocks: the kernel's other arrangement of waves
                                                                (24, 8, 64, 16), (20, 20, 48, 8), (18, 18, 112, 16), (26, 13, 128, 16), (26, 26, 96, 8),
                                                                (26, 26, 16, 8), (26, 13, 32, 16), (28, 7, 80, 16), (2, 2, 96, 8), (3, 1, 112, 16),
                                                                # head sizes beyond 128: blocks of four waves only
                                                                (2, 1, 256, 16), (3, 3, 192, 8), (2, 2, 144, 12), (12, 4, 160, 16), (1, 1, 208, 16)])
@pytest.mark.parametrize("window", [0, 37])
@pytest.mark.parametrize("tile", [64, 32, 128])
def test_attention_prefill_tiles(heads, kv_heads, head_dim, page_size, window, tile):
    """The tiled kernel against float64 attention over the gathered pages (every head size in
    steps of 16 up to 128 in both arrangements of waves and with tiles of 32 queries, up to 64
    also with tiles of 128, larger ones in the one arrangement they have, and refused with
    the other tiles: the
    kernel reads LDS by assembly into registers that the compiler must leave alone until the
    wait, which a run of every variant checks): fresh prompts and later portions of many
    lengths in one launch (1 < count, portions that start inside a page, more than one tile,
    a tile's last rows empty), fragmented tables, NaN behind every request's last key."""
    from pagedserve_amd.ops import kernels

    dtype = torch.bfloat16
    # (cached before the portion, tokens of the portion)
    items = [(0, 2), (0, 64), (0, 65), (0, 200), (30, 23), (17, 130), (100, 16), (63, 3), (250, 70)]
    totals = [past + new for past, new in items]
    k_pool, v_pool, tables = _paged_fixture(dtype, totals, kv_heads, head_dim, page_size, 51)
    for index, total in enumerate(totals):
        if total % page_size:
            last = int(tables[index, total // page_size])
            k_pool[last, :, total % page_size:] = float("nan")
            v_pool[last, :, total % page_size:] = float("nan")
    tokens = sum(new for _, new in items)
    q = _rand((tokens, heads * head_dim), dtype, 52)
    tok_item, tok_pos, tile_item, tile_q0, cu = [], [], [], [], [0]
    for index, (past, new) in enumerate(items):
        tok_item += [index] * new
        tok_pos += list(range(past, past + new))
        cu.append(cu[-1] + new)
        for q0 in range(0, new, tile):
            tile_item.append(index)
            tile_q0.append(q0)

    def dev(values):
        return torch.tensor(values, dtype=torch.int32, device="cuda")

    scale = head_dim ** -0.5
    out = torch.full_like(q, float("nan"))
    if tile != kernels.PREFILL_TILE and head_dim > (128 if tile == kernels.PREFILL_SMALL_TILE
                                                     else kernels.PREFILL_LARGE_TILE_HEAD_DIM):
        with pytest.raises(kernels.KernelError, match="head sizes up to"):
            kernels.attention_prefill(q, k_pool, v_pool, out, dev(tile_item), dev(tile_q0), dev(cu),
                                      dev(totals), tables, heads, scale, window=window, query_tile=tile)
        return
    expected = _attention_expected(q, k_pool, v_pool, tables, tok_item, tok_pos, heads, scale, window)
    kernels.attention_prefill(q, k_pool, v_pool, out, dev(tile_item), dev(tile_q0), dev(cu), dev(totals),
                              tables, heads, scale, window=window, query_tile=tile)
    assert torch.isfinite(out.float()).all()
    torch.testing.assert_close(out.double(), expected, atol=5e-3, rtol=5e-3)


@pytest.mark.parametrize("heads,kv_heads,head_dim,page_size", [(1, 1, 32, 16), (4, 4, 16, 8), (6, 2, 48, 16), (2, 2, 128, 4), (12, 12, 64, 16),
                                                                (3, 1, 80, 12), (5, 5, 4, 3), (3, 3, 20, 5), (2, 1, 100, 16), (7, 7, 12, 1),
                                                                (25, 25, 64, 16), (2, 2, 68, 8)])
@pytest.mark.parametrize("window", [0, 37])
def test_attention_tiled_f32(heads, kv_heads, head_dim, page_size, window):
    """The 32-bit tiled kernel against float64 attention over the gathered pages, and against
    the one-wave-per-token kernel that it stands in for: fresh prompts and later portions of
    many lengths in one launch (portions that start inside a page, more than one tile, a tile's
    last rows empty, two tokens), fragmented tables, NaN behind every request's last key, head
    sizes that are multiples of 4 on both sides of 64; other head sizes are refused."""
    from pagedserve_amd.ops import kernels

    dtype = torch.float32
    items = [(0, 2), (0, 64), (0, 65), (0, 200), (30, 23), (17, 130), (100, 16), (63, 3), (250, 70)]
    totals = [past + new for past, new in items]
    k_pool, v_pool, tables = _paged_fixture(dtype, totals, kv_heads, head_dim, page_size, 53)
    for index, total in enumerate(totals):
        if total % page_size:
            last = int(tables[index, total // page_size])
            k_pool[last, :, total % page_size:] = float("nan")
            v_pool[last, :, total % page_size:] = float("nan")
    tokens = sum(new for _, new in items)
    q = _rand((tokens, heads * head_dim), dtype, 54)
    tok_item, tok_pos, tile_item, tile_q0, cu = [], [], [], [], [0]
    for index, (past, new) in enumerate(items):
        tok_item += [index] * new
        tok_pos += list(range(past, past + new))
        cu.append(cu[-1] + new)
        for q0 in range(0, new, kernels.PREFILL_TILE):
            tile_item.append(index)
            tile_q0.append(q0)

    def dev(values):
        return torch.tensor(values, dtype=torch.int32, device="cuda")

    scale = head_dim ** -0.5
    assert kernels.tiled_f32_supported(dtype, head_dim)
    # the tiles in another order than the items': every block finds its own rows
    order = list(reversed(range(len(tile_item))))
    out = torch.full_like(q, float("nan"))
    kernels.attention_tiled_f32(q, k_pool, v_pool, out, dev([tile_item[i] for i in order]),
                                dev([tile_q0[i] for i in order]), dev(cu), dev(totals), tables, heads, scale,
                                window=window)
    assert torch.isfinite(out).all()
    expected = _attention_expected(q, k_pool, v_pool, tables, tok_item, tok_pos, heads, scale, window)
    torch.testing.assert_close(out.double(), expected, atol=3e-5, rtol=3e-5)
    rowwise = torch.full_like(q, float("nan"))
    kernels.attention_rowwise(q, k_pool, v_pool, rowwise, dev(tok_item), dev(tok_pos), tables, heads, scale,
                              window=window)
    torch.testing.assert_close(out, rowwise, atol=2e-5, rtol=2e-5)


def test_attention_tiled_f32_refuses_what_it_cannot_take():
    from pagedserve_amd.ops import kernels

    assert not kernels.tiled_f32_supported(torch.float32, 6) and not kernels.tiled_f32_supported(torch.float32, 132)
    assert not kernels.tiled_f32_supported(torch.bfloat16, 64)
    index = torch.zeros(1, dtype=torch.int32, device="cuda")
    cu = torch.tensor([0, 2], dtype=torch.int32, device="cuda")
    lens = torch.tensor([2], dtype=torch.int32, device="cuda")
    tables = torch.zeros((1, 4), dtype=torch.int32, device="cuda")
    for head_dim in (6, 132):
        q = torch.zeros((2, head_dim), device="cuda")
        pool = torch.zeros((4, 1, 8, head_dim), device="cuda")
        with pytest.raises(kernels.KernelError, match="multiple of 4 up to 128"):
            kernels.attention_tiled_f32(q, pool, pool.clone(), torch.zeros_like(q), index, index, cu, lens, tables,
                                        1, 1.0)
    q = torch.zeros((2, 64), device="cuda", dtype=torch.bfloat16)
    pool = torch.zeros((4, 1, 8, 64), device="cuda", dtype=torch.bfloat16)
    with pytest.raises(kernels.KernelError):
        kernels.attention_tiled_f32(q, pool, pool.clone(), torch.zeros_like(q), index, index, cu, lens, tables, 1, 1.0)


@pytest.mark.parametrize("heads,kv_heads,head_dim,page_size", [(12, 12, 64, 16), (4, 4, 16, 8), (6, 2, 48, 16), (25, 25, 64, 16),
                                                                (3, 1, 32, 12), (16, 4, 64, 5)])
@pytest.mark.parametrize("window", [0, 37])
def test_attention_mixed_is_both_kernels_in_one_launch(heads, kv_heads, head_dim, page_size, window):
    """One launch for the one-token items and the items of several tokens of a step, listed in
    any order among each other: every row against float64 attention over the gathered pages,
    and bit for bit what the two kernels give that it is made of (the decode kernel with one
    range of keys, the tiled kernel with tiles of 64 queries where it takes its four-wave
    blocks).  NaN lies behind every request's last key and in the pages that nobody owns."""
    from pagedserve_amd.ops import kernels

    dtype = torch.bfloat16
    # (cached before the step, tokens of the step)
    items = [(130, 1), (0, 70), (15, 1), (511, 1), (30, 200), (0, 1), (63, 3), (250, 1), (17, 130), (99, 1)]
    totals = [past + new for past, new in items]
    k_pool, v_pool, tables = _paged_fixture(dtype, totals, kv_heads, head_dim, page_size, 71)
    for index, total in enumerate(totals):
        if total % page_size:
            last = int(tables[index, total // page_size])
            k_pool[last, :, total % page_size:] = float("nan")
            v_pool[last, :, total % page_size:] = float("nan")
    tokens = sum(new for _, new in items)
    q = _rand((tokens, heads * head_dim), dtype, 72)
    tok_item, tok_pos, singles, tile_item, tile_q0, cu = [], [], [], [], [], [0]
    for index, (past, new) in enumerate(items):
        if new == 1:
            singles.append(len(tok_item))
        else:
            for q0 in range(0, new, kernels.PREFILL_TILE):
                tile_item.append(index)
                tile_q0.append(q0)
        tok_item += [index] * new
        tok_pos += list(range(past, past + new))
        cu.append(cu[-1] + new)

    def dev(values):
        return torch.tensor(values, dtype=torch.int32, device="cuda")

    scale = head_dim ** -0.5
    assert kernels.mixed_supported(dtype, head_dim, tables.shape[1])
    out = torch.full_like(q, float("nan"))
    kernels.attention_mixed(q, k_pool, v_pool, out, dev(singles), dev(tok_item), dev(tok_pos), dev(tile_item),
                            dev(tile_q0), dev(cu), dev(totals), tables, heads, scale, window=window)
    assert torch.isfinite(out.float()).all()
    expected = _attention_expected(q, k_pool, v_pool, tables, tok_item, tok_pos, heads, scale, window)
    torch.testing.assert_close(out.double(), expected, atol=5e-3, rtol=5e-3)
    # the same blocks launched kind by kind (max_kv_len below 512: the tiled kernel's blocks of
    # four waves, which are the ones that the common launch runs)
    apart = torch.full_like(q, float("nan"))
    kernels.attention_decode(q, k_pool, v_pool, apart, dev(tok_item), dev(tok_pos), tables, heads, scale, 1,
                             window=window, waves=4, tok_list=dev(singles))
    kernels.attention_prefill(q, k_pool, v_pool, apart, dev(tile_item), dev(tile_q0), dev(cu), dev(totals),
                              tables, heads, scale, window=window, max_kv_len=256)
    assert torch.equal(out, apart)
    # a call site's memo: the second call with the same addresses goes straight to the library
    memo = {}
    first, second = torch.zeros_like(q), torch.zeros_like(q)
    lists = (dev(singles), dev(tok_item), dev(tok_pos), dev(tile_item), dev(tile_q0), dev(cu), dev(totals))
    for target in (first, first, second):
        target.zero_()
        kernels.attention_mixed(q, k_pool, v_pool, target, *lists, tables, heads, scale, window=window, memo=memo)
        assert torch.equal(target, out)
    assert len(memo) == 2 + 1 and all(type(kept) is tuple for kept in memo.values())   # (+ the site's own entry)
    # the same call of another layer (other pools) in a step whose index arrays are new to both:
    # the first is checked, the second takes the first's arguments with its own pools
    other_k, other_v = (k_pool * 0.5).contiguous(), (v_pool * 2.0).contiguous()
    other_memo = {}
    third = torch.zeros_like(q)
    kernels.attention_mixed(q, other_k, other_v, third, *lists, tables, heads, scale, window=window, memo=other_memo)
    expected_other = third.clone()
    assert not torch.equal(expected_other, out)
    new_lists = tuple(index.clone() for index in lists)
    shared = {}
    checks = []
    real_check = kernels._check
    kernels._check = lambda *args, **kwargs: (checks.append(args[1]), real_check(*args, **kwargs))[1]
    try:
        # (the layers of a step write to one buffer: the target is part of what they share)
        first.zero_()
        kernels.attention_mixed(q, k_pool, v_pool, first, *new_lists, tables, heads, scale, window=window,
                                memo=memo, shared=shared)
        assert checks and len(shared) == 1
        own_pools = first.clone()
        del checks[:]
        first.zero_()
        kernels.attention_mixed(q, other_k, other_v, first, *new_lists, tables, heads, scale, window=window,
                                memo=other_memo, shared=shared)
        assert not checks
        other_pools = first.clone()
        # pools that this site has not been checked with take the whole way
        fresh_k = other_k.clone()
        first.zero_()
        kernels.attention_mixed(q, fresh_k, other_v, first, *new_lists, tables, heads, scale, window=window,
                                memo=other_memo, shared=shared)
        assert checks
    finally:
        kernels._check = real_check
    assert torch.equal(own_pools, out) and torch.equal(other_pools, expected_other) and torch.equal(first, expected_other)
    with pytest.raises(kernels.KernelError, match="launch the two kernels"):
        wide = torch.zeros(4, 2 * 128, dtype=dtype, device="cuda")
        pool = torch.zeros(4, 2, page_size, 128, dtype=dtype, device="cuda")
        kernels.attention_mixed(wide, pool, pool, wide.clone(), dev([0]), dev([0, 1, 1, 1]), dev([0, 0, 1, 2]),
                                dev([1]), dev([0]), dev([0, 1, 4]), dev([1, 3]),
                                torch.zeros(2, 2, dtype=torch.int32, device="cuda"), 2, 0.1)


@pytest.mark.parametrize("tile", [64, 32, 128])
def test_attention_prefill_far_key_and_causality(tile):
    """One early key is made to dominate for late queries only if they may see it; the query
    just before it must not feel it (a mask off by one would)."""
    from pagedserve_amd.ops import kernels

    heads, head_dim, page_size, total = 1, 64, 16, 300
    k_pool, v_pool, tables = _paged_fixture(torch.bfloat16, [total], heads, head_dim, page_size, 61)
    k_pool *= 0.05
    q = _rand((total, head_dim), torch.bfloat16, 62, 0.05)
    direction = torch.ones(head_dim, device="cuda") / 8.0
    target = 137
    page = int(tables[0, target // page_size])
    k_pool[page, 0, target % page_size] = (direction * 40).to(torch.bfloat16)
    for row in (136, 137, 138, 299):
        q[row] = (direction * 8).to(torch.bfloat16)
    out = torch.empty_like(q)

    def dev(values):
        return torch.tensor(values, dtype=torch.int32, device="cuda")

    starts = list(range(0, total, tile))
    kernels.attention_prefill(q, k_pool, v_pool, out, dev([0] * len(starts)), dev(starts),
                              dev([0, total]), dev([total]), tables, heads, head_dim ** -0.5,
                              query_tile=tile)
    value = v_pool[page, 0, target % page_size].float()
    for row in (137, 138, 299):
        torch.testing.assert_close(out[row].float(), value, atol=5e-3, rtol=5e-3)
    assert float((out[136].float() - value).abs().max()) > 0.3


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", [(1, 48, 64), (8, 2304, 768), (16, 100, 1024), (13, 257, 96), (17, 192, 768), (5, 64, 1600), (200, 320, 96),
                                   (12, 144, 1280), (16, 208, 1792), (9, 96, 1104), (16, 4800, 1600), (7, 80, 1800),
                                   (3, 4112, 64), (8, 6400, 1280), (13, 8192, 768), (5, 5000, 96), (11, 4700, 1024),
                                   (40, 4800, 1600), (64, 8192, 768), (24, 4500, 320), (17, 4112, 1792),
                                   (64, 6400, 1600), (33, 2000, 1280), (48, 100, 2048), (61, 72, 1088),
                                   (100, 768, 3072), (130, 1024, 1024), (224, 768, 3072), (200, 100, 2048), (65, 1600, 6400),
                                   (40, 2304, 768), (64, 3072, 768), (33, 100, 1024), (50, 8000, 64), (64, 16400, 64)])
@pytest.mark.parametrize("epilogue", ["none", "gelu_tanh", "residual"])
@pytest.mark.parametrize("rms", [False, True])
def test_linear_with_pending_norm(dtype, m, n, k, epilogue, rms):
    """Norm + product as one call: fused for bfloat16 with up to 16 rows, k <= 1792 and up to
    8,192 columns, two launches otherwise (17 to 64 rows: the normed rows travel in the lanes'
    operand order); with and without a row gather."""
    from pagedserve_amd.ops import kernels

    h = _rand((m + 3, k), torch.float32, 70, 2.0) + 0.5
    gamma = 1.0 + _rand((k,), torch.float32, 71, 0.2)
    beta = None if rms else _rand((k,), torch.float32, 72, 0.2)
    w = _rand((n, k), dtype, 73, 1.0 / math.sqrt(k))
    bias = _rand((n,), torch.float32, 74)
    for rows in (None, torch.randperm(m + 3)[:m].int().cuda()):
        source = h[:m] if rows is None else h
        count = m
        scratch = torch.empty((count, k), dtype=dtype, device="cuda")
        pending = kernels.PendingNorm(source, gamma, beta, 1e-6, rms, scratch, rows)
        picked = (source if rows is None else source[rows.long()]).double()
        if rms:
            normed = picked / torch.sqrt((picked * picked).mean(-1, keepdim=True) + 1e-6) * gamma.double()
        else:
            normed = F.layer_norm(picked, (k,), gamma.double(), beta.double(), 1e-6)
        if dtype == torch.bfloat16:
            normed = normed.to(torch.bfloat16).double()
        product = normed @ w.double().t() + bias.double()
        if epilogue == "residual":
            out = _rand((count, n), torch.float32, 75)
            expected = out.double() + product
        else:
            out = torch.full((count, n), float("nan"), dtype=dtype, device="cuda")
            expected = F.gelu(product, approximate="tanh") if epilogue == "gelu_tanh" else product
        kernels.linear(pending, w, bias, out, epilogue=epilogue)
        atol, rtol = (4e-5, 2e-5) if dtype == torch.float32 else (4e-2, 2e-2)
        torch.testing.assert_close(out.double(), expected, atol=atol, rtol=rtol)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,k,geometry", [(1, 64, (4, 2, 16, 8)), (9, 64, (4, 2, 16, 8)), (40, 64, (4, 2, 16, 8)),
                                          (150, 64, (4, 2, 16, 8)), (1, 100, (4, 2, 16, 8)), (9, 100, (4, 2, 16, 8)),
                                          (40, 100, (4, 2, 16, 8)), (150, 100, (4, 2, 16, 8)),
                                          (1500, 128, (12, 12, 64, 16)), (700, 64, (5, 1, 48, 12))])
def test_linear_scatters_keys_and_values(dtype, m, k, geometry):
    """A [q | k | v] product that also stores k and v in their pages equals product + kv_write
    (k = 100 takes the plain kernel, which scatters in a second launch; the large cases take
    other tile shapes of the tiled kernel)."""
    from pagedserve_amd.ops import kernels

    heads, kv_heads, head_dim, page_size = geometry
    q_cols, kv_cols = heads * head_dim, kv_heads * head_dim
    n = q_cols + 2 * kv_cols
    lens = [m // 2 + 3, m - m // 2 + 11] if m > 1 else [5]
    k_pool, v_pool, tables = _paged_fixture(dtype, lens, kv_heads, head_dim, page_size, 81)
    tok_item, tok_pos = [], []
    counts = [m // 2, m - m // 2] if m > 1 else [1]
    for item, (count, length) in enumerate(zip(counts, lens)):
        tok_item += [item] * count
        tok_pos += list(range(length - count, length))
    tok_item = torch.tensor(tok_item, dtype=torch.int32, device="cuda")
    tok_pos = torch.tensor(tok_pos, dtype=torch.int32, device="cuda")
    x = _rand((m, k), dtype, 82)
    w = _rand((n, k), dtype, 83, 1.0 / math.sqrt(k))
    bias = _rand((n,), torch.float32, 84)
    plain = torch.empty((m, n), dtype=dtype, device="cuda")
    kernels.linear(x, w, bias, plain)
    k_ref, v_ref = k_pool.clone(), v_pool.clone()
    kernels.kv_write(plain[:, q_cols:q_cols + kv_cols], plain[:, q_cols + kv_cols:], k_ref, v_ref, tok_item, tok_pos, tables)
    out = torch.empty_like(plain)
    kernels.linear(x, w, bias, out, scatter=(k_pool, v_pool, tok_item, tok_pos, tables, q_cols, kv_cols))
    torch.testing.assert_close(out, plain, atol=0, rtol=0)
    assert torch.equal(k_pool.view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                       k_ref.view(torch.int16 if dtype == torch.bfloat16 else torch.int32))
    assert torch.equal(v_pool.view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                       v_ref.view(torch.int16 if dtype == torch.bfloat16 else torch.int32))
    # a caller that reads keys and values from the pages alone: the query columns and the
    # pages are the same, the other columns may stay as they were
    k_pool.zero_()
    v_pool.zero_()
    k_ref.zero_()
    v_ref.zero_()
    kernels.kv_write(plain[:, q_cols:q_cols + kv_cols], plain[:, q_cols + kv_cols:], k_ref, v_ref, tok_item, tok_pos, tables)
    out = torch.zeros_like(plain)
    kernels.linear(x, w, bias, out, scatter=(k_pool, v_pool, tok_item, tok_pos, tables, q_cols, kv_cols),
                   scatter_only=True)
    torch.testing.assert_close(out[:, :q_cols], plain[:, :q_cols], atol=0, rtol=0)
    assert torch.equal(k_pool, k_ref) and torch.equal(v_pool, v_ref)


@pytest.mark.parametrize("m,geometry", [(8, (6, 3, 32, 8, 192)), (24, (6, 3, 32, 8, 192)), (64, (6, 3, 32, 8, 192)),
                                        (5, (25, 25, 64, 16, 1600)), (16, (40, 20, 64, 16, 704)),
                                        (64, (25, 25, 64, 16, 1600)), (37, (40, 20, 64, 16, 704))])
def test_norm_product_scatters_keys_and_values(m, geometry):
    """Norm, [q | k | v] product and the store into the pages as one call (one launch up to 16
    rows): the output is that of the norm and the product one after the other (up to the
    rounding of the normed rows), and the pages hold exactly the key and value columns of it.
    (The last two have more tiles of 16 columns than compute units: their columns are dealt
    out evenly over blocks of two tiles.)"""
    from pagedserve_amd.ops import kernels

    dtype = torch.bfloat16
    heads, kv_heads, head_dim, page_size, k = geometry
    q_cols, kv_cols = heads * head_dim, kv_heads * head_dim
    n = q_cols + 2 * kv_cols
    lens = [5 + index for index in range(m)]
    k_pool, v_pool, tables = _paged_fixture(dtype, lens, kv_heads, head_dim, page_size, 301)
    tok_item = torch.arange(m, dtype=torch.int32, device="cuda")
    tok_pos = torch.tensor([length - 1 for length in lens], dtype=torch.int32, device="cuda")
    h = _rand((m, k), torch.float32, 302, 2.0)
    gamma = 1.0 + _rand((k,), torch.float32, 303, 0.2)
    beta = _rand((k,), torch.float32, 304, 0.2)
    w = _rand((n, k), dtype, 305, 1.0 / math.sqrt(k))
    bias = _rand((n,), torch.float32, 306)
    packed = kernels.pack_decode_weight(w)
    normed = kernels.norm(h, gamma, beta, 1e-5, torch.empty((m, k), dtype=dtype, device="cuda"))
    plain = torch.empty((m, n), dtype=dtype, device="cuda")
    kernels.linear(normed, w, bias, plain, packed=packed)
    k_ref, v_ref = k_pool.clone(), v_pool.clone()
    out = torch.empty_like(plain)
    scratch = torch.empty((m, k), dtype=dtype, device="cuda")
    kernels.linear(kernels.PendingNorm(h, gamma, beta, 1e-5, False, scratch), w, bias, out, packed=packed,
                   scatter=(k_pool, v_pool, tok_item, tok_pos, tables, q_cols, kv_cols))
    torch.testing.assert_close(out.float(), plain.float(), atol=1e-2, rtol=5e-3)
    kernels.kv_write(out[:, q_cols:q_cols + kv_cols], out[:, q_cols + kv_cols:], k_ref, v_ref, tok_item, tok_pos, tables)
    view = torch.int16
    assert torch.equal(k_pool.view(view), k_ref.view(view)) and torch.equal(v_pool.view(view), v_ref.view(view))


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_decode_sixteen_waves(dtype):
    from pagedserve_amd.ops import kernels

    heads, head_dim, page_size = 12, 64, 16
    contexts = [1, 17, 300, 513, 1024, 700, 64, 999]
    k_pool, v_pool, tables = _paged_fixture(dtype, contexts, heads, head_dim, page_size, 91)
    q = _rand((len(contexts), heads * head_dim), dtype, 92)
    tok_item = torch.arange(len(contexts), dtype=torch.int32, device="cuda")
    tok_pos = torch.tensor([c - 1 for c in contexts], dtype=torch.int32, device="cuda")
    expected = _attention_expected(q, k_pool, v_pool, tables, tok_item, tok_pos, heads, 0.125)
    out = torch.full_like(q, float("nan"))
    kernels.attention_decode(q, k_pool, v_pool, out, tok_item, tok_pos, tables, heads, 0.125, 1, waves=16)
    atol, rtol = (3e-5, 3e-5) if dtype == torch.float32 else (2e-2, 2e-2)
    torch.testing.assert_close(out.double(), expected, atol=atol, rtol=rtol)
    # two and three ranges per request, merged by the reduce kernel
    for splits in (2, 3):
        partial = torch.full((len(contexts) * heads * splits * (head_dim + 2),), float("nan"), device="cuda")
        out = torch.full_like(q, float("nan"))
        kernels.attention_decode(q, k_pool, v_pool, out, tok_item, tok_pos, tables, heads, 0.125, splits,
                                 partial=partial, waves=16)
        torch.testing.assert_close(out.double(), expected, atol=atol, rtol=rtol)



PACKED_SHAPES = [(1, 50, 64), (8, 768, 3072), (8, 2304, 768), (16, 3072, 768), (17, 768, 768), (5, 1000, 320),
                 (64, 2304, 768), (48, 100, 3072), (9, 16411, 320), (16, 330, 1600), (40, 400, 1600), (300, 1000, 320),
                 (40, 1600, 6400), (33, 1290, 5184), (8, 4800, 1600), (3, 5008, 128),
                 (40, 4800, 1600), (64, 6400, 1280), (20, 4112, 64), (33, 5008, 192), (50, 8192, 832),
                 (100, 768, 3072), (190, 1024, 4096), (128, 768, 768)]


@pytest.mark.parametrize("m,n,k", PACKED_SHAPES)
@pytest.mark.parametrize("epilogue", ["none", "gelu_tanh", "residual"])
def test_linear_with_packed_weights(m, n, k, epilogue):
    """The copy of a weight matrix in the lanes' operand order gives the product that the
    matrix itself gives, bit for bit where partial sums are not added atomically: plain, with
    a pending norm, and with the key/value scatter; a row count that is no multiple of 16, a k
    beyond one round of loads, many rows (where the copy is not used)."""
    from pagedserve_amd.ops import kernels

    dtype = torch.bfloat16
    a = _rand((m, k), dtype, 210, 1.0)
    w = _rand((n, k), dtype, 211, 1.0 / math.sqrt(k))
    bias = _rand((n,), torch.float32, 212)
    packed = kernels.pack_decode_weight(w)
    assert packed is not None and packed.numel() == -(-n // 16) * 16 * k
    # the layout: row r, column c of w
    for r, c in ((0, 0), (n - 1, k - 1), (min(n - 1, 17), 37)):
        tile, row = divmod(r, 16)
        step, rest = divmod(c, 64)
        group, rest = divmod(rest, 16)
        half, e = divmod(rest, 8)
        assert packed[tile, step, half, group, row, e] == w[r, c]
    start = _rand((m, n), torch.float32, 213)

    def run(x, use_packed):
        out = start.clone() if epilogue == "residual" else torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
        kernels.linear(x, w, bias, out, epilogue=epilogue, packed=packed if use_packed else None)
        return out

    plain, with_copy = run(a, False), run(a, True)
    # (partial sums of ranges of k are added atomically: the skinny kernel's residual epilogue)
    atomic = epilogue == "residual" and k > 1024 and (m <= 64 or (m <= 224 and m * n <= 200000))
    if atomic:
        torch.testing.assert_close(with_copy, plain, atol=1e-4, rtol=1e-5)
    else:
        assert torch.equal(with_copy, plain)
    if m <= 64:
        h = _rand((m, k), torch.float32, 214, 2.0)
        gamma = 1.0 + _rand((k,), torch.float32, 215, 0.2)
        beta = _rand((k,), torch.float32, 216, 0.2)
        scratch = torch.empty((m, k), dtype=dtype, device="cuda")
        pending = lambda: kernels.PendingNorm(h, gamma, beta, 1e-5, False, scratch, None)
        plain, with_copy = run(pending(), False), run(pending(), True)
        if atomic:
            torch.testing.assert_close(with_copy, plain, atol=1e-4, rtol=1e-5)
        else:
            assert torch.equal(with_copy, plain)
    assert kernels.pack_decode_weight(_rand((32, 100), dtype, 217)) is None
    assert kernels.pack_decode_weight(_rand((32, 128), torch.float32, 218)) is None
    with pytest.raises(kernels.KernelError, match="packed copy"):
        kernels.linear(a, w, bias, run(a, False), epilogue=epilogue, packed=packed[:-1].contiguous() if packed.shape[0] > 1 else packed.float())


@pytest.mark.parametrize("m", [17, 32, 47, 64])
@pytest.mark.parametrize("inner,width", [(3072, 768), (320, 128), (1600, 1600), (6400, 1600)])
def test_linear_chain_with_packed_activations(m, inner, width):
    """Norm, product, activation, product as a decode step of 17 to 64 rows runs them: the
    normed rows and the hidden rows may travel in the lanes' operand order.  The result equals
    the chain with every buffer row by row, bit for bit up to the order of atomic adds."""
    from pagedserve_amd.ops import kernels

    dtype = torch.bfloat16
    h = _rand((m, width), torch.float32, 230, 2.0)
    gamma = 1.0 + _rand((width,), torch.float32, 231, 0.2)
    beta = _rand((width,), torch.float32, 232, 0.2)
    up = _rand((inner, width), dtype, 233, 1.0 / math.sqrt(width))
    down = _rand((width, inner), dtype, 234, 1.0 / math.sqrt(inner))
    up_bias, down_bias = _rand((inner,), torch.float32, 235), _rand((width,), torch.float32, 236)
    start = _rand((m, width), torch.float32, 237)
    workspace_rows = 80                      # room for the rows rounded up to 16

    def chain(allow_packed):
        scratch = torch.full((workspace_rows, width), float("nan"), dtype=dtype, device="cuda")
        hidden = torch.full((workspace_rows, inner), float("nan"), dtype=dtype, device="cuda")[:m]
        # a scratch slice without room behind it keeps the norm row by row
        normed = scratch[:m] if allow_packed else scratch[:m].clone()
        pending = kernels.PendingNorm(h, gamma, beta, 1e-5, False, normed, None)
        if allow_packed:
            _, was_packed = kernels.linear(pending, up, up_bias, hidden, epilogue="gelu_tanh", packed_out=True)
        else:
            kernels.linear(pending, up, up_bias, hidden, epilogue="gelu_tanh")
            was_packed = False
        out = start.clone()
        kernels.linear(hidden, down, down_bias, out, epilogue="residual", a_packed=was_packed)
        return out, was_packed

    plain, _ = chain(False)
    fast, was_packed = chain(True)
    # the first product is skinny when k <= 1024 or the rows are too few for the tiled kernel:
    # then its output travels packed
    assert was_packed == ((width <= 1024 or m <= 32) and inner % 64 == 0)
    torch.testing.assert_close(fast, plain, atol=1e-4, rtol=1e-5)
    reference = start.double() + F.gelu(
        (F.layer_norm(h.double(), (width,), gamma.double(), beta.double(), 1e-5).to(dtype).double()
         @ up.double().t() + up_bias.double()), approximate="tanh").to(dtype).double() @ down.double().t() + down_bias.double()
    assert (fast.double() - reference).abs().max().item() <= 2e-2 * reference.abs().max().item()


def _wide_entry():
    import ctypes

    from pagedserve_amd.ops import library

    lib = library.load_library()
    fn = lib.ps_gemm_nt_wide
    fn.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int] * 8 + [ctypes.c_void_p]
    fn.restype = ctypes.c_int
    return lib, fn


@pytest.mark.parametrize("m,n,k", [(256, 512, 1024), (300, 1000, 320), (333, 770, 64), (512, 3072, 1024), (97, 257, 128),
                                   (2048, 768, 3072), (700, 1600, 1600), (130, 2304, 704)])
@pytest.mark.parametrize("rows_per_block", [32, 64])
@pytest.mark.parametrize("epilogue", ["none", "gelu_tanh", "residual"])
def test_gemm_wide_block_shapes(m, n, k, rows_per_block, epilogue):
    """The product whose weights come out of the packed copy straight into registers, at each
    of its block shapes: one k tile and many (the ring of three and its last tiles), rows and
    columns that end inside a block, a column count that ends inside a 16-row tile of the copy."""
    from pagedserve_amd.ops import kernels

    if epilogue == "gelu_tanh" and rows_per_block != 64 and m > 400:
        pytest.skip("one block shape is enough for the activation at the larger sizes")
    lib, fn = _wide_entry()
    a = _rand((m, k), torch.bfloat16, 310, 1.0)
    w = _rand((n, k), torch.bfloat16, 311, 1.0 / math.sqrt(k))
    bias = _rand((n,), torch.float32, 312)
    packed = kernels.pack_decode_weight(w)
    product = a.double() @ w.double().t() + bias.double()
    if epilogue == "residual":
        out = _rand((m, n), torch.float32, 313)
        expected = out.double() + product
    else:
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        expected = F.gelu(product, approximate="tanh") if epilogue == "gelu_tanh" else product
    status = fn(a.data_ptr(), packed.data_ptr(), bias.data_ptr(), out.data_ptr(), m, n, k, a.stride(0),
                out.stride(0), 0 if out.dtype == torch.float32 else 1, kernels.EPILOGUES[epilogue],
                rows_per_block, torch.cuda.current_stream().cuda_stream)
    assert status == 0, lib.ps_last_error().decode()
    atol, rtol = (1e-4, 1e-5) if epilogue == "residual" else (4e-2, 2e-2)
    torch.testing.assert_close(out.double(), expected, atol=atol, rtol=rtol)


def test_linear_takes_the_wide_product_for_long_k():
    """Through ``kernels.linear``: many rows, a long k and the packed copy select the wide
    product (same result as without the copy, which takes the kernel with both operands in
    LDS), also with the key/value scatter behind it."""
    from pagedserve_amd.ops import kernels

    m, k = 1300, 1024
    heads, kv_heads, head_dim, page_size = 32, 16, 64, 16
    q_cols, kv_cols = heads * head_dim, kv_heads * head_dim
    n = q_cols + 2 * kv_cols          # 4,096 columns: 16 x 21 blocks of 64 rows x 256 columns
    lens = [700, 650]
    k_pool, v_pool, tables = _paged_fixture(torch.bfloat16, lens, kv_heads, head_dim, page_size, 320)
    tok_item = torch.tensor([0] * 680 + [1] * 620, dtype=torch.int32, device="cuda")
    tok_pos = torch.tensor(list(range(20, 700)) + list(range(30, 650)), dtype=torch.int32, device="cuda")
    x = _rand((m, k), torch.bfloat16, 321)
    w = _rand((n, k), torch.bfloat16, 322, 1.0 / math.sqrt(k))
    bias = _rand((n,), torch.float32, 323)
    packed = kernels.pack_decode_weight(w)
    plain = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    kernels.linear(x, w, bias, plain)
    k_ref, v_ref = k_pool.clone(), v_pool.clone()
    kernels.kv_write(plain[:, q_cols:q_cols + kv_cols], plain[:, q_cols + kv_cols:], k_ref, v_ref, tok_item, tok_pos, tables)
    out = torch.empty_like(plain)
    kernels.linear(x, w, bias, out, packed=packed,
                   scatter=(k_pool, v_pool, tok_item, tok_pos, tables, q_cols, kv_cols))
    expected = x.double() @ w.double().t() + bias.double()
    torch.testing.assert_close(out.double(), expected, atol=1e-2, rtol=5e-3)
    # the two kernels add the k tiles in the same order: the same bits
    assert torch.equal(out, plain)
    assert torch.equal(k_pool.view(torch.int16), k_ref.view(torch.int16))
    assert torch.equal(v_pool.view(torch.int16), v_ref.view(torch.int16))


@pytest.mark.parametrize("heads,kv_heads,head_dim,page_size", [(12, 12, 64, 16), (4, 2, 128, 12), (2, 1, 256, 16), (3, 3, 192, 8),
                                                               (5, 5, 64, 16)])
@pytest.mark.parametrize("count", [1, 2, 3, 5, 8, 16])
@pytest.mark.parametrize("splits", [1, 3, 8, 20, 64])
def test_attention_records_merged_inside_the_output_projection(heads, kv_heads, head_dim, page_size, count, splits):
    """Decode attention that leaves only its per-range records, and the output projection that
    merges them head by head: residual + softmax(q K^T) V W^T + bias in float64 over the
    gathered pages; contexts around page edges, ranges without keys, a width that ends inside
    a tile of 16 columns, rows beyond the count untouched; with one, two and four heads to a
    block (head counts that are no multiple of either), and with the library's own choice."""
    from pagedserve_amd.ops import kernels

    dtype = torch.bfloat16
    contexts = [1, 15, 16, 17, 31, 33, 128, 512, 700, 64, 2, 300, 90, 257, 1000, 48][:count]
    k_pool, v_pool, tables = _paged_fixture(dtype, contexts, kv_heads, head_dim, page_size, 401)
    q = _rand((count, heads * head_dim), dtype, 402)
    width = 200 if heads * head_dim > 200 else 40
    w = _rand((width, heads * head_dim), dtype, 403, 1.0 / math.sqrt(heads * head_dim))
    bias = _rand((width,), torch.float32, 404)
    packed = kernels.pack_decode_weight(w)
    tok_item = torch.arange(count, dtype=torch.int32, device="cuda")
    tok_pos = torch.tensor([c - 1 for c in contexts], dtype=torch.int32, device="cuda")
    scale = head_dim ** -0.5
    start = _rand((count + 2, width), torch.float32, 405)
    residual = start.clone()
    partial = torch.full((count * heads * splits * (head_dim + 2) + 8,), float("nan"), device="cuda")
    assert kernels.merge_linear_supported(dtype, count, head_dim, packed)
    kernels.attention_decode_partial(q, k_pool, v_pool, partial, tok_item, tok_pos, tables, heads, scale, splits)
    kernels.attention_merge_linear(partial, count, heads, head_dim, splits, w, packed, bias, residual)
    context = _attention_expected(q, k_pool, v_pool, tables, tok_item, tok_pos, heads, scale)
    expected = start[:count].double() + context.to(dtype).double() @ w.double().t() + bias.double()
    torch.testing.assert_close(residual[:count].double(), expected, atol=5e-4, rtol=5e-4)
    assert torch.equal(residual[count:], start[count:])
    for heads_per_block in (1, 2, 4):
        grouped = start.clone()
        kernels.attention_merge_linear(partial, count, heads, head_dim, splits, w, packed, bias, grouped,
                                       heads_per_block=heads_per_block)
        torch.testing.assert_close(grouped[:count].double(), expected, atol=5e-4, rtol=5e-4)
        # the same products, summed in another order
        torch.testing.assert_close(grouped[:count], residual[:count], atol=1e-4, rtol=1e-4)
        assert torch.equal(grouped[count:], start[count:])
    # rows named by a list land at the listed tokens
    chosen = torch.tensor(list(range(count))[::-1], dtype=torch.int32, device="cuda")
    residual = start.clone()
    kernels.attention_decode_partial(q, k_pool, v_pool, partial, tok_item, tok_pos, tables, heads, scale, splits,
                                     tok_list=chosen)
    kernels.attention_merge_linear(partial, count, heads, head_dim, splits, w, packed, bias, residual, tok_list=chosen)
    torch.testing.assert_close(residual[:count].double(), expected, atol=5e-4, rtol=5e-4)
    assert not kernels.merge_linear_supported(dtype, 17, head_dim, packed)
    assert not kernels.merge_linear_supported(dtype, count, 48, packed)
    assert not kernels.merge_linear_supported(torch.float32, count, head_dim, packed)


@pytest.mark.parametrize("m,n,k", [(1, 50257, 768), (8, 50257, 768), (16, 1000, 320), (20, 20011, 768), (32, 16411, 320),
                                   (5, 257, 64), (3, 41, 128), (9, 1000, 1600)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_head_product_chooses_the_tokens(m, n, k, with_bias):
    """The product of few bfloat16 rows also writes each row's column of the largest value,
    the lowest such column on a tie, as the sampling kernel does from the stored logits; three
    calls in a row with other inputs use the same keys, which every call leaves at zero."""
    from pagedserve_amd.ops import kernels

    dtype = torch.bfloat16
    w = _rand((n, k), dtype, 400, 1.0 / math.sqrt(k))
    bias = _rand((n,), torch.float32, 401) if with_bias else None
    packed = kernels.pack_decode_weight(w)
    top = kernels.TopChoice(m, "cuda")
    for call in range(3):
        a = _rand((m, k), dtype, 402 + call, 1.0)
        if call == 2:
            # a tie for the largest value of every row: the column that wins gets a twin, once
            # before and once behind it
            plain = torch.empty((m, n), dtype=torch.float32, device="cuda")
            kernels.linear(a, w, bias, plain, packed=packed)
            w = w.clone()
            for row in range(m):
                winner = int(plain[row].argmax())
                twin = (winner + 1 + 2 * row) % n if row % 2 else (winner - 1 - 2 * row) % n
                w[twin] = w[winner]
                if bias is not None:
                    bias[twin] = bias[winner]
            packed = kernels.pack_decode_weight(w)
        out = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
        tokens = torch.full((m + 3,), -7, dtype=torch.int32, device="cuda")
        _, chosen = kernels.linear(a, w, bias, out, packed=packed, choose=(top, tokens))
        assert chosen
        expected = torch.empty(m, dtype=torch.int32, device="cuda")
        kernels.sample(out, None, None, expected)
        assert torch.equal(tokens[:m], expected), (call, tokens[:m], expected)
        assert torch.equal(expected.long(), out.argmax(dim=1))
        assert (tokens[m:] == -7).all()
        assert int(top.keys.abs().sum()) == 0 and int(top.ticket.abs().sum()) == 0


def test_head_product_leaves_the_choice_where_it_cannot_make_it():
    """More rows than the kernels for few rows take, and the 32-bit path: the call says that it
    chose nothing, and the tokens stay as they were."""
    from pagedserve_amd.ops import kernels

    for dtype, m, n, k in ((torch.bfloat16, 40, 20011, 128), (torch.float32, 4, 300, 64)):
        a = _rand((m, k), dtype, 410, 1.0)
        w = _rand((n, k), dtype, 411, 1.0 / math.sqrt(k))
        out = torch.empty((m, n), dtype=torch.float32, device="cuda")
        tokens = torch.full((m,), -7, dtype=torch.int32, device="cuda")
        top = kernels.TopChoice(m, "cuda")
        _, chosen = kernels.linear(a, w, None, out, choose=(top, tokens))
        assert not chosen and (tokens == -7).all()
        torch.testing.assert_close(out.double(), a.double() @ w.double().t(), atol=2e-4, rtol=2e-4)
    with pytest.raises(kernels.KernelError, match="plain float output"):
        kernels.linear(a, w, None, out, epilogue="gelu_tanh", choose=(top, tokens))


def test_the_tile_that_the_step_lists_is_the_kernels_own():
    """Queries per tile and the widest block table of the tiled prefill kernel are constants of
    the HIP source; the Python side lists a step's tiles by the same numbers."""
    from pagedserve_amd.ops import kernels

    assert kernels.prefill_limits() == (kernels.PREFILL_TILE, kernels.PREFILL_TABLE_MAX)
    assert kernels.prefill_small_tile() == kernels.PREFILL_SMALL_TILE
    assert kernels.prefill_large_tile() == (kernels.PREFILL_LARGE_TILE, kernels.PREFILL_LARGE_TILE_HEAD_DIM)


def test_linear_checks_shared_by_the_layers_of_a_step():
    """The same call site of several layers in a step with a row count that none has seen: the
    first layer's call is checked and leaves its argument block for the step; the others take
    it with their own weights, bias and norm parameters from a block of their own, without a
    check, and give the bits of a checked call.  Sites that differ in a size or in which
    operands they have take the whole way."""
    from pagedserve_amd.ops import kernels

    k, n = 256, 192
    rows = _rand((64, k), torch.bfloat16, 730)
    h = _rand((64, k), torch.float32, 731)
    scratch = torch.empty((64, k), dtype=torch.bfloat16, device="cuda")
    out = torch.empty((64, n), dtype=torch.bfloat16, device="cuda")

    def site(seed, columns=n, with_bias=True):
        w = _rand((columns, k), torch.bfloat16, seed, k ** -0.5)
        return dict(w=w, bias=_rand((columns,), torch.float32, seed + 1) if with_bias else None,
                    packed=kernels.pack_decode_weight(w), gamma=_rand((k,), torch.float32, seed + 2),
                    beta=_rand((k,), torch.float32, seed + 3), memo={}, norm_memo={})

    def call(site_, count, shared=None, memo=True, normed=False, target=None):
        target = out if target is None else target
        target.zero_()
        x = kernels.PendingNorm(h[:count], site_["gamma"], site_["beta"], 1e-5, False, scratch[:count]) \
            if normed else rows[:count]
        kept = site_["norm_memo" if normed else "memo"] if memo else None
        kernels.linear(x, site_["w"], site_["bias"], target[:count, :site_["w"].shape[0]], epilogue="gelu_tanh",
                       packed=site_["packed"], memo=kept, shared=shared)
        return target[:count, :site_["w"].shape[0]].clone()

    layers = [site(740), site(750), site(760)]
    narrow, bare = site(770, columns=128), site(780, with_bias=False)
    for normed in (False, True):
        for each in layers + [narrow, bare]:
            call(each, 8, normed=normed)              # every site has been checked once, at other rows
        checks = []
        real_check = kernels._check
        kernels._check = lambda *args, **kwargs: (checks.append(args[1]), real_check(*args, **kwargs))[1]
        try:
            for count in (24, 40):
                shared = {}
                got = []
                for index, each in enumerate(layers):
                    del checks[:]
                    got.append(call(each, count, shared, normed=normed))
                    assert bool(checks) == (index == 0), (normed, count, index, checks)
                for each in (narrow, bare):           # other sizes, no bias: nothing to take over
                    del checks[:]
                    got.append(call(each, count, shared, normed=normed))
                    assert checks
                # a second step of these rows finds every block in the site's own memo
                del checks[:]
                again = [call(each, count, {}, normed=normed) for each in layers + [narrow, bare]]
                assert not checks
                for each, result, repeated in zip(layers + [narrow, bare], got, again):
                    plain = call(each, count, memo=False, normed=normed)
                    assert torch.equal(result.view(torch.int16), plain.view(torch.int16))
                    assert torch.equal(repeated.view(torch.int16), plain.view(torch.int16))
                assert not torch.equal(got[0], got[1]) and not torch.equal(got[1], got[2])
        finally:
            kernels._check = real_check
    # a site that is called with two sets of norm parameters (a block that runs twice in a step
    # has two pairs of pools in the same way): each call takes what it was checked with
    first, second = layers[0], dict(layers[0], gamma=layers[1]["gamma"], beta=layers[1]["beta"])
    call(second, 8, normed=True)
    shared = {}
    call(layers[2], 56, shared, normed=True)
    for each in (first, second, first):
        got = call(each, 56, shared, normed=True)
        plain = call(each, 56, memo=False, normed=True)
        assert torch.equal(got.view(torch.int16), plain.view(torch.int16))
    assert not torch.equal(call(first, 56, shared, normed=True), call(second, 56, shared, normed=True))


def test_linear_memo_of_a_call_site():
    """A call site's memo: the second call with the same row count and operand addresses goes
    straight to the library and gives the bits of the checked call; other rows or another
    buffer are other entries; the flags that the library reports (rows handed on in the packed
    order) come back on a hit as well."""
    from pagedserve_amd.ops import kernels

    k, n = 768, 256
    w = _rand((n, k), torch.bfloat16, 700, k ** -0.5)
    bias = _rand((n,), torch.float32, 701)
    packed = kernels.pack_decode_weight(w)
    rows = torch.empty((64, k), dtype=torch.bfloat16, device="cuda")
    out = torch.empty((64, n), dtype=torch.bfloat16, device="cuda")
    memo = {}
    for count in (8, 40, 8, 40, 8):
        rows[:count] = _rand((count, k), torch.bfloat16, 702 + len(memo))
        out.zero_()       # (rows handed on in the packed order leave the places of absent rows alone)
        got, handed_on = kernels.linear(rows[:count], w, bias, out[:count], epilogue="gelu_tanh", packed=packed,
                                        packed_out=True, memo=memo)
        plain = torch.zeros((64, n), dtype=torch.bfloat16, device="cuda")
        _, plain_handed_on = kernels.linear(rows[:count], w, bias, plain[:count], epilogue="gelu_tanh",
                                            packed=packed, packed_out=True)
        assert handed_on == plain_handed_on == (count > 16)
        assert torch.equal(got.view(torch.int16), plain[:count].view(torch.int16))
    assert len(memo) == 2 + 1      # (+ "site": the last checked block, for steps that share checks)
    other = torch.zeros((64, n), dtype=torch.bfloat16, device="cuda")
    kernels.linear(rows[:8], w, bias, other[:8], epilogue="gelu_tanh", packed=packed, packed_out=True, memo=memo)
    assert len(memo) == 3 + 1 and torch.equal(other[:8].view(torch.int16), out[:8].view(torch.int16))
    # a pending norm in front: keyed by the stream's rows, the row list and the scratch
    h = _rand((64, k), torch.float32, 710)
    gamma, beta = _rand((k,), torch.float32, 711), _rand((k,), torch.float32, 712)
    scratch = torch.empty((64, k), dtype=torch.bfloat16, device="cuda")
    memo = {}
    results = []
    for _ in range(2):
        result = torch.empty((8, n), dtype=torch.bfloat16, device="cuda")
        holder = out[:8]
        kernels.linear(kernels.PendingNorm(h[:8], gamma, beta, 1e-5, False, scratch[:8]), w, bias, holder, memo=memo)
        result.copy_(holder)
        results.append(result)
        if len(results) == 1:
            h[:8] = _rand((8, k), torch.float32, 720)    # the same addresses, other values: a hit reads them
    assert len(memo) == 1 + 1 and not torch.equal(results[0], results[1])
    # what is kept per call is nothing that the garbage collector has to walk (a stream of
    # requests leaves tens of thousands of entries behind)
    import gc
    assert all(type(kept) is bytes and not gc.is_tracked(kept) for kept in memo.values())
    expected = F.layer_norm(h[:8].double(), (k,), gamma.double(), beta.double(), 1e-5)
    expected = expected.to(torch.bfloat16).double() @ w.double().t() + bias.double()
    torch.testing.assert_close(results[1].double(), expected, atol=5e-3, rtol=5e-3)
