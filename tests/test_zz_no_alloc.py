"""The entry point that allocates nothing: ``ps_attention_decode_static``.

It is called through ``ctypes`` as a caller outside this package would, and compared with
``ps_attention_decode`` (partial results in a buffer of the caller) on two calls in a row on
one stream, the second with a smaller input: the second call finds the first one's partial
results in the shared array and must not be disturbed by them.  Then sizes beyond the array
are refused with an error that says so.
"""

import ctypes
from ctypes import c_float, c_int, c_int64, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu

STATIC_ARGS = [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p,
               c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int,
               c_int, c_int, c_int, c_void_p]
BUFFER_ARGS = [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64,
               c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
               c_int, c_float, c_int, c_int, c_int, c_int, c_void_p]
STATIC_FLOATS = 2 * 1024 * 1024


def _library():
    from pagedserve_amd.ops.library import find_or_build

    lib = ctypes.CDLL(find_or_build())
    lib.ps_attention_decode_static.argtypes = STATIC_ARGS
    lib.ps_attention_decode_static.restype = c_int
    lib.ps_attention_decode.argtypes = BUFFER_ARGS
    lib.ps_attention_decode.restype = c_int
    lib.ps_last_error.restype = ctypes.c_char_p
    return lib


def _case(dtype, contexts, heads, kv_heads, head_dim, page_size, seed):
    """Pools with every request's pages scattered, NaN wherever no request owns a slot."""
    g = torch.Generator().manual_seed(seed)
    pages_per = [-(-length // page_size) for length in contexts]
    total = sum(pages_per) + 3
    order = (torch.randperm(total - 1, generator=g) + 1).tolist()
    tables = torch.full((len(contexts), max(pages_per) + 1), -1, dtype=torch.int32)
    k_pool = torch.full((total, kv_heads, page_size, head_dim), float("nan"))
    v_pool = torch.full((total, kv_heads, page_size, head_dim), float("nan"))
    cursor = 0
    for index, (count, length) in enumerate(zip(pages_per, contexts)):
        for logical in range(count):
            page = order[cursor + logical]
            tables[index, logical] = page
            filled = min(page_size, length - logical * page_size)
            k_pool[page, :, :filled] = torch.randn((kv_heads, filled, head_dim), generator=g)
            v_pool[page, :, :filled] = torch.randn((kv_heads, filled, head_dim), generator=g)
        cursor += count
    q = torch.randn((len(contexts), heads * head_dim), generator=g)
    return (q.to(dtype).cuda(), k_pool.to(dtype).cuda(), v_pool.to(dtype).cuda(), tables.cuda(),
            torch.arange(len(contexts), dtype=torch.int32, device="cuda"),
            torch.tensor([c - 1 for c in contexts], dtype=torch.int32, device="cuda"))


def _both(lib, case, heads, kv_heads, head_dim, page_size, splits, dtype_code):
    q, k_pool, v_pool, tables, tok_item, tok_pos = case
    count = q.shape[0]
    stream = torch.cuda.current_stream().cuda_stream
    common = (tok_item.data_ptr(), tok_pos.data_ptr(), tables.data_ptr(), tables.shape[1], count,
              heads, kv_heads, head_dim, page_size, k_pool.shape[0], head_dim ** -0.5, 0, splits, 4,
              dtype_code, stream)
    got = torch.full_like(q, float("nan"))
    status = lib.ps_attention_decode_static(q.data_ptr(), q.stride(0), k_pool.data_ptr(),
                                            v_pool.data_ptr(), got.data_ptr(), got.stride(0),
                                            None, *common)
    assert status == 0, lib.ps_last_error().decode()
    expected = torch.full_like(q, float("nan"))
    partial = torch.full((count * heads * splits * (head_dim + 2),), float("nan"), device="cuda")
    status = lib.ps_attention_decode(q.data_ptr(), q.stride(0), k_pool.data_ptr(),
                                     v_pool.data_ptr(), expected.data_ptr(), expected.stride(0),
                                     partial.data_ptr(), partial.numel(), None, *common)
    assert status == 0, lib.ps_last_error().decode()
    torch.cuda.synchronize()
    return got, expected


@pytest.mark.parametrize("dtype,code", [(torch.float32, 0), (torch.bfloat16, 1)])
def test_static_scratch_decode_matches_the_buffer_variant_twice(dtype, code):
    lib = _library()
    heads, kv_heads, head_dim, page_size = 6, 2, 48, 16
    first = _case(dtype, [700, 33, 1, 512, 129, 64, 17], heads, kv_heads, head_dim, page_size, 3)
    got, expected = _both(lib, first, heads, kv_heads, head_dim, page_size, 7, code)
    assert torch.isfinite(expected.float()).all()
    # the same kernels in the same order on the same inputs: the results are the same bits
    assert torch.equal(got, expected)
    # the second call is smaller (fewer requests, fewer ranges) and finds the first one's
    # partial results in the array
    second = _case(dtype, [90, 300], heads, kv_heads, head_dim, page_size, 4)
    got, expected = _both(lib, second, heads, kv_heads, head_dim, page_size, 3, code)
    assert torch.isfinite(expected.float()).all()
    assert torch.equal(got, expected)
    # and against the formula itself
    q, k_pool, v_pool, tables, _, tok_pos = second
    for index in range(q.shape[0]):
        length = int(tok_pos[index]) + 1
        pages = tables[index, : -(-length // page_size)].long()
        keys = k_pool[pages].permute(1, 0, 2, 3).reshape(kv_heads, -1, head_dim)[:, :length]
        values = v_pool[pages].permute(1, 0, 2, 3).reshape(kv_heads, -1, head_dim)[:, :length]
        keys = keys.double().repeat_interleave(heads // kv_heads, 0)
        values = values.double().repeat_interleave(heads // kv_heads, 0)
        scores = torch.einsum("hd,hkd->hk", q[index].double().reshape(heads, head_dim), keys)
        weights = torch.softmax(scores * head_dim ** -0.5, dim=-1)
        formula = torch.einsum("hk,hkd->hd", weights, values).reshape(-1)
        tolerance = 3e-5 if dtype == torch.float32 else 2e-2
        torch.testing.assert_close(got[index].double(), formula, atol=tolerance, rtol=tolerance)


def test_static_scratch_decode_refuses_what_does_not_fit():
    lib = _library()
    heads, kv_heads, head_dim, page_size, splits = 64, 64, 256, 16, 64
    count = STATIC_FLOATS // (heads * splits * (head_dim + 2)) + 1
    q = torch.zeros((count, heads * head_dim), device="cuda")
    pool = torch.zeros((2, kv_heads, page_size, head_dim), device="cuda")
    tables = torch.zeros((count, 1), dtype=torch.int32, device="cuda")
    index = torch.zeros(count, dtype=torch.int32, device="cuda")
    status = lib.ps_attention_decode_static(
        q.data_ptr(), q.stride(0), pool.data_ptr(), pool.data_ptr(), q.data_ptr(), q.stride(0),
        None, index.data_ptr(), index.data_ptr(), tables.data_ptr(), 1, count, heads, kv_heads,
        head_dim, page_size, 2, 1.0, 0, splits, 4, 0, torch.cuda.current_stream().cuda_stream)
    assert status != 0
    message = lib.ps_last_error().decode()
    assert "static scratch" in message and str(STATIC_FLOATS) in message
