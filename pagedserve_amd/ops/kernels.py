"""Python faces of the HIP kernels: shape checks on the host, then one C call.

Every function takes torch tensors that live on the GPU, checks what the kernel and
its grid assume (devices, dtypes, contiguity, extents) and launches on torch's
current stream.  There is no other implementation behind these functions.
"""

import ctypes
from ctypes import c_float, c_int, c_int64, c_void_p

import torch

from .library import load_library

F32 = 0
BF16 = 1

EPILOGUES = {"none": 0, "gelu_tanh": 1, "gelu_erf": 2, "residual": 3}

_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}

_SIGNATURES = {
    "ps_embed": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                 c_int, c_int, c_int, c_float, c_int, c_void_p],
    "ps_norm": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_int,
                c_int, c_void_p],
    "ps_gemm_nt": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                   c_int, c_int, c_int, c_void_p],
    "ps_kv_write": [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                    c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ps_attention_rowwise": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
                             c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                             c_int, c_float, c_int, c_int, c_void_p],
    "ps_attention_decode": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
                            c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                            c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_int,
                            c_void_p],
    "ps_attention_decode_partial": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
                                    c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                    c_int, c_int, c_float, c_int, c_int, c_int, c_int, c_void_p],
    "ps_attention_merge_linear": [c_void_p, c_int64, c_void_p, c_int, c_int, c_int, c_int, c_void_p,
                                  c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p],
    "ps_attention_tiled_f32": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
                               c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                               c_int, c_int, c_int, c_float, c_int, c_void_p],
    "ps_attention_prefill": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
                             c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                             c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_int, c_void_p],
    "ps_attention_mixed": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int,
                           c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                           c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_void_p],
    "ps_sample": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
}

_BOUND = {}


def _fn(name):
    fn = _BOUND.get(name)
    if fn is None:
        fn = getattr(load_library(), name)
        fn.argtypes = _SIGNATURES[name]
        fn.restype = c_int
        _BOUND[name] = fn
    return fn


class KernelError(RuntimeError):
    pass


def _call(name, *args):
    status = _fn(name)(*args)
    if status != 0:
        message = load_library().ps_last_error().decode("utf-8", "replace")
        raise KernelError(f"{name} failed ({status}): {message}")


_STREAM_HANDLE = None


def _stream():
    if _STREAM_HANDLE is not None:
        return _STREAM_HANDLE
    return torch.cuda.current_stream().cuda_stream


class on_stream:
    """While active, every kernel of this module is launched on ``stream`` (which must be
    torch's current stream, so that torch's own work keeps its order with them) without asking
    torch for it at each launch: that question costs as much as the rest of a launch."""

    def __init__(self, stream: "torch.cuda.Stream"):
        self.handle = stream.cuda_stream

    def __enter__(self):
        global _STREAM_HANDLE
        self.previous = _STREAM_HANDLE
        _STREAM_HANDLE = self.handle
        return self

    def __exit__(self, *exc):
        global _STREAM_HANDLE
        _STREAM_HANDLE = self.previous
        return False


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise KernelError(f"dtype {dtype} is not supported by the kernels "
                          "(float32 and bfloat16 are)") from None


def _check(tensor, name, dtype=None, ndim=None):
    if not isinstance(tensor, torch.Tensor):
        raise KernelError(f"{name} must be a tensor")
    if not tensor.is_cuda:
        raise KernelError(f"{name} must live on the GPU; the engine has no CPU path")
    if dtype is not None and tensor.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, got {tensor.dtype}")
    if ndim is not None and tensor.ndim != ndim:
        raise KernelError(f"{name} must have {ndim} dimensions, got shape {tuple(tensor.shape)}")
    return tensor


def _rows(tensor, name):
    """2-D tensor with unit stride in its last dimension; returns the row stride."""
    if tensor.ndim != 2 or (tensor.shape[1] > 1 and tensor.stride(1) != 1):
        raise KernelError(f"{name} must be 2-D with contiguous rows, got shape "
                          f"{tuple(tensor.shape)} strides {tuple(tensor.stride())}")
    return tensor.stride(0) if tensor.shape[0] > 1 else max(tensor.stride(0), tensor.shape[1])


def _ptr(tensor):
    return 0 if tensor is None else tensor.data_ptr()


def embed(table, pos_table, ids, positions, out, token_src=None, carried=None, scale=1.0):
    """out[t] = scale * table[id(t)] + pos_table[positions[t]] as float (pos_table may be None).
    id(t) is ``ids[t]``, or ``carried[token_src[t]]`` where ``token_src[t] >= 0``: a token
    that an earlier step chose on the device."""
    _check(table, "table", ndim=2)
    _check(ids, "ids", torch.int32, 1)
    _check(out, "out", torch.float32, 2)
    tokens = ids.numel()
    width = table.shape[1]
    if not (table.is_contiguous() and out.is_contiguous() and ids.is_contiguous()):
        raise KernelError("embed: tensors must be contiguous")
    if out.shape[0] < tokens or out.shape[1] != width:
        raise KernelError(f"embed: out {tuple(out.shape)} does not fit {tokens} rows of {width}")
    max_positions = 0
    if pos_table is not None:
        _check(pos_table, "pos_table", table.dtype, 2)
        _check(positions, "positions", torch.int32, 1)
        if pos_table.shape[1] != width or not pos_table.is_contiguous():
            raise KernelError("embed: position table must be contiguous and as wide as the table")
        if positions.numel() != tokens or not positions.is_contiguous():
            raise KernelError("embed: one position per token is needed")
        max_positions = pos_table.shape[0]
    if token_src is not None:
        _check(token_src, "token_src", torch.int32, 1)
        _check(carried, "carried", torch.int32, 1)
        if token_src.numel() != tokens or not token_src.is_contiguous() or not carried.is_contiguous():
            raise KernelError("embed: one source index per token is needed")
    _call("ps_embed", table.data_ptr(), _ptr(pos_table), ids.data_ptr(), _ptr(token_src),
          _ptr(carried if token_src is not None else None),
          _ptr(positions if pos_table is not None else None), out.data_ptr(), tokens, width,
          table.shape[0], max_positions, float(scale), dtype_code(table.dtype), _stream())
    return out


def norm(x, gamma, beta, eps, out, rows=None, rms=False):
    """out[r] = norm(x[rows[r]]) * gamma + beta; statistics in float."""
    _check(x, "x", torch.float32, 2)
    _check(gamma, "gamma", torch.float32, 1)
    _check(out, "out", ndim=2)
    width = x.shape[1]
    if not (x.is_contiguous() and out.is_contiguous() and gamma.is_contiguous()):
        raise KernelError("norm: tensors must be contiguous")
    if gamma.numel() != width or out.shape[1] != width:
        raise KernelError("norm: widths of x, gamma and out differ")
    if beta is not None:
        _check(beta, "beta", torch.float32, 1)
        if beta.numel() != width or not beta.is_contiguous():
            raise KernelError("norm: beta does not match the width")
    if rows is not None:
        _check(rows, "rows", torch.int32, 1)
        n_rows = rows.numel()
    else:
        n_rows = x.shape[0]
    if out.shape[0] < n_rows:
        raise KernelError("norm: out has too few rows")
    _call("ps_norm", x.data_ptr(), _ptr(rows), gamma.data_ptr(), _ptr(beta), out.data_ptr(),
          n_rows, width, float(eps), 1 if rms else 0, dtype_code(out.dtype), _stream())
    return out


def gemm_nt(a, w, bias, out, epilogue="none"):
    """out[m, n] = epilogue(sum_k a[m, k] w[n, k] + bias[n]).

    ``epilogue='residual'`` adds the product into the float tensor ``out``."""
    _check(a, "a", ndim=2)
    _check(w, "w", a.dtype, 2)
    _check(out, "out", ndim=2)
    lda = _rows(a, "a")
    ldc = _rows(out, "out")
    m, k = a.shape
    n = w.shape[0]
    if w.shape[1] != k or not w.is_contiguous():
        raise KernelError(f"gemm_nt: w {tuple(w.shape)} must be contiguous [n, {k}]")
    if out.shape[0] != m or out.shape[1] != n:
        raise KernelError(f"gemm_nt: out {tuple(out.shape)} must be [{m}, {n}]")
    if bias is not None:
        _check(bias, "bias", torch.float32, 1)
        if bias.numel() != n or not bias.is_contiguous():
            raise KernelError("gemm_nt: bias does not match n")
    if epilogue not in EPILOGUES:
        raise KernelError(f"gemm_nt: unknown epilogue {epilogue!r}")
    _call("ps_gemm_nt", a.data_ptr(), w.data_ptr(), _ptr(bias), out.data_ptr(), m, n, k, lda, ldc,
          dtype_code(a.dtype), dtype_code(out.dtype), EPILOGUES[epilogue], _stream())
    return out


class _LinearArgs(ctypes.Structure):
    _fields_ = [
        ("a", c_void_p), ("w", c_void_p), ("bias", c_void_p), ("c", c_void_p),
        ("m", c_int), ("n", c_int), ("k", c_int), ("lda", c_int), ("ldc", c_int),
        ("dtype", c_int), ("c_dtype", c_int), ("epilogue", c_int),
        ("norm_h", c_void_p), ("norm_rows", c_void_p), ("gamma", c_void_p), ("beta", c_void_p),
        ("norm_out", c_void_p), ("eps", c_float), ("rms", c_int), ("ldh", c_int),
        ("k_pool", c_void_p), ("v_pool", c_void_p), ("tok_item", c_void_p), ("tok_pos", c_void_p),
        ("tables", c_void_p),
        ("table_width", c_int), ("q_cols", c_int), ("kv_cols", c_int), ("head_dim", c_int),
        ("kv_heads", c_int), ("page_size", c_int), ("num_pages", c_int),
        ("w_packed", c_void_p),
        ("a_packed", c_int), ("c_packed_request", c_int), ("c_rows", c_int),
        ("norm_out_rows", c_int), ("c_layout", ctypes.POINTER(c_int)),
        ("top_tokens", c_void_p), ("top_keys", c_void_p), ("top_ticket", c_void_p),
        ("top_done", ctypes.POINTER(c_int)),
        ("scatter_only", c_int),
    ]


class PendingNorm:
    """A norm that has not run yet: the float rows, the parameters, and scratch for the
    normed rows.  ``linear`` fuses it into the product when the kernel can; ``materialize``
    runs it on its own."""

    def __init__(self, h, gamma, beta, eps, rms, scratch, rows=None):
        self.h = h
        self.gamma = gamma
        self.beta = beta
        self.eps = float(eps)
        self.rms = bool(rms)
        self.scratch = scratch
        self.rows = rows

    @property
    def count(self):
        return self.rows.numel() if self.rows is not None else self.h.shape[0]

    def materialize(self):
        count = self.count
        return norm(self.h, self.gamma, self.beta, self.eps, self.scratch[:count], rows=self.rows,
                    rms=self.rms)[:count]


def pack_decode_weight(w):
    """A second copy of the bfloat16 matrix ``w [n, k]`` (k a multiple of 64, else None) for
    the products of few rows: rows padded to a multiple of 16, every 16 x 64 tile laid out in
    the order in which a wave's lanes hold the MFMA operand (``csrc/pagedserve_hip.h`` gives the
    formula), so that a wave's load is 1 KB of consecutive memory.  Made once when weights are
    bound; it doubles the memory of the matrices it is made for."""
    if w.dtype != torch.bfloat16 or w.ndim != 2 or w.shape[1] % 64 != 0 or not w.is_cuda:
        return None
    n, k = w.shape
    padded_rows = -(-n // 16) * 16
    source = w if padded_rows == n else torch.cat([w, w.new_zeros((padded_rows - n, k))])
    # [tile, row in tile, step, lane group, half, 8] -> [tile, step, half, lane group, row, 8]
    return source.view(padded_rows // 16, 16, k // 64, 4, 2, 8).permute(0, 2, 4, 3, 1, 5).contiguous()


def _row_capacity(tensor, columns: int) -> int:
    """Rows of ``columns`` values that fit from the tensor's first element to the end of its
    storage (a workspace slice ``buffer[:tokens]`` has room for the whole buffer)."""
    if tensor.ndim != 2 or tensor.shape[1] != columns or not tensor.is_contiguous():
        return 0
    elements = tensor.untyped_storage().nbytes() // tensor.element_size() - tensor.storage_offset()
    return int(elements // columns)


TOP_SLOTS = 16   # keys per row of a TopChoice (csrc/linear.h: PS_TOP_SLOTS)


class TopChoice:
    """What a product needs to choose each row's token in its own epilogue: 16 keys per row
    and 17 tickets, zero between launches (the kernel leaves them so).  One per stream: launches
    that share it must not overlap."""

    def __init__(self, rows: int, device):
        self.rows = int(rows)
        # 256 bytes from key to key and from ticket to ticket (csrc/linear.h: PS_TOP_STRIDE)
        self.keys = torch.zeros(self.rows * TOP_SLOTS * 32, dtype=torch.int64, device=device)
        self.ticket = torch.zeros((1 + TOP_SLOTS) * 64, dtype=torch.int32, device=device)


_MEMO_LIMIT = 512
# What a memoized call keeps is the bytes of its argument block, nothing that the garbage
# collector has to walk (a stream of requests leaves tens of thousands of blocks behind; as
# ctypes structures with two result integers each they made a full collection take 90 ms, in
# the middle of a step).  The two result integers that a block points at are these, shared by
# all memoized calls: a call's results are read before the next call is made.
_MEMO_LAYOUT = c_int(0)
_MEMO_DONE = c_int(0)


def _memo_key(x, out, scatter, a_packed, choose):
    """What may differ between two calls of one call site, in two parts: the row count and
    the addresses of the step's buffers and index arrays, which the same call site of another
    layer meets too, and the addresses that tell the site's own operands apart where it may be
    called with several (its norm's parameters; the cache pools, of which a block that runs
    twice in a step has two pairs).  Weights, bias and flags are the site's own and in neither."""
    if isinstance(x, PendingNorm):
        step = (x.count, x.h.data_ptr(), _ptr(x.rows), x.scratch.data_ptr(), out.data_ptr())
        site = (x.gamma.data_ptr(),)
    else:
        step = (x.shape[0], x.data_ptr(), x.stride(0), out.data_ptr(), a_packed)
        site = ()
    if scatter is not None:
        step += (scatter[2].data_ptr(), scatter[3].data_ptr(), scatter[4].data_ptr())
        site += (scatter[0].data_ptr(), scatter[1].data_ptr())
    if choose is not None:
        step += (choose[1].data_ptr(),)
    return step, site


def _field_ranges(names):
    return tuple((getattr(_LinearArgs, name).offset,
                  getattr(_LinearArgs, name).offset + getattr(_LinearArgs, name).size) for name in names)


# The fields of an argument block by who decides them.  The site's own: its weights and bias,
# equal on every call, and the norm parameters and pools that the call was made with (the second
# part of ``_memo_key``).  The step's: equal for the same call site of every layer within a step
# (the layers share the workspace and the index arrays).  All others are sizes, codes and flags.
_SITE_FIELDS = ("w", "bias", "gamma", "beta", "k_pool", "v_pool", "w_packed")
_STEP_FIELDS = ("a", "c", "m", "lda", "ldc", "norm_h", "norm_rows", "norm_out", "tok_item", "tok_pos",
                "tables", "table_width", "a_packed", "c_rows", "norm_out_rows", "c_layout",
                "top_tokens", "top_keys", "top_ticket", "top_done")
_SITE_RANGES = _field_ranges(_SITE_FIELDS)
_SIZE_RANGES = _field_ranges(name for name, _ in _LinearArgs._fields_
                             if name not in _SITE_FIELDS and name not in _STEP_FIELDS)
_NULL = bytes(ctypes.sizeof(c_void_p))


def _sibling_block(sibling: bytes, own: bytes):
    """The argument block of this site for a step whose block for the same call site of another
    layer is ``sibling`` (checked in this step, same buffers and index arrays), from ``own``, a
    checked block of this site for other rows: the step's fields of the one with the site's
    fields of the other.  None where the two sites do not agree in every size, code and flag,
    or in which of their own operands they have at all."""
    for begin, end in _SIZE_RANGES:
        if sibling[begin:end] != own[begin:end]:
            return None
    block = bytearray(sibling)
    for begin, end in _SITE_RANGES:
        if (sibling[begin:end] == _NULL) != (own[begin:end] == _NULL):
            return None
        block[begin:end] = own[begin:end]
    return bytes(block)


def linear(x, w, bias, out, epilogue="none", scatter=None, packed=None, a_packed=False,
           packed_out=False, choose=None, scatter_only=False, memo=None, shared=None):
    """out = epilogue(x w^T + bias) where ``x`` is a tensor or a ``PendingNorm``.

    ``scatter = (k_pool, v_pool, tok_item, tok_pos, tables, q_cols, kv_cols)`` also stores the
    key and value columns of a ``[q | k | v]`` output into their cache pages.  ``packed`` is
    ``pack_decode_weight(w)`` or None; the kernels for few rows read it instead of ``w``.
    ``scatter_only=True`` says that nobody reads the key and value columns of ``out``: a kernel
    may then leave them unwritten (unspecified afterwards), which the one for many rows does.

    Between two products of 17 to 64 rows the activations may travel in the order in which the
    second one's lanes hold them (``csrc/linear.h: packed_offset``).  ``packed_out=True`` allows
    that for ``out`` (whose storage must have room for the rows rounded up to 16) and makes the
    call return ``(out, written_packed)``; the buffer then goes to the next call with
    ``a_packed=written_packed`` and means nothing to anyone else.

    ``choose = (TopChoice, tokens)`` asks for ``tokens[r]`` = the column of the largest value of
    row ``r`` of a float ``out`` (the lowest on ties), as ``sample`` gives it without a
    temperature; the call then returns ``(out, chosen)``, and where ``chosen`` is False the
    kernel that ran could not do it and ``tokens`` is untouched.

    ``memo``: a dict that belongs to ONE call site, whose ``w``, ``bias``, ``packed``, epilogue
    and flags are the same on every call (a part's product).  The checked argument block of a
    call is kept in it under the row count and the addresses of the other operands, and a call
    that finds its block goes straight to the library: checking and filling the block costs
    the host more than the launch, and a step that is not replayed from a graph issues four
    such calls a layer.  Whoever binds other weights clears the dict; and because a block also
    holds the room behind the addresses (rows that a buffer has space for), a site keeps one
    dict per set of buffers (``parts.base.site_memo``).

    ``shared``: a dict that lives for ONE step and is handed to the calls of all layers.  A
    step with a row count that a site has not seen finds nothing in the site's memo; but the
    same call site of the layer before has just had its block checked for the very same
    buffers and index arrays, and left it here.  This site's block is then that one with the
    site's own operands (weights, bias, norm parameters, pools) taken from a block that this
    site was checked with for the same norm parameters and pools, provided the two agree in
    every size, code and flag: one check per step instead of one per layer."""
    if memo is not None:
        step_key, site_key = _memo_key(x, out, scatter, a_packed, choose)
        key = step_key + site_key
        kept = memo.get(key)
        if kept is None and shared is not None:
            # (a checked block of this site with these very norm parameters and pools)
            sibling, own = shared.get(step_key), memo.get(("site",) + site_key)
            if sibling is not None and own is not None:
                kept = _sibling_block(sibling, own)
                if kept is not None:
                    if len(memo) >= _MEMO_LIMIT:
                        memo.clear()
                        memo[("site",) + site_key] = own
                    memo[key] = kept
        if kept is not None:
            # (the library reads the block and writes through the pointers in it only)
            status = _BOUND["ps_linear_bytes"](kept, _stream())
            if status != 0:
                raise KernelError(f"ps_linear failed ({status}): "
                                  f"{load_library().ps_last_error().decode('utf-8', 'replace')}")
            if packed_out:
                return out, bool(_MEMO_LAYOUT.value)
            if choose is not None:
                return out, bool(_MEMO_DONE.value)
            return out
    _check(w, "w", ndim=2)
    _check(out, "out", ndim=2)
    n, k = w.shape
    if not w.is_contiguous():
        raise KernelError("linear: w must be contiguous")
    args = _LinearArgs()
    if isinstance(x, PendingNorm):
        _check(x.h, "norm input", torch.float32, 2)
        _check(x.gamma, "gamma", torch.float32, 1)
        if x.h.shape[1] != k or x.gamma.numel() != k or not x.h.is_contiguous():
            raise KernelError("linear: norm input rows must be contiguous and k wide")
        if x.beta is not None:
            _check(x.beta, "beta", torch.float32, 1)
        m = x.count
        _check(x.scratch, "norm scratch", w.dtype, 2)
        if x.scratch.shape[0] < m or x.scratch.shape[1] != k or not x.scratch.is_contiguous():
            raise KernelError("linear: norm scratch must be contiguous [>= m, k]")
        if x.rows is not None:
            _check(x.rows, "rows", torch.int32, 1)
        args.norm_h = x.h.data_ptr()
        args.norm_rows = _ptr(x.rows)
        args.gamma = x.gamma.data_ptr()
        args.beta = _ptr(x.beta)
        args.norm_out = x.scratch.data_ptr()
        args.eps = x.eps
        args.rms = 1 if x.rms else 0
        args.ldh = k
        args.lda = k
        args.norm_out_rows = _row_capacity(x.scratch, k)
        if a_packed:
            raise KernelError("linear: a pending norm has no packed rows")
    else:
        _check(x, "x", w.dtype, 2)
        if x.shape[1] != k:
            raise KernelError(f"linear: x {tuple(x.shape)} does not match w {tuple(w.shape)}")
        m = x.shape[0]
        args.a = x.data_ptr()
        args.lda = _rows(x, "x")
        if a_packed:
            if _row_capacity(x, k) < -(-m // 16) * 16:
                raise KernelError("linear: packed input rows need a dense buffer with room for "
                                  "the row count rounded up to 16")
            args.a_packed = 1
    if out.shape[0] != m or out.shape[1] != n:
        raise KernelError(f"linear: out {tuple(out.shape)} must be [{m}, {n}]")
    if bias is not None:
        _check(bias, "bias", torch.float32, 1)
        if bias.numel() != n or not bias.is_contiguous():
            raise KernelError("linear: bias does not match n")
    if epilogue not in EPILOGUES:
        raise KernelError(f"linear: unknown epilogue {epilogue!r}")
    args.w = w.data_ptr()
    if packed is not None:
        if (packed.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or not packed.is_cuda
                or not packed.is_contiguous() or k % 64 != 0
                or packed.numel() != -(-n // 16) * 16 * k):
            raise KernelError(f"linear: the packed copy does not belong to w {tuple(w.shape)}")
        args.w_packed = packed.data_ptr()
    args.bias = _ptr(bias)
    args.c = out.data_ptr()
    args.m, args.n, args.k = m, n, k
    args.ldc = _rows(out, "out")
    args.dtype = dtype_code(w.dtype)
    args.c_dtype = dtype_code(out.dtype)
    args.epilogue = EPILOGUES[epilogue]
    if scatter is not None:
        k_pool, v_pool, tok_item, tok_pos, tables, q_cols, kv_cols = scatter
        pages, kv_heads, page_size, head_dim = _check_pools(k_pool, v_pool, w.dtype)
        _check_step_index(tok_item, tok_pos, tables, m)
        args.k_pool = k_pool.data_ptr()
        args.v_pool = v_pool.data_ptr()
        args.tok_item = tok_item.data_ptr()
        args.tok_pos = tok_pos.data_ptr()
        args.tables = tables.data_ptr()
        args.table_width = tables.shape[1]
        args.q_cols, args.kv_cols = int(q_cols), int(kv_cols)
        args.head_dim, args.kv_heads = head_dim, kv_heads
        args.page_size, args.num_pages = page_size, pages
        args.scatter_only = 1 if scatter_only else 0
    layout = _MEMO_LAYOUT if memo is not None else c_int(0)
    if packed_out:
        args.c_packed_request = 1
        args.c_rows = _row_capacity(out, n)
        args.c_layout = ctypes.pointer(layout)
    done = _MEMO_DONE if memo is not None else c_int(0)
    if choose is not None:
        top, tokens = choose
        _check(tokens, "tokens", torch.int32, 1)
        if out.dtype != torch.float32 or epilogue != "none" or scatter is not None or packed_out:
            raise KernelError("linear: tokens are chosen from a plain float output")
        if tokens.numel() < m or not tokens.is_contiguous():
            raise KernelError(f"linear: {m} rows need as many tokens")
        if top.rows >= m:            # (more rows than there are keys for: the caller samples)
            args.top_tokens = tokens.data_ptr()
            args.top_keys = top.keys.data_ptr()
            args.top_ticket = top.ticket.data_ptr()
            args.top_done = ctypes.pointer(done)
    lib = load_library()
    fn = _BOUND.get("ps_linear")
    if fn is None:
        lib.ps_linear_args_size.restype = c_int
        if lib.ps_linear_args_size() != ctypes.sizeof(_LinearArgs):
            raise KernelError("ps_linear: the argument block of this module "
                              f"({ctypes.sizeof(_LinearArgs)} bytes) is not the library's "
                              f"({lib.ps_linear_args_size()} bytes); rebuild the library")
        fn = lib.ps_linear
        fn.argtypes = [ctypes.POINTER(_LinearArgs), c_void_p]
        fn.restype = c_int
        _BOUND["ps_linear"] = fn
        # the same entry point taking the block as a bytes object (a second function object:
        # argument types belong to the object, not to the symbol)
        from_bytes = lib["ps_linear"]
        from_bytes.argtypes = [ctypes.c_char_p, c_void_p]
        from_bytes.restype = c_int
        _BOUND["ps_linear_bytes"] = from_bytes
    status = fn(ctypes.byref(args), _stream())
    if status != 0:
        raise KernelError(f"ps_linear failed ({status}): {lib.ps_last_error().decode('utf-8', 'replace')}")
    if memo is not None:
        if len(memo) >= _MEMO_LIMIT:
            memo.clear()
        memo[key] = memo[("site",) + site_key] = bytes(args)
        if shared is not None:
            shared[step_key] = memo[key]
    if packed_out:
        return out, bool(layout.value)
    if choose is not None:
        return out, bool(done.value)
    return out


def _check_pools(k_pool, v_pool, dtype):
    _check(k_pool, "k_pool", dtype, 4)
    _check(v_pool, "v_pool", dtype, 4)
    if k_pool.shape != v_pool.shape or not (k_pool.is_contiguous() and v_pool.is_contiguous()):
        raise KernelError("key and value pools must be contiguous and of one shape")
    return k_pool.shape  # pages, kv_heads, page_size, head_dim


def _check_step_index(tok_item, tok_pos, tables, tokens, direct_items=False):
    """``direct_items``: the caller's kernel takes ``tok_item=None`` for "token t is item t"."""
    _check(tok_pos, "tok_pos", torch.int32, 1)
    _check(tables, "tables", torch.int32, 2)
    if tok_item is None:
        if not direct_items:
            raise KernelError("this kernel needs the item index of every token")
        if tables.shape[0] < tokens:
            raise KernelError("without item indices the block table needs a row per token")
    else:
        _check(tok_item, "tok_item", torch.int32, 1)
        if tok_item.numel() < tokens or not tok_item.is_contiguous():
            raise KernelError("one item index per token is needed, contiguous")
    if tok_pos.numel() < tokens:
        raise KernelError("one position per token is needed")
    if not (tok_pos.is_contiguous() and tables.is_contiguous()):
        raise KernelError("step index tensors must be contiguous")


def kv_write(k, v, k_pool, v_pool, tok_item, tok_pos, tables):
    """Store rows of k and v ([tokens, kv_heads*head_dim]) at their positions' pages."""
    _check(k, "k", ndim=2)
    _check(v, "v", k.dtype, 2)
    pages, kv_heads, page_size, head_dim = _check_pools(k_pool, v_pool, k.dtype)
    stride = _rows(k, "k")
    if _rows(v, "v") != stride or v.shape != k.shape:
        raise KernelError("kv_write: k and v must share shape and row stride")
    if k.shape[1] != kv_heads * head_dim:
        raise KernelError(f"kv_write: rows of {k.shape[1]} do not match {kv_heads} x {head_dim}")
    tokens = k.shape[0]
    _check_step_index(tok_item, tok_pos, tables, tokens)
    _call("ps_kv_write", k.data_ptr(), v.data_ptr(), stride, k_pool.data_ptr(), v_pool.data_ptr(),
          tok_item.data_ptr(), tok_pos.data_ptr(), tables.data_ptr(), tables.shape[1], tokens,
          kv_heads, head_dim, page_size, pages, dtype_code(k.dtype), _stream())


def _attention_args(q, k_pool, v_pool, out, tok_item, tok_pos, tables, heads, tok_list,
                    direct_items=False):
    _check(q, "q", ndim=2)
    _check(out, "out", q.dtype, 2)
    pages, kv_heads, page_size, head_dim = _check_pools(k_pool, v_pool, q.dtype)
    q_stride = _rows(q, "q")
    out_stride = _rows(out, "out")
    tokens = q.shape[0]
    if q.shape[1] != heads * head_dim or out.shape[1] != heads * head_dim or out.shape[0] != tokens:
        raise KernelError("attention: q/out rows must hold heads x head_dim values")
    _check_step_index(tok_item, tok_pos, tables, tokens, direct_items)
    count = tokens
    if tok_list is not None:
        _check(tok_list, "tok_list", torch.int32, 1)
        if not tok_list.is_contiguous():
            raise KernelError("attention: tok_list must be contiguous")
        count = tok_list.numel()
    return pages, kv_heads, page_size, head_dim, q_stride, out_stride, count


def attention_rowwise(q, k_pool, v_pool, out, tok_item, tok_pos, tables, heads, scale, window=0,
                      tok_list=None):
    """out[t, h] = softmax(q[t, h] . K * scale) V over the cached keys of t's request, for the
    tokens in ``tok_list`` (all when it is None)."""
    pages, kv_heads, page_size, head_dim, q_stride, out_stride, count = _attention_args(
        q, k_pool, v_pool, out, tok_item, tok_pos, tables, heads, tok_list)
    _call("ps_attention_rowwise", q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
          out.data_ptr(), out_stride, _ptr(tok_list), tok_item.data_ptr(), tok_pos.data_ptr(),
          tables.data_ptr(), tables.shape[1], count, heads, kv_heads, head_dim, page_size, pages,
          float(scale), int(window), dtype_code(q.dtype), _stream())
    return out


def decode_keys_per_block(head_dim: int, waves: int = 4) -> int:
    """Keys that one block of the split-KV kernel visits per iteration."""
    lanes = -(-head_dim // 8)
    lanes_per_key = 2 if lanes <= 2 else 4 if lanes <= 4 else 8 if lanes <= 8 else 16 if lanes <= 16 else 32
    return (64 // lanes_per_key) * (8 if waves == 16 else 4) * waves


def attention_decode(q, k_pool, v_pool, out, tok_item, tok_pos, tables, heads, scale, splits,
                     partial=None, window=0, tok_list=None, waves=4):
    """The same result as ``attention_rowwise`` by the split-KV kernel; ``partial`` is float
    scratch of ``count * heads * splits * (head_dim + 2)`` values when ``splits > 1``.
    ``tok_item=None`` says that token t is item t (row t of ``tables``), as in a step of single
    tokens: the kernel then fetches its block table one trip to memory earlier."""
    pages, kv_heads, page_size, head_dim, q_stride, out_stride, count = _attention_args(
        q, k_pool, v_pool, out, tok_item, tok_pos, tables, heads, tok_list, direct_items=True)
    floats = 0
    if splits > 1:
        _check(partial, "partial", torch.float32)
        if not partial.is_contiguous():
            raise KernelError("attention_decode: scratch must be contiguous")
        floats = partial.numel()
    _call("ps_attention_decode", q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
          out.data_ptr(), out_stride, _ptr(partial if splits > 1 else None), floats,
          _ptr(tok_list), _ptr(tok_item), tok_pos.data_ptr(), tables.data_ptr(),
          tables.shape[1], count, heads, kv_heads, head_dim, page_size, pages, float(scale),
          int(window), int(splits), int(waves), dtype_code(q.dtype), _stream())
    return out


def decode_supported(head_dim) -> bool:
    """Whether the split-KV kernel takes this head size (a lane fetches eight consecutive head
    dimensions of a key in one piece); the row-wise kernel takes every size up to 256."""
    return head_dim % 8 == 0 and 0 < head_dim <= 256


def merge_linear_supported(dtype, tokens, head_dim, packed) -> bool:
    """Whether ``attention_decode_partial`` + ``attention_merge_linear`` take a step: bfloat16,
    up to 16 single-token items, a head size that is a multiple of 64, and the packed copy of the
    output projection's matrix."""
    return (dtype == torch.bfloat16 and packed is not None and 1 <= tokens <= 16
            and head_dim % 64 == 0 and head_dim <= 256)


def attention_decode_partial(q, k_pool, v_pool, partial, tok_item, tok_pos, tables, heads, scale, splits,
                             window=0, tok_list=None, waves=4):
    """The per-range records of decode attention only (``partial``: float scratch of
    ``count * heads * splits * (head_dim + 2)`` values); ``attention_merge_linear`` merges them.
    ``tok_item=None``: token t is item t, as for ``attention_decode``."""
    _check(q, "q", ndim=2)
    pages, kv_heads, page_size, head_dim = _check_pools(k_pool, v_pool, q.dtype)
    q_stride = _rows(q, "q")
    tokens = q.shape[0]
    if q.shape[1] != heads * head_dim:
        raise KernelError("attention: q rows must hold heads x head_dim values")
    _check_step_index(tok_item, tok_pos, tables, tokens, direct_items=True)
    count = tokens
    if tok_list is not None:
        _check(tok_list, "tok_list", torch.int32, 1)
        if not tok_list.is_contiguous():
            raise KernelError("attention: tok_list must be contiguous")
        count = tok_list.numel()
    _check(partial, "partial", torch.float32)
    if not partial.is_contiguous():
        raise KernelError("attention_decode_partial: scratch must be contiguous")
    _call("ps_attention_decode_partial", q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
          partial.data_ptr(), partial.numel(), _ptr(tok_list), _ptr(tok_item), tok_pos.data_ptr(),
          tables.data_ptr(), tables.shape[1], count, heads, kv_heads, head_dim, page_size, pages,
          float(scale), int(window), int(splits), int(waves), dtype_code(q.dtype), _stream())
    return count


def attention_merge_linear(partial, count, heads, head_dim, splits, w, packed, bias, residual, tok_list=None,
                           heads_per_block=0):
    """residual[t] += (merged attention output of row r) w^T + bias for the ``count`` rows whose
    records ``attention_decode_partial`` left in ``partial``; ``packed`` is ``pack_decode_weight(w)``.
    ``heads_per_block``: 0 (the library chooses), 1, 2 or 4 heads whose results a block sums
    before it adds them to the rows."""
    _check(partial, "partial", torch.float32)
    _check(residual, "residual", torch.float32, 2)
    _check(w, "w", torch.bfloat16, 2)
    n, k = w.shape
    if k != heads * head_dim or residual.shape[1] != n:
        raise KernelError(f"attention_merge_linear: w {tuple(w.shape)} does not fit {heads} heads of "
                          f"{head_dim} and rows of {residual.shape[1]}")
    if packed is None or packed.dtype != torch.bfloat16 or not packed.is_contiguous() \
            or packed.numel() != -(-n // 16) * 16 * k:
        raise KernelError("attention_merge_linear: the packed copy does not belong to w")
    if bias is not None:
        _check(bias, "bias", torch.float32, 1)
        if bias.numel() != n:
            raise KernelError("attention_merge_linear: bias does not match n")
    if tok_list is None and residual.shape[0] < count:
        raise KernelError("attention_merge_linear: fewer residual rows than records")
    _call("ps_attention_merge_linear", partial.data_ptr(), partial.numel(), _ptr(tok_list), int(count),
          int(heads), int(head_dim), int(splits), packed.data_ptr(), _ptr(bias), residual.data_ptr(),
          _rows(residual, "residual"), n, int(heads_per_block), _stream())
    return residual


PREFILL_TILE = 64          # queries per block of the tiled prefill kernel
PREFILL_SMALL_TILE = 32    # and of its variant for steps with few tiles (head sizes up to 128)
PREFILL_LARGE_TILE = 128   # and of its variant for long prompts (head sizes up to 64)
PREFILL_LARGE_TILE_HEAD_DIM = 64
PREFILL_TABLE_MAX = 2048   # block-table entries of an item that it keeps in LDS
_PREFILL_CHECKED = False


def prefill_limits():
    """(queries per tile, widest block table) as the loaded library was built."""
    lib = load_library()
    lib.ps_attention_prefill_query_tile.restype = c_int
    lib.ps_attention_prefill_table_max.restype = c_int
    return lib.ps_attention_prefill_query_tile(), lib.ps_attention_prefill_table_max()


def prefill_small_tile():
    """Queries per tile of the variant for few tiles, as the loaded library was built."""
    lib = load_library()
    lib.ps_attention_prefill_small_tile.restype = c_int
    return lib.ps_attention_prefill_small_tile()


def prefill_large_tile():
    """(queries per tile, largest head size) of the variant for long prompts, as the loaded
    library was built."""
    lib = load_library()
    lib.ps_attention_prefill_large_tile.restype = c_int
    lib.ps_attention_prefill_large_tile_head_dim.restype = c_int
    return lib.ps_attention_prefill_large_tile(), lib.ps_attention_prefill_large_tile_head_dim()


def _check_prefill_constants():
    global _PREFILL_CHECKED
    if not _PREFILL_CHECKED:
        built = prefill_limits() + (prefill_small_tile(),) + prefill_large_tile()
        if built != (PREFILL_TILE, PREFILL_TABLE_MAX, PREFILL_SMALL_TILE, PREFILL_LARGE_TILE,
                     PREFILL_LARGE_TILE_HEAD_DIM):
            raise KernelError(f"attention_prefill: this module lists queries in tiles of {PREFILL_TILE}, "
                              f"{PREFILL_SMALL_TILE} or {PREFILL_LARGE_TILE} (head sizes up to "
                              f"{PREFILL_LARGE_TILE_HEAD_DIM}) and tables of up to {PREFILL_TABLE_MAX}, "
                              f"the library was built for {built}; rebuild the library")
        _PREFILL_CHECKED = True


def prefill_supported(dtype, head_dim, table_width=0) -> bool:
    """Whether the tiled matrix-core kernel takes this storage type, head size and width of
    the block tables (it keeps a tile's table entries in LDS)."""
    return (dtype == torch.bfloat16 and head_dim % 16 == 0 and head_dim <= 256
            and table_width <= PREFILL_TABLE_MAX)


def prefill_small_tile_pays(heads, head_dim, tiles) -> bool:
    """Whether ``tiles`` tiles of 64 queries of ``heads`` heads leave so many compute units
    without a block (half of them or more) that tiles of 32 queries are the better cut: a
    prompt portion of some hundred tokens beside decoded ones."""
    return head_dim <= 128 and 2 * heads * tiles <= compute_units()


def prefill_large_tile_pays(heads, head_dim, large_tiles, max_kv_len=0) -> bool:
    """Whether ``large_tiles`` tiles of 128 queries of ``heads`` heads are the better cut: from
    three blocks per compute unit on (two are resident at a time; with fewer the block that
    sees the most keys decides, and it is twice as long) and where a request holds 2,048 keys
    or more (``max_kv_len``: no query sees more; 0 = unknown).  Measured against the tiles of
    64, four of whose blocks share a compute unit: 2 x 4,096 tokens of 12 heads, 768 blocks, 86
    against 97 us; 2 x 4,096 of 25 heads 178 against 202; 2 x 3,072 of 25 heads 107 against 117;
    4 x 2,048 of 12 heads 57 against 59; but 4 x 1,024 of 25 heads, 800 blocks, 35 against 33; 16 x
    512 of 12 heads 24 against 22; 2 x 3,072 of 12 heads, 576 blocks, 65 against 56."""
    return (head_dim <= PREFILL_LARGE_TILE_HEAD_DIM and heads * large_tiles >= 3 * compute_units()
            and (max_kv_len <= 0 or max_kv_len >= 2048))


def attention_prefill(q, k_pool, v_pool, out, tile_item, tile_q0, cu_tokens, kv_lens, tables,
                      heads, scale, window=0, max_kv_len=0, query_tile=PREFILL_TILE, memo=None,
                      shared=None):
    """Attention of items with several tokens, ``query_tile`` (64, 32 or 128) queries per block,
    on the matrix cores.  Blocks start in the order of the tile list, which is cut for that size:
    the tiles that see the most keys belong first.
    ``max_kv_len`` (no query sees more keys; 0 = unknown) only steers the launch shape.
    ``memo``, ``shared``: as in ``attention_mixed``."""
    key = step_key = None
    if memo is not None:
        step_key = ("prefill", q.data_ptr(), q.shape[0], out.data_ptr(),
                    tile_item.data_ptr(), tile_item.numel(), tile_q0.data_ptr(), cu_tokens.data_ptr(),
                    cu_tokens.numel(), kv_lens.data_ptr(), tables.data_ptr(), tables.shape[1], heads, scale,
                    window, max_kv_len, query_tile)
        key = step_key + (k_pool.data_ptr(), v_pool.data_ptr())
        kept = memo.get(key) or _sibling_call(memo, shared, key, step_key, k_pool, v_pool)
        if kept is not None:
            _call("ps_attention_prefill", *kept, _stream())
            return out
    _check_prefill_constants()
    _check(q, "q", torch.bfloat16, 2)
    _check(out, "out", torch.bfloat16, 2)
    pages, kv_heads, page_size, head_dim = _check_pools(k_pool, v_pool, q.dtype)
    q_stride = _rows(q, "q")
    out_stride = _rows(out, "out")
    if q.shape[1] != heads * head_dim or out.shape != q.shape:
        raise KernelError("attention_prefill: q/out rows must hold heads x head_dim values")
    for name, tensor in (("tile_item", tile_item), ("tile_q0", tile_q0), ("cu_tokens", cu_tokens),
                         ("kv_lens", kv_lens)):
        _check(tensor, name, torch.int32, 1)
        if not tensor.is_contiguous():
            raise KernelError(f"attention_prefill: {name} must be contiguous")
    _check(tables, "tables", torch.int32, 2)
    tiles = tile_item.numel()
    items = kv_lens.numel()
    if tile_q0.numel() != tiles or cu_tokens.numel() != items + 1 or tables.shape[0] != items \
            or not tables.is_contiguous():
        raise KernelError("attention_prefill: inconsistent tile or item arrays")
    _kept_call("ps_attention_prefill", memo, key,
               (q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
                out.data_ptr(), out_stride, tile_item.data_ptr(), tile_q0.data_ptr(), tiles,
                cu_tokens.data_ptr(), kv_lens.data_ptr(), tables.data_ptr(), tables.shape[1], heads,
                kv_heads, head_dim, page_size, pages, float(scale), int(window), int(max_kv_len),
                int(query_tile), dtype_code(q.dtype)),
               shared, step_key, (kv_heads, head_dim, page_size, pages, q.dtype))
    return out


def tiled_f32_supported(dtype, head_dim) -> bool:
    """Whether ``attention_tiled_f32`` takes the shape: float storage, head sizes that are
    multiples of 4 up to 128."""
    return dtype == torch.float32 and head_dim % 4 == 0 and 4 <= head_dim <= 128


_TILED_F32_CHECKED = False


def attention_tiled_f32(q, k_pool, v_pool, out, tile_item, tile_q0, cu_tokens, kv_lens, tables, heads,
                        scale, window=0):
    """Attention of items with several tokens in true 32-bit, ``PREFILL_TILE`` queries per
    block: keys and values pass through LDS once per tile of queries instead of once per query
    (``attention_rowwise``), scores and sums are plain float arithmetic.  The tile list is the
    one of ``attention_prefill`` at that size."""
    global _TILED_F32_CHECKED
    if not _TILED_F32_CHECKED:
        lib = load_library()
        lib.ps_attention_tiled_f32_tile.restype = c_int
        if lib.ps_attention_tiled_f32_tile() != PREFILL_TILE:
            raise KernelError(f"the library's 32-bit tiled attention takes tiles of "
                              f"{lib.ps_attention_tiled_f32_tile()} queries, this module lists tiles "
                              f"of {PREFILL_TILE}; rebuild the library")
        _TILED_F32_CHECKED = True
    _check(q, "q", torch.float32, 2)
    _check(out, "out", torch.float32, 2)
    pages, kv_heads, page_size, head_dim = _check_pools(k_pool, v_pool, q.dtype)
    q_stride = _rows(q, "q")
    out_stride = _rows(out, "out")
    if q.shape[1] != heads * head_dim or out.shape != q.shape:
        raise KernelError("attention_tiled_f32: q/out rows must hold heads x head_dim values")
    for name, tensor in (("tile_item", tile_item), ("tile_q0", tile_q0), ("cu_tokens", cu_tokens),
                         ("kv_lens", kv_lens)):
        _check(tensor, name, torch.int32, 1)
        if not tensor.is_contiguous():
            raise KernelError(f"attention_tiled_f32: {name} must be contiguous")
    _check(tables, "tables", torch.int32, 2)
    tiles = tile_item.numel()
    items = kv_lens.numel()
    if tile_q0.numel() != tiles or cu_tokens.numel() != items + 1 or tables.shape[0] != items \
            or not tables.is_contiguous():
        raise KernelError("attention_tiled_f32: inconsistent tile or item arrays")
    _call("ps_attention_tiled_f32", q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
          out.data_ptr(), out_stride, tile_item.data_ptr(), tile_q0.data_ptr(), tiles,
          cu_tokens.data_ptr(), kv_lens.data_ptr(), tables.data_ptr(), tables.shape[1], heads,
          kv_heads, head_dim, page_size, pages, float(scale), int(window), _stream())
    return out


def mixed_supported(dtype, head_dim, table_width=0) -> bool:
    """Whether one launch can take a step's one-token items and its items of several tokens
    together (``attention_mixed``): bfloat16, head sizes of 16 to 64 in steps of 16."""
    return (dtype == torch.bfloat16 and head_dim % 16 == 0 and 16 <= head_dim <= 64
            and table_width <= PREFILL_TABLE_MAX)


def _kept_call(name, memo, key, args, shared=None, step_key=None, pool_shape=None):
    """Calls ``name`` with ``args`` and keeps them under ``key``: the next call of this site
    with the same addresses and counts skips the checks that led to them (a step that is not
    replayed from a graph is issued by the host at the GPU's own pace, and the checks of an
    attention call take as long as three launches).  ``shared`` (a dict that lives for one
    step) gets them too, under the part of the key that the same call of the other layers
    shares, with the pools' shape and type."""
    _call(name, *args, _stream())
    if memo is not None:
        if len(memo) >= 256:
            memo.clear()
        memo[key] = args
        memo["site", args[2], args[3]] = pool_shape
        if shared is not None:
            shared[step_key] = (args, pool_shape)


def _sibling_call(memo, shared, key, step_key, k_pool, v_pool):
    """The arguments of an attention call whose checks the same call of another layer has
    passed in this step (same queries' buffer, same index arrays), for this site's pools:
    theirs with the two pool addresses replaced, if these are the pools that this site has been
    checked with and of the other site's shape and type.  None otherwise."""
    if shared is None:
        return None
    pools = (k_pool.data_ptr(), v_pool.data_ptr())
    sibling, own = shared.get(step_key), memo.get(("site",) + pools)
    if sibling is None or own is None:
        return None
    args, pool_shape = sibling
    if own != pool_shape:
        return None
    args = args[:2] + pools + args[4:]
    if len(memo) >= 256:
        memo.clear()
        memo[("site",) + pools] = own
    memo[key] = args
    return args


def attention_mixed(q, k_pool, v_pool, out, tok_list, tok_item, positions, tile_item, tile_q0,
                    cu_tokens, kv_lens, tables, heads, scale, window=0, memo=None, shared=None):
    """The attention of a step that mixes decoded tokens with prompt portions, in one launch:
    the tokens listed in ``tok_list`` (the step's one-token items) as ``attention_decode`` with
    one range of keys computes them, the tiles of 64 queries listed in ``tile_item`` /
    ``tile_q0`` as ``attention_prefill`` does; blocks of both kinds share the compute units.
    ``memo`` (a dict of the call site, for the buffers of one workspace): what a checked call
    handed to the library, by the operands' addresses and counts.  ``shared`` (a dict that
    lives for one step, handed to the calls of all layers): what the same call of the layer
    before was checked with in this step; only the pools differ, and a site whose pools have
    been checked before takes the rest from there."""
    key = step_key = None
    if memo is not None:
        step_key = ("mixed", q.data_ptr(), q.shape[0], out.data_ptr(),
                    tok_list.data_ptr(), tok_list.numel(), tok_item.data_ptr(), positions.data_ptr(),
                    tile_item.data_ptr(), tile_item.numel(), tile_q0.data_ptr(), cu_tokens.data_ptr(),
                    cu_tokens.numel(), kv_lens.data_ptr(), tables.data_ptr(), tables.shape[1], heads, scale, window)
        key = step_key + (k_pool.data_ptr(), v_pool.data_ptr())
        kept = memo.get(key) or _sibling_call(memo, shared, key, step_key, k_pool, v_pool)
        if kept is not None:
            _call("ps_attention_mixed", *kept, _stream())
            return out
    _check_prefill_constants()
    _check(q, "q", torch.bfloat16, 2)
    _check(out, "out", torch.bfloat16, 2)
    pages, kv_heads, page_size, head_dim = _check_pools(k_pool, v_pool, q.dtype)
    q_stride = _rows(q, "q")
    out_stride = _rows(out, "out")
    if q.shape[1] != heads * head_dim or out.shape != q.shape:
        raise KernelError("attention_mixed: q/out rows must hold heads x head_dim values")
    for name, tensor in (("tok_list", tok_list), ("tok_item", tok_item), ("positions", positions),
                         ("tile_item", tile_item), ("tile_q0", tile_q0), ("cu_tokens", cu_tokens),
                         ("kv_lens", kv_lens)):
        _check(tensor, name, torch.int32, 1)
        if not tensor.is_contiguous():
            raise KernelError(f"attention_mixed: {name} must be contiguous")
    _check(tables, "tables", torch.int32, 2)
    tiles = tile_item.numel()
    items = kv_lens.numel()
    tokens = q.shape[0]
    if tile_q0.numel() != tiles or cu_tokens.numel() != items + 1 or tables.shape[0] != items \
            or not tables.is_contiguous() or tok_item.numel() != tokens or positions.numel() != tokens \
            or tok_list.numel() > tokens:
        raise KernelError("attention_mixed: inconsistent token, tile or item arrays")
    _kept_call("ps_attention_mixed", memo, key,
               (q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
                out.data_ptr(), out_stride, tok_list.data_ptr(), tok_list.numel(), tok_item.data_ptr(),
                positions.data_ptr(), tile_item.data_ptr(), tile_q0.data_ptr(), tiles,
                cu_tokens.data_ptr(), kv_lens.data_ptr(), tables.data_ptr(), tables.shape[1], heads,
                kv_heads, head_dim, page_size, pages, float(scale), int(window), dtype_code(q.dtype)),
               shared, step_key, (kv_heads, head_dim, page_size, pages, q.dtype))
    return out


def sample(logits, inv_temperature, uniform, out):
    """out[r] = argmax(logits[r]) where inv_temperature[r] == 0, else the inverse-CDF draw of
    softmax(logits[r] * inv_temperature[r]) at uniform[r]."""
    _check(logits, "logits", torch.float32, 2)
    _check(out, "out", torch.int32, 1)
    ld = _rows(logits, "logits")
    rows, vocab = logits.shape
    if out.numel() < rows:
        raise KernelError("sample: out has too few entries")
    if inv_temperature is not None:
        _check(inv_temperature, "inv_temperature", torch.float32, 1)
        _check(uniform, "uniform", torch.float32, 1)
        if inv_temperature.numel() < rows or uniform.numel() < rows:
            raise KernelError("sample: one temperature and one uniform number per row are needed")
    _call("ps_sample", logits.data_ptr(), ld, _ptr(inv_temperature), _ptr(uniform),
          out.data_ptr(), rows, vocab, _stream())
    return out


class StepGraph:
    """An executable HIP graph of the launches issued between ``begin`` and ``end`` on the
    current (non-default) stream."""

    def __init__(self):
        self.handle = None
        self.nodes = 0
        self.replays = 0

    @staticmethod
    def begin():
        lib = load_library()
        lib.ps_graph_begin.argtypes = [c_void_p]
        lib.ps_graph_begin.restype = c_int
        if lib.ps_graph_begin(_stream()) != 0:
            raise KernelError(lib.ps_last_error().decode())

    def end(self):
        lib = load_library()
        lib.ps_graph_end.argtypes = [c_void_p, ctypes.POINTER(c_void_p), ctypes.POINTER(c_int)]
        lib.ps_graph_end.restype = c_int
        handle = c_void_p()
        nodes = c_int(0)
        if lib.ps_graph_end(_stream(), ctypes.byref(handle), ctypes.byref(nodes)) != 0:
            raise KernelError(lib.ps_last_error().decode())
        self.handle = handle
        self.nodes = nodes.value

    @staticmethod
    def abort():
        lib = load_library()
        lib.ps_graph_abort.argtypes = [c_void_p]
        lib.ps_graph_abort(_stream())

    def launch(self):
        fn = _BOUND.get("ps_graph_launch")
        if fn is None:
            fn = load_library().ps_graph_launch
            fn.argtypes = [c_void_p, c_void_p]
            fn.restype = c_int
            _BOUND["ps_graph_launch"] = fn
        if fn(self.handle, _stream()) != 0:
            raise KernelError(load_library().ps_last_error().decode())
        self.replays += 1

    def destroy(self):
        if self.handle is not None:
            lib = load_library()
            lib.ps_graph_destroy.argtypes = [c_void_p]
            lib.ps_graph_destroy(self.handle)
            self.handle = None


_COMPUTE_UNITS = None


def compute_units() -> int:
    """Compute units of the current device (asked once)."""
    global _COMPUTE_UNITS
    if _COMPUTE_UNITS is None:
        _COMPUTE_UNITS = max(1, device_info()["compute_units"])
    return _COMPUTE_UNITS


def device_info():
    units = ctypes.c_int(0)
    lds = ctypes.c_int(0)
    arch = ctypes.create_string_buffer(64)
    fn = load_library().ps_device_info
    fn.restype = c_int
    status = fn(ctypes.byref(units), ctypes.byref(lds), arch, 64)
    if status != 0:
        raise KernelError(load_library().ps_last_error().decode())
    return {"compute_units": units.value, "lds_bytes": lds.value, "arch": arch.value.decode()}
