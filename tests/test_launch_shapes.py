"""The rule that picks the decode attention's launch shape, on the CPU: whatever the sizes, the
ranges fit the scratch that the part asks for, and the documented cases come out as documented."""

import pytest

from pagedserve_amd.ops import kernels
from pagedserve_amd.parts.attention import Attention


def _part(heads, head_dim=64, window=0):
    part = Attention.__new__(Attention)
    part.heads, part.head_dim, part.window = heads, head_dim, window
    part.width = heads * head_dim
    return part


@pytest.mark.parametrize("units", [256, 304, 64])
def test_ranges_fit_the_scratch_and_the_kernel(monkeypatch, units):
    monkeypatch.setattr(kernels, "compute_units", lambda: units)
    for heads in (1, 2, 3, 12, 16, 25, 40, 96):
        for head_dim in (8, 64, 128, 256):
            for window in (0, 300):
                part = _part(heads, head_dim, window)
                for count in list(range(1, 70)) + [100, 128, 256, 300]:
                    for context in (1, 17, 100, 256, 300, 1000, 1024, 2048, 4096, 8192, 16384, 1 << 20):
                        splits, waves = part._splits(count, context)
                        assert 1 <= splits <= 64 and waves in (4, 16)
                        # what Attention._range_records holds: six blocks per unit beside one per pair
                        assert count * heads * splits <= 6 * units + count * heads
                        merged = part._merged_splits(count, context)
                        assert 0 <= merged <= 64
                        assert count * heads * merged <= 6 * units + count * heads


def test_documented_cases(monkeypatch):
    monkeypatch.setattr(kernels, "compute_units", lambda: 256)
    part = _part(12)
    assert part._splits(64, 1024) == (1, 4)          # three pairs per unit at 1,024 keys
    assert part._splits(100, 8192) == (1, 4)         # more than three and a half pairs per unit
    assert part._splits(32, 8192) == (4, 4)          # one and a half pairs per unit, long contexts
    assert part._splits(32, 1024) == (1, 4)
    assert part._splits(24, 1024) == (4, 4)          # between one and one and a half
    assert part._splits(24, 300) == (1, 4)
    assert part._splits(20, 1024) == (1, 16)         # up to one pair per unit
    assert part._splits(17, 16384) == (8, 4)         # ... over thousands of keys
    assert part._splits(8, 16384) == (2, 16)
    assert part._splits(1, 16384) == (64, 4)         # few pairs: ranges until four blocks per unit
    assert part._merged_splits(8, 1024) == 8 and part._merged_splits(1, 16384) == 64
    assert part._merged_splits(17, 1024) == 0
    # few pairs merge inside the projection at every length; from half a pair per unit on only
    # where the keys feed three ranges
    assert part._merged_splits(8, 200) == 2 and part._merged_splits(1, 20) == 1
    assert part._merged_splits(16, 200) == 0 and part._merged_splits(16, 1024) == 4
    # wide models: not where the projection's blocks would read the records too often
    assert _part(16)._merged_splits(4, 1024) == 8 and _part(16)._merged_splits(8, 1024) == 0
    assert _part(16)._merged_splits(8, 400) == 4 and _part(16)._merged_splits(12, 400) == 0
    assert _part(25)._merged_splits(2, 1024) == 8 and _part(25)._merged_splits(4, 1024) == 0
    assert _part(25)._merged_splits(4, 400) == 4
    # a window bounds the keys that a query sees
    assert _part(12, window=256)._splits(32, 8192) == (1, 4)


def test_query_tiles_of_the_prefill_attention(monkeypatch):
    """Which of the tiled kernel's three tile sizes a step takes: 32 queries while tiles of 64
    leave half of the compute units without a block, 128 from three blocks per unit on (head
    sizes up to 64), 64 otherwise; never both of the special ones."""
    monkeypatch.setattr(kernels, "compute_units", lambda: 256)
    small, large = kernels.prefill_small_tile_pays, kernels.prefill_large_tile_pays
    # a portion of 512 tokens beside decoded ones: 8 tiles of 64, 4 of 128
    assert small(12, 64, 8) and small(16, 64, 8) and not small(25, 64, 8)
    assert not large(12, 64, 4) and not large(25, 64, 4)
    # the prefill step of 2 x 1,024 tokens stays with tiles of 64 at every GPT-2 shape
    for heads in (12, 16, 25):
        assert not small(heads, 64, 32) and not large(heads, 64, 16)
    # long prompts
    assert large(12, 64, 64) and large(25, 64, 32) and large(16, 64, 48) and not large(16, 64, 47)
    assert large(12, 64, 64, 4096) and large(12, 64, 64, 2048) and not large(25, 64, 48, 1024)
    assert not large(12, 128, 64) and not large(12, 80, 640) and not small(1, 144, 1)
    for heads in (1, 3, 12, 25, 64):
        for tiles in range(1, 400):
            assert not (small(heads, 64, tiles) and large(heads, 64, -(-tiles // 2)))


def test_one_attention_launch_for_mixed_steps(monkeypatch):
    """Decoded tokens and prompt portions of a step share one attention launch where the kernel
    takes the shape, except a handful of tokens over long contexts and prompts long enough for
    tiles of 128 queries."""
    import types

    import torch

    monkeypatch.setattr(kernels, "compute_units", lambda: 256)

    class Count:
        def __init__(self, count):
            self.count = count

        def numel(self):
            return self.count

    def ctx(max_kv_len, large_tiles=4):
        return types.SimpleNamespace(max_kv_len=max_kv_len,
                                     query_tiles={kernels.PREFILL_LARGE_TILE: (Count(large_tiles), None)})

    tables = types.SimpleNamespace(shape=(8, 64))
    part = _part(12)
    part.dtype, part.fuse_mixed = torch.bfloat16, True
    assert part._one_launch(32, ctx(1024), tables) and part._one_launch(8, ctx(1024), tables)
    assert part._one_launch(6, ctx(1024), tables) and not part._one_launch(5, ctx(1024), tables)
    assert part._one_launch(2, ctx(512), tables) and not part._one_launch(2, ctx(1024), tables)
    assert not part._one_launch(32, ctx(4096, large_tiles=64), tables)      # long prompts: tiles of 128
    windowed = _part(12, window=256)
    windowed.dtype, windowed.fuse_mixed = torch.bfloat16, True
    assert windowed._one_launch(2, ctx(1024), tables)                       # a window bounds the keys
    for other in (_part(12, head_dim=128), _part(12, head_dim=40)):
        other.dtype, other.fuse_mixed = torch.bfloat16, True
        assert not other._one_launch(32, ctx(1024), tables)
    part.dtype = torch.float32
    assert not part._one_launch(32, ctx(1024), tables)
    part.dtype, part.fuse_mixed = torch.bfloat16, False
    assert not part._one_launch(32, ctx(1024), tables)


def test_argument_blocks_shared_between_the_layers_of_a_step():
    """``kernels._sibling_block``: the block of the same call site of another layer, with this
    site's own operands; nothing where the sites differ in a size or in the operands they have."""
    import ctypes

    names = [name for name, _ in kernels._LinearArgs._fields_]
    assert set(kernels._SITE_FIELDS) | set(kernels._STEP_FIELDS) <= set(names)
    assert not set(kernels._SITE_FIELDS) & set(kernels._STEP_FIELDS)

    def block(**fields):
        args = kernels._LinearArgs()
        for name, value in fields.items():
            setattr(args, name, value)
        return bytes(args)

    def read(data):
        return kernels._LinearArgs.from_buffer_copy(data)

    sizes = dict(n=192, k=256, epilogue=2, dtype=1, c_dtype=1, eps=1e-5, head_dim=64, q_cols=768)
    own = block(w=0x1000, bias=0x2000, gamma=0x3000, k_pool=0x4000, v_pool=0x5000, w_packed=0x6000,
                a=0x10, c=0x20, m=8, lda=256, ldc=192, tok_item=0x30, **sizes)
    sibling = block(w=0x9000, bias=0xA000, gamma=0xB000, k_pool=0xC000, v_pool=0xD000, w_packed=0xE000,
                    a=0x50, c=0x60, m=40, lda=512, ldc=384, tok_item=0x70, tables=0x80, table_width=64,
                    norm_h=0x90, **sizes)
    made = read(kernels._sibling_block(sibling, own))
    assert (made.w, made.bias, made.gamma, made.k_pool, made.v_pool, made.w_packed) == \
        (0x1000, 0x2000, 0x3000, 0x4000, 0x5000, 0x6000)
    assert (made.a, made.c, made.m, made.lda, made.ldc, made.tok_item, made.tables, made.table_width,
            made.norm_h) == (0x50, 0x60, 40, 512, 384, 0x70, 0x80, 64, 0x90)
    assert (made.n, made.k, made.epilogue, made.head_dim, made.q_cols) == (192, 256, 2, 64, 768)
    assert made.beta is None
    for name, value in (("n", 128), ("k", 512), ("epilogue", 1), ("c_dtype", 2), ("eps", 1e-6),
                        ("scatter_only", 1), ("page_size", 16), ("rms", 1), ("c_packed_request", 1)):
        other = read(sibling)
        setattr(other, name, value)
        assert kernels._sibling_block(bytes(other), own) is None, name
    for name in ("bias", "gamma", "w_packed", "k_pool"):
        other = read(own)
        setattr(other, name, None)                 # this site has no such operand, the other has
        assert kernels._sibling_block(sibling, bytes(other)) is None, name
    assert ctypes.sizeof(kernels._LinearArgs) == len(own)
