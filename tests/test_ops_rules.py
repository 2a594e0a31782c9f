"""The host-side rules that choose kernels and how they cut their work (no GPU needed)."""
import ctypes

import pytest

from qil_amd import ops


@pytest.fixture(scope='module')
def lib():
    """The kernel library's planners are host code: they run without a GPU once the library is built."""
    try:
        return ops.library.load()
    except ops.library.KernelLibraryError as error:
        pytest.skip(f'kernel library not available here: {error}')


def test_row_kernel_parts_scale_with_the_work():
    """One row of 2,048 keys is cut into parts of 64 keys, eight rows into parts of 128, sixty-four into parts of
    512; never below 64 or above 512, and a power of two."""
    kv_heads = 8
    assert ops._rows_part(1, kv_heads, 2048) == 64
    assert ops._rows_part(8, kv_heads, 2048) == 128
    assert ops._rows_part(8, kv_heads, 2100) == 128
    assert ops._rows_part(8, kv_heads, 8192) == 512
    assert ops._rows_part(64, kv_heads, 2048) == 512
    assert ops._rows_part(1, 1, 5) == 64
    assert ops._rows_part(128, 8, 100000) == 512
    last = 0
    for context in range(1, 40000, 977):
        part = ops._rows_part(4, 2, context)
        assert part in (64, 128, 256, 512) and part >= last
        last = part


def test_decode_parts_cover_the_context():
    for rows, kv_heads, context in ((1, 8, 2048), (8, 8, 2048), (64, 8, 2048), (3, 1, 70000), (16, 4, 17), (1, 2, 1)):
        part, parts = ops._decode_parts(rows, kv_heads, context)
        assert part % 64 == 0 and ops.DECODE_MIN_PART <= part <= ops.DECODE_MAX_PART
        assert parts >= 1 and part * parts >= context and part * (parts - 1) < context


def test_decode_parts_fill_their_rounds_of_blocks():
    """More blocks than CUs run in rounds: where one part a row would leave the last round mostly empty the context
    is cut so that the rounds fill; where the rounds are full anyway, or the context is short, it stays whole."""
    kv_heads = 8
    assert ops._decode_parts(32, kv_heads, 2048) == (2048, 1)         # 256 blocks: one round
    assert ops._decode_parts(33, kv_heads, 2048) == (512, 4)          # 264 blocks -> 1,056: 5 rounds, 82 % full
    assert ops._decode_parts(40, kv_heads, 2048) == (1024, 2)
    assert ops._decode_parts(48, kv_heads, 2048) == (2048, 1)         # 384 blocks: the second round is half full
    assert ops._decode_parts(64, kv_heads, 2048) == (2048, 1)
    assert ops._decode_parts(65, kv_heads, 2048) == (1024, 2)
    assert ops._decode_parts(33, kv_heads, 8192) == (1216, 7)         # long parts: filled to 90 %
    assert ops._decode_parts(33, kv_heads, 700) == (704, 1)           # too short to cut
    for rows in range(1, 300, 7):
        for context in (1, 300, 2048, 5000, 40000, 131072):
            part, parts = ops._decode_parts(rows, kv_heads, context)
            assert part % 64 == 0 and ops.DECODE_MIN_PART <= part <= ops.DECODE_MAX_PART
            assert parts >= 1 and part * parts >= context and part * (parts - 1) < context


def test_products_of_257_to_512_rows_go_to_blocks_of_rows_where_the_library_is_slow(lib):
    down, qkv, gate_up = (4096, 12288), (6144, 4096), (24576, 4096)
    assert lib.qil_gemm_bf16_mid_rows_takes(512, *down) and lib.qil_gemm_bf16_mid_rows_takes(257, *down)
    assert lib.qil_gemm_bf16_mid_rows_takes(300, *qkv) and not lib.qil_gemm_bf16_mid_rows_takes(400, *qkv)
    assert not lib.qil_gemm_bf16_mid_rows_takes(300, *gate_up)
    assert not lib.qil_gemm_bf16_mid_rows_takes(256, *down) and not lib.qil_gemm_bf16_mid_rows_takes(513, *down)
    assert not lib.qil_gemm_bf16_mid_rows_takes(300, 4100, 4096) and not lib.qil_gemm_bf16_mid_rows_takes(300, 4096, 4000)
    for rows in (257, 300, 512):                              # the plan of such a product: whole stages, 4 or more a split
        splits = lib.qil_gemm_bf16_mid_splits(rows, *down)
        assert 1 <= splits <= 16 and (12288 // 64) % splits == 0 and 12288 // 64 // splits >= 4
    assert lib.qil_gemm_bf16_mid_splits(1025, *down) == 0


def test_float32_products_split_k_to_fill_the_chip(lib):
    """Up to 16 rows and 17 to 64 rows are whole-line kernels with K in whole stages of 64 columns, three or more a
    split; the blocks of 128 columns times the splits stay within the CUs where they can."""
    for rows in (1, 16, 17, 64):
        for n, k in ((4096, 4096), (6144, 4096), (1024, 3072), (24576, 4096), (130, 192)):
            splits = lib.qil_gemm_f32_splits(rows, n, k)
            assert splits >= 1 and k % (64 * splits) == 0 and k // (64 * splits) >= 3, (rows, n, k, splits)
    assert lib.qil_gemm_f32_splits(20, 4096, 4096) == 8        # 32 blocks of columns x 8 = 256
    assert lib.qil_gemm_f32_splits(20, 24576, 4096) == 1       # 192 blocks of columns already
    assert lib.qil_gemm_f32_splits(20, 4096, 100) >= 1         # no whole stage: another kernel, still a valid answer


def test_general_tile_kernel_cuts_the_keys_of_few_row_tiles(lib):
    part = ctypes.c_int(0)
    float32, bfloat16 = 0, 1
    # one portion of 128 rows, 16 heads in 8 groups: 32 blocks of row tiles -> parts of 128 keys
    assert lib.qil_attn_tile_key_parts(1, 128, 16, 8, 128, 2048, float32, ctypes.byref(part)) == 16 and part.value == 128
    assert lib.qil_attn_tile_key_parts(1, 128, 16, 8, 128, 2700, float32, ctypes.byref(part)) == 22 and part.value == 128
    # a whole prompt of 2,048 rows fills the chip by itself; a short context is not worth cutting
    assert lib.qil_attn_tile_key_parts(1, 2048, 16, 8, 128, 2048, float32, ctypes.byref(part)) == 1
    assert lib.qil_attn_tile_key_parts(1, 128, 16, 8, 128, 400, float32, ctypes.byref(part)) == 1
    for context in (512, 1000, 5000, 40000):
        for dtype in (float32, bfloat16):
            parts = lib.qil_attn_tile_key_parts(2, 64, 8, 2, 96, context, dtype, ctypes.byref(part))
            if parts > 1:
                assert part.value % 64 == 0 and part.value >= 128 and parts <= 32
                assert part.value * parts >= context > part.value * (parts - 1)
