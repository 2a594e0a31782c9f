"""The host-side rules that choose how the attention kernels cut a context (no GPU needed)."""
from qil_amd import ops


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
