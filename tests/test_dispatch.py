"""Host-side choices that shape kernel launches (no GPU needed): which bfloat16 product takes
a shape, how decode attention shares a context out, how runs of rows are paired into blocks."""
import pytest

from alofa_amd import ops
from alofa_amd.errors import AlofaError


def test_product_kernel_by_shape():
    assert ops.few_rows_kernel(65, 8, 8) == "tiled"                               # beyond the streaming kernel's rows
    assert ops.few_rows_kernel(1, 151936, 896) == "tiled"                         # a vocabulary-long matrix, from the first row on
    assert ops.few_rows_kernel(1, 2 * 18944, 3584, swiglu=True) == "stream"       # (not so for the fused gate/up form)
    for rows in (1, 8, 16, 64):
        assert ops.few_rows_kernel(rows, 1152, 896) == "stream"                   # 0.5B-sized projections stream at every batch
    assert ops.few_rows_kernel(8, 3584, 18944) == "tiled" and ops.few_rows_kernel(4, 3584, 18944) == "stream"
    assert ops.few_rows_kernel(16, 4608, 3584) == "stream" and ops.few_rows_kernel(17, 4608, 3584) == "tiled"
    with pytest.raises(AlofaError):
        ops._product_entry("stream", 65, 64, 64)
    with pytest.raises(AlofaError):
        ops._product_entry("fast", 4, 64, 64)


def test_decode_splits_follow_the_context():
    short = ops.decode_splits(8, 14, 2, 64, 1024)
    assert short == 1                                                             # the waves of one block cover a short context
    assert ops.decode_splits(8, 14, 2, 64, 1 << 13) > ops.decode_splits(8, 14, 2, 64, 1 << 12) > 1   # about two steps of 32 keys a wave
    assert ops.decode_splits(8, 14, 2, 64, 1 << 16) == 256 // 16                   # until the blocks fill the chip
    assert ops.decode_splits(64, 14, 2, 64, 1 << 13) <= ops.decode_splits(8, 14, 2, 64, 1 << 13)    # many blocks already: fewer parts
    assert ops.decode_waves(64) == 8 and ops.decode_waves(128) == 4 and ops.decode_waves(256) == 4


def test_runs_are_paired_long_with_short():
    runs = [(0, 64 * i, 64, 64 * i) for i in range(8)]                            # one prompt of 512 tokens: 1..8 key tiles
    blocks = ops.pair_tiles(runs)
    assert len(blocks) == 4
    assert sorted(tuple(r) for b in blocks for r in b) == sorted(runs)
    assert all((b[0][3] + b[1][3]) == 64 * 7 for b in blocks)                     # longest with shortest, and so on
    odd = ops.pair_tiles(runs[:3])
    assert len(odd) == 2 and odd[1][1] == [0, 0, 0, 0]
    windowed = ops.pair_tiles(runs, window=100)                                   # with a window every run walks two or three tiles
    assert sorted(tuple(r) for b in windowed for r in b) == sorted(runs)
