"""Host-side choices that shape kernel launches (no GPU needed): which bfloat16 product takes
a shape, how decode attention shares a context out, how runs of rows are paired into blocks."""
import pytest

from alofa_amd import ops
from alofa_amd.errors import AlofaError


def test_product_kernel_by_shape():
    assert ops.few_rows_kernel(65, 8, 8) == "tiled"                               # beyond the streaming kernel's rows
    assert ops.few_rows_kernel(1, 151936, 896) == "tiled"                         # a vocabulary-long matrix, from the first row on
    assert ops.few_rows_kernel(1, 2 * 18944, 3584, swiglu=True) == "rows"         # (not so for the fused gate/up form)
    for rows in (17, 64):
        assert ops.few_rows_kernel(rows, 1152, 896) == "stream"                   # 0.5B-sized projections stream from 17 rows on
    for rows in (9, 16):                                                          # nine to sixteen rows: plain products of small weights only
        assert ops.few_rows_kernel(rows, 896, 4864) == "rows" and ops.few_rows_kernel(rows, 1152, 896, normed=True) == "stream"
        assert ops.few_rows_kernel(rows, 2 * 4864, 896, swiglu=True) == "stream" and ops.few_rows_kernel(rows, 3584, 3584) == "stream"
    # at most eight rows: the vector-unit kernel, while the rows it reads once per four columns and its arithmetic stay light
    for rows in (1, 2, 4, 8):
        assert ops.few_rows_kernel(rows, 1152, 896) == "rows" and ops.few_rows_kernel(rows, 896, 4864) == "rows"
        assert ops.few_rows_kernel(rows, 1152, 896, normed=True) == "rows"
    assert ops.few_rows_kernel(4, 2 * 27648, 5120, swiglu=True, normed=True) == "tiled" and ops.few_rows_kernel(2, 2 * 27648, 5120, swiglu=True) == "rows"
    # gate and up of a small model with the norm: the streaming kernel from three rows on (its blocks are dealt out evenly), the vector units below
    assert ops.few_rows_kernel(2, 2 * 4864, 896, swiglu=True, normed=True) == "rows" and ops.few_rows_kernel(3, 2 * 4864, 896, swiglu=True, normed=True) == "stream"
    assert ops.few_rows_kernel(4, 2 * 4864, 896, swiglu=True, normed=True) == "stream" and ops.few_rows_kernel(5, 2 * 4864, 896, swiglu=True, normed=True) == "stream"
    assert ops.few_rows_kernel(4, 2 * 4864, 896, swiglu=True) == "rows" and ops.few_rows_kernel(4, 2 * 18944, 3584, swiglu=True, normed=True) == "rows"
    assert ops.few_rows_kernel(4, 4608, 3584, normed=True) == "rows" and ops.few_rows_kernel(4, 7168, 5120, normed=True) == "stream"
    assert ops.few_rows_kernel(8, 4608, 3584, normed=True) == "stream" and ops.few_rows_kernel(8, 5120, 5120) == "rows"
    assert ops.few_rows_kernel(2, 3584, 18944) == "rows" and ops.few_rows_kernel(4, 5120, 13824) == "rows"    # long rows: its looping form
    assert ops.few_rows_kernel(3, 3584, 18944) == "tiled" and ops.few_rows_kernel(4, 3584, 18944) == "tiled"  # (not where its blocks come in three and a half rounds)
    assert ops.few_rows_kernel(4, 2048, 11008) == "rows" and ops.few_rows_kernel(4, 5120, 27648) == "rows"
    assert ops.few_rows_kernel(2, 2 * 4864, 8192, swiglu=True) == "stream" and ops.few_rows_kernel(2, 1024, 8192, normed=True) == "stream"    # (plain products only)
    assert ops.few_rows_kernel(2, 2 * 18944, 8192, swiglu=True) == "tiled"        # gate and up of 256 M weights or more: the tiled kernel's wide tiles
    assert ops.few_rows_kernel(8, 3584, 18944) == "tiled"
    assert ops.few_rows_kernel(16, 3584, 3584) == "stream" and ops.few_rows_kernel(16, 4608, 3584) == "tiled" and ops.few_rows_kernel(17, 3584, 3584) == "tiled"
    # five to eight rows of more values than the vector-unit kernel takes in one go: not its looping form
    assert ops.few_rows_kernel(8, 1536, 8960) == "stream" and ops.few_rows_kernel(4, 1536, 8960) == "rows" and ops.few_rows_kernel(8, 896, 4864) == "rows"
    # nine to sixteen rows against a long, narrow matrix: the tiled kernel, which shares K out over more blocks
    assert ops.few_rows_kernel(12, 2048, 11008) == "tiled" and ops.few_rows_kernel(12, 1536, 8960) == "tiled" and ops.few_rows_kernel(12, 2048, 2048) == "rows"
    # beyond 32 rows the tiled kernel takes smaller matrices than below
    assert ops.few_rows_kernel(32, 2560, 2048) == "stream" and ops.few_rows_kernel(48, 2560, 2048) == "tiled" and ops.few_rows_kernel(64, 2048, 2048) == "stream"
    assert ops._product_entry(None, 8, 896, 4864) == "alofa_gemm_rows" and ops._product_entry("stream", 8, 896, 4864) == "alofa_gemm_skinny"
    with pytest.raises(AlofaError):
        ops._product_entry("rows", 17, 64, 64)
    with pytest.raises(AlofaError):
        ops._product_entry("rows", 9, 64, 64, normed=True)
    with pytest.raises(AlofaError):
        ops._product_entry("stream", 65, 64, 64)
    with pytest.raises(AlofaError):
        ops._product_entry("fast", 4, 64, 64)


def test_a_norm_in_front_of_a_large_product_of_few_rows_runs_apart():
    # the vector-unit kernel reads float32 rows once per four columns: against a large matrix the norm's own kernel costs less
    assert ops.norm_goes_apart(8, 4608, 3584) and ops.norm_goes_apart(6, 4608, 3584) and not ops.norm_goes_apart(2, 4608, 3584)
    assert ops.norm_goes_apart(2, 7168, 5120) and ops.norm_goes_apart(4, 7168, 5120) and not ops.norm_goes_apart(1, 7168, 5120)
    assert not ops.norm_goes_apart(8, 7168, 5120)                  # (the plain product of so many values is not the vector units' either)
    assert not ops.norm_goes_apart(8, 1152, 896) and not ops.norm_goes_apart(8, 2560, 2048) and not ops.norm_goes_apart(12, 4608, 3584)


def test_a_norm_behind_a_product_moves_it_to_the_kernel_that_adds_shares():
    # 17 to 64 rows, a long K, few columns: the tiled kernel's second launch takes the norm with it (the 0.5B down projection)
    assert ops.norm_rides_on_shares(17, 896, 4864) and ops.norm_rides_on_shares(64, 896, 4864)
    assert not ops.norm_rides_on_shares(16, 896, 4864) and not ops.norm_rides_on_shares(65, 896, 4864)      # the norm rides elsewhere / all is tiled anyway
    assert not ops.norm_rides_on_shares(32, 896, 896)              # a short K is not shared out
    assert not ops.norm_rides_on_shares(32, 3584, 18944)           # tiled already (and shared out): nothing to move
    assert not ops.norm_rides_on_shares(32, 8192, 4096)            # too many columns for the launch that adds shares


def test_decode_splits_follow_the_context(monkeypatch):
    monkeypatch.setattr(ops, "_compute_units", 256)                                # the rule counts the chip's compute units: an MI355X's here
    assert ops.decode_splits(8, 14, 2, 64, 512) == 1                              # the waves of one block cover two steps each
    assert ops.decode_splits(8, 14, 2, 64, 1024) == 4 and ops.decode_splits(32, 14, 2, 64, 1024) == 4 and ops.decode_splits(64, 14, 2, 64, 1024) == 1    # four parts up to four steps, with room for four
    assert ops.decode_splits(8, 14, 2, 64, 2048) == 8                             # a part per step of all the waves
    assert ops.decode_splits(8, 14, 2, 64, 1 << 12) == 8 and ops.decode_splits(8, 14, 2, 64, 1 << 13) == 16    # at most eight, then a part per two steps
    assert ops.decode_splits(8, 14, 2, 64, 1 << 16) == 256 // 16                   # until the blocks fill the chip
    assert ops.decode_splits(64, 14, 2, 64, 2048) == 1 and ops.decode_splits(64, 14, 2, 64, 4096) == 2 and ops.decode_splits(32, 14, 2, 64, 2048) == 4    # many blocks already: fewer parts
    assert ops.decode_splits(8, 28, 4, 128, 256) == 1 and ops.decode_splits(8, 28, 4, 128, 512) == 4 and ops.decode_splits(8, 28, 4, 128, 4096) == 8
    assert ops.decode_splits(32, 28, 4, 128, 512) == 1 and ops.decode_splits(32, 28, 4, 128, 1024) == 1 and ops.decode_splits(32, 28, 4, 128, 2048) == 2 and ops.decode_splits(64, 28, 4, 128, 4096) == 1
    monkeypatch.setattr(ops, "_compute_units", 64)                                 # a smaller chip is full sooner
    assert ops.decode_splits(8, 14, 2, 64, 1024) == 4 and ops.decode_splits(8, 14, 2, 64, 1 << 16) == 4 and ops.decode_splits(32, 14, 2, 64, 1 << 16) == 1
    assert ops.HAND_OVER_MAX_PARTS == 8
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
