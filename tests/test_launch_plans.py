"""The kernel library's launch decisions that are plain host arithmetic: asked of the built library without a GPU
(`KernelSizes`), at the compute-unit count it assumes there (256)."""

import pytest

from beholdd.kernels import KernelSizes


@pytest.fixture(scope="module")
def sizes():
    import ctypes
    library = KernelSizes(verbose_build=False)
    i = ctypes.c_int
    library.lib.bh_attention_bf16_splits.argtypes, library.lib.bh_attention_bf16_splits.restype = [i] * 5, i
    library.lib.bh_gemm_bf16_norm_blocks.argtypes, library.lib.bh_gemm_bf16_norm_blocks.restype = [i] * 5, i
    return library


def workgroups(sizes, sequences, context, heads=32, kv_heads=8):
    splits = sizes.lib.bh_attention_bf16_splits(sequences, 1, heads, kv_heads, context - 1)
    return splits, sequences * kv_heads * splits


def test_key_splits_fill_whole_rounds_of_workgroups(sizes):
    """A decode step's attention runs in rounds of one workgroup per compute unit: the split count never leaves a
    second round of a few workgroups that are sized for one round (288 to 384 of them for 9 to 14 sequences before)."""
    assert workgroups(sizes, 8, 8192) == (4, 256)
    assert workgroups(sizes, 1, 8192) == (32, 256)
    assert workgroups(sizes, 16, 8192) == (2, 256)
    assert workgroups(sizes, 32, 8192) == (1, 256)
    assert workgroups(sizes, 12, 8192) == (5, 480)
    assert workgroups(sizes, 6, 8192) == (5, 240)
    for sequences in range(1, 33):
        splits, count = workgroups(sizes, sequences, 8192)
        rounds = -(-count // 256)
        assert count > 0.75 * rounds * 256, (sequences, splits, count)      # no round of a few workgroups behind full ones
        assert splits <= 128 // 4                                           # every wave of a workgroup has a page
    # more workgroups than compute units: three splits just above one per compute unit, two just above two, else none
    assert [workgroups(sizes, n, 8192)[0] for n in (33, 40, 44, 48, 56, 64, 68, 72, 80, 128)] == [3, 3, 3, 1, 1, 1, 2, 2, 1, 1]
    # short caches are not split (fewer than eight pages), and a split never has fewer than four pages
    assert workgroups(sizes, 8, 448)[0] == 1 and workgroups(sizes, 8, 640)[0] == 2 and workgroups(sizes, 1, 1024)[0] == 4


def test_the_norm_that_rides_counts_the_workgroups_of_wider_spans(sizes):
    """Products of up to 32 rows whose blocks of 16 weight rows number between one and two per compute unit run with
    workgroups of 20 or 24 rows; a norm behind such a product gets one partial sum per workgroup."""
    blocks = lambda m, n, k: sizes.lib.bh_gemm_bf16_norm_blocks(m, n, k, 1, 0)
    assert blocks(8, 4096, 4096) == 256            # one block of 16 rows per compute unit
    assert blocks(8, 5120, 5120) == 256            # 320 blocks: spans of 20 rows
    assert blocks(32, 6144, 4096) == 256           # 384 blocks: spans of 24 rows
    assert blocks(8, 7168, 5120) == 448            # 28 rows could lie in three blocks: left to the blocks of 16
    assert blocks(8, 8192, 4096) == 512 and blocks(8, 2560, 4096) == 160
