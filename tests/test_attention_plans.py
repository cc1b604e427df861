"""How the attention part divides its work: numbers of splits and the workspace they need."""

from kvcore_amd.parts.attention import (PREFILL_MAX_SPLITS, decode_splits, prefill_split_rows,
                                        prefill_splits)


def test_portions_of_prompts_split_their_keys_only_when_rows_are_few_and_keys_many():
    nkv, g = 8, 4
    # a whole prompt, and enough rows for every compute unit: one block per tile
    assert prefill_splits(2048, nkv, g, 2048, 2048, 0) == 1
    assert prefill_splits(8192, nkv, g, 8192, 8192, 0) == 1
    assert prefill_splits(4096, nkv, g, 4096, 40000, 0) == 1
    # a portion after a long context
    assert prefill_splits(2048, nkv, g, 2048, 8192, 0) == 2
    assert prefill_splits(512, nkv, g, 512, 8704, 0) == 8
    assert prefill_splits(16, nkv, g, 16, 8208, 0) == PREFILL_MAX_SPLITS
    # short contexts are never split, however few the rows
    assert prefill_splits(16, nkv, g, 16, 200, 0) == 1
    assert prefill_splits(64, nkv, g, 2, 97, 0) == 1
    # a window bounds the keys a row sees
    assert prefill_splits(64, nkv, g, 64, 100000, 128) == 1
    assert prefill_splits(64, nkv, g, 64, 100000, 4096) > 1


def test_workspace_bound_holds_for_every_step_size():
    for nkv, g in ((8, 4), (8, 8), (1, 4), (2, 3), (1, 64), (4, 1), (16, 2), (1, 1), (3, 5)):
        bound = prefill_split_rows(nkv, g)
        for T in range(1, 20000, 7):
            n = prefill_splits(T, nkv, g, T, 10 ** 6, 0)
            assert 1 <= n <= PREFILL_MAX_SPLITS
            assert n == 1 or T * n <= bound, (nkv, g, T, n)


def test_single_tokens_split_until_the_chip_is_full():
    assert decode_splits(8, 8, 640, 8, 0) == 4
    assert decode_splits(1, 8, 640, 8, 0) >= 4
    assert decode_splits(64, 8, 640, 4, 0) == 1
    assert decode_splits(1, 8, 100000, 8, 0) == 32
    assert decode_splits(1, 8, 100000, 8, 64) <= 2  # a window of 64 keys is a handful of blocks


def test_row_counts_choose_how_norms_and_products_meet():
    import torch

    from kvcore_amd.ops import library as ops

    bf16, f32 = torch.bfloat16, torch.float32
    # the products do the norms' work up to 16 rows; from 17 to 192 a kernel of its own finishes them
    assert ops.rows_fusable(1, bf16) and ops.rows_fusable(16, bf16)
    assert not ops.rows_fusable(17, bf16) and ops.rows_sinkable(17, bf16)
    assert ops.rows_sinkable(192, bf16) and not ops.rows_sinkable(193, bf16)
    # never both, and float32 neither
    for rows in range(0, 200):
        assert not (ops.rows_fusable(rows, bf16) and ops.rows_sinkable(rows, bf16))
        assert not ops.rows_fusable(rows, f32) and not ops.rows_sinkable(rows, f32)


def test_slices_along_k_stay_within_the_bound_a_block_reserves_for():
    from kvcore_amd.ops import library as ops

    for N in (64, 200, 2048, 4096, 8192, 14336, 16384, 20000, 28672, 32768, 57344, 128256):
        bound = ops.mid_slices_bound(N)
        assert 1 <= bound <= 64
        for K in (512, 1024, 4096, 14336, 28672, 65536):
            s = ops.mid_slices(N, K)
            assert 1 <= s <= bound, (N, K, s, bound)
            assert s <= K // 512
    assert ops.mid_slices(4096, 4096) == 4 and ops.mid_slices(128256, 4096) == 1
    assert ops.mid_slices(4096, 520) == 0  # a K the kernel does not take
