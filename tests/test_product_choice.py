"""The one table that says which kernel multiplies how many rows by which matrix
(``ops.choose_product``): the shapes of the three Llama sizes land where they were measured to
be fastest, and a kernel whose operands do not fit is never chosen."""

from __future__ import annotations

import pytest

from kvcore_amd.ops.library import choose_product


def test_row_counts_and_sizes_choose_the_kernel():
    qkv_8b, down_8b, head, down_70b, o_1b = (6144, 4096), (4096, 14336), (128256, 4096), (8192, 28672), (2048, 2048)
    for N, K in (qkv_8b, down_8b, head, down_70b, o_1b):
        for M in (1, 2, 8):
            assert choose_product(M, N, K) == "few rows"
        for M in (65, 512, 2048):
            assert choose_product(M, N, K) == "vendor"
    assert choose_product(12, *head) == "few rows" and choose_product(13, *head) == "vendor"
    assert choose_product(16, *head) == "vendor"
    assert choose_product(17, *head) == "shared rows" and choose_product(64, *head) == "shared rows"
    assert choose_product(16, *qkv_8b) == "few rows" and choose_product(17, *qkv_8b) == "vendor"
    assert choose_product(9, *down_8b) == "vendor" and choose_product(9, *down_70b) == "vendor"
    assert choose_product(32, *o_1b) == "few rows" and choose_product(33, *o_1b) == "vendor"


def test_a_kernel_that_cannot_take_the_operands_is_not_chosen():
    assert choose_product(4, 4096, 4096, few_rows_ok=False) == "vendor"
    assert choose_product(40, 128256, 4096, shared_rows_ok=False) == "vendor"
    assert choose_product(40, 128256, 4096, few_rows_ok=False) == "shared rows"


@pytest.mark.parametrize("limit", [1, 3, 6, 8, 11, 16, 20, 64, 100, 200, 1024])
def test_decode_graph_sizes(limit):
    """The batch sizes at which steps of single tokens are captured: rising, ending at the
    engine's limit, every size from 8 to 16 (a padded row costs the few-row products what a
    live one does), and never more than twice the live requests beyond one."""
    from kvcore_amd.engine.runner import _decode_buckets

    sizes = _decode_buckets(limit)
    assert sizes == sorted(set(sizes)) and sizes[0] == 1 and sizes[-1] == limit
    assert all(b in sizes for b in range(8, min(limit, 16) + 1))
    for live in range(1, limit + 1):
        padded = next(b for b in sizes if b >= live)
        assert padded <= limit and padded < 2 * live + (live == 1)
        if live > 16:
            assert padded - live < 32
