"""Decisions and layouts of the small-batch kernels that need no GPU: where the epilogues
that take other kernels' work apply, and the order of rows that the rotating one wants."""

import torch

from halite_amd.kernels import ops


def test_where_the_products_take_the_norm_and_the_rotation_into_themselves():
    tiled = torch.empty(0)
    # up to 16 rows: always, if there is a tiled copy and the width is a multiple of 8
    assert ops.norm_folds(1, 4096, 4096, tiled) and ops.norm_folds(16, 4096, 14336, tiled)
    assert not ops.norm_folds(8, 4096, 4096, None) and not ops.norm_folds(8, 4096, 4100, tiled)
    assert not ops.norm_folds(0, 4096, 4096, tiled)
    # 17 to 32 rows: matrices of up to 32 M elements whose rows are at most twice as long as they are many
    assert ops.norm_folds(17, 6144, 4096, tiled) and ops.norm_folds(32, 4096, 4096, tiled)
    assert not ops.norm_folds(32, 4096, 14336, tiled)  # down: long rows, and too large
    assert not ops.norm_folds(32, 3072, 8192, tiled)   # down of a smaller model: long rows
    assert not ops.norm_folds(32, 10240, 8192, tiled)  # too large
    assert not ops.norm_folds(33, 4096, 4096, tiled)


def test_rows_paired_for_the_rotating_epilogue():
    heads, D, width = 5, 48, 8
    w = torch.arange(heads * D, dtype=torch.float32)[:, None].repeat(1, width)  # row r holds r
    paired = ops.pair_rows_for_rotation(w, D)
    assert paired.shape == w.shape and sorted(paired[:, 0].tolist()) == list(range(heads * D))
    rows = paired[:, 0].long().view(heads, D // 16, 16)  # [head][tile of 16 rows][row in tile]
    for h in range(heads):
        for j in range(D // 16):
            first, second = rows[h, j, :8], rows[h, j, 8:]
            assert first.tolist() == [h * D + 8 * j + c for c in range(8)]
            assert second.tolist() == [h * D + D // 2 + 8 * j + c for c in range(8)]  # the partners
