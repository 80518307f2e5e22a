"""The two fragment-order layouts, pinned on the CPU element by element: the copy of a matrix
that the decode products read, and the normalised rows of a decode step in the same order.
Both put element (row, k) of a piece of 16 rows x 32 of K at lane (k % 32) / 8 * 16 + row % 16,
value k % 8 of that lane: the order in which a 16x16x32 matrix instruction takes its operands."""
import torch

from kappai_amd.kernels import ops


def place_in_piece(row: int, k: int) -> int:
    return ((k % 32) // 8 * 16 + row % 16) * 8 + k % 8


def test_matrix_copy_in_fragment_order():
    N, K = 48, 96
    w = torch.arange(N * K, dtype=torch.float32).remainder(251).to(torch.bfloat16).reshape(N, K)
    flat = ops.fragment_order(w).reshape(-1)
    for n in range(N):
        for k in range(K):
            piece = (n // 16) * (K // 32) + k // 32
            assert flat[piece * 512 + place_in_piece(n, k)] == w[n, k], (n, k)
    assert ops.fragment_order(w[:40]) is None and ops.fragment_order(w[:, :72]) is None
    assert ops.fragment_order(w.float()) is None


def test_rows_in_fragment_order_come_back_as_rows():
    n, D = 11, 96
    rows = torch.arange(n * D, dtype=torch.float32).remainder(241).to(torch.bfloat16).reshape(n, D)
    data = torch.full((16 * D,), -1.0, dtype=torch.bfloat16)
    for i in range(n):
        for k in range(D):
            data[(k // 32) * 512 + place_in_piece(i, k)] = rows[i, k]
    frag = ops.FragmentRows(data.reshape(16, D), n, resid=torch.zeros(n, D))
    assert frag.shape == (n, D) and frag.dtype == torch.bfloat16
    assert torch.equal(frag.materialize(), rows)
    assert ops.FragmentRows.fits(16, 2048, torch.bfloat16)
    assert not ops.FragmentRows.fits(17, 2048, torch.bfloat16)       # one tile of 16 rows
    assert not ops.FragmentRows.fits(8, 2040, torch.bfloat16)        # whole pieces of 32 of K
    assert not ops.FragmentRows.fits(8, 2048, torch.float32)
