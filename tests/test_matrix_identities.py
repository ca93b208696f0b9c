"""The constant-matrix identities the reference's kernels rest on, brute-forced on small integer tiles with numpy
(exact arithmetic, so a transposed operand, a strict instead of a non-strict triangle or a wrong side of the
product fails):

  * reduction, 16 segments of 16 per tile: A . R, R = ones in the first column, leaves the 16 row sums in column 0
    (reference src/reduction/kernel.cuh:45-48);
  * reduction, one segment of 256 per tile: (R_row . A) . R_col is the sum of the whole tile (kernel.cuh:241-298);
  * scan, 16 segments of 16 per tile: A . U, U = upper triangular ones, is the row-wise inclusive prefix sum
    (src/prefixsum/kernel.cuh:48-83);
  * scan, one segment of 256 per tile (row-major order): L . A . O + A . U, L = strictly lower triangular ones,
    O = all ones (kernel.cuh:303-363);
  * carries: a tile's scan plus a constant matrix filled with the carry (the reference's fill_fragment(out, carry))
    continues a longer segment.

The build's kernels use the same identities with the tile as the B operand of a 16x16x32 product: ones . X gives
every column's total, and block upper-triangular ones U1 / U2 . X the prefix sums inside the two halves of a
column of 32; both are restated here on integer data as well."""
import numpy as np
import pytest


@pytest.fixture(scope="module")
def tiles():
    rng = np.random.default_rng(2024)
    return rng.integers(-9, 10, size=(50, 16, 16)).astype(np.int64)


def test_reduction_identities(tiles):
    R = np.zeros((16, 16), np.int64)
    R[:, 0] = 1
    Rrow = np.zeros((16, 16), np.int64)
    Rrow[0, :] = 1
    for A in tiles:
        P = A @ R
        assert np.array_equal(P[:, 0], A.sum(axis=1)) and not P[:, 1:].any()
        T = (Rrow @ A) @ R
        assert T[0, 0] == A.sum() and T.sum() == A.sum()
        # the wrong side gives column sums, which differ on a generic tile
        assert not np.array_equal((R.T @ A)[0, :], A.sum(axis=1)) or np.array_equal(A.sum(axis=0), A.sum(axis=1))


def test_scan_identities(tiles):
    U = np.triu(np.ones((16, 16), np.int64))           # U[k][j] = 1 for k <= j
    L = np.tril(np.ones((16, 16), np.int64), k=-1)     # strictly lower: rows before i
    O = np.ones((16, 16), np.int64)
    for A in tiles:
        S16 = A @ U
        assert np.array_equal(S16, np.cumsum(A, axis=1))
        S256 = L @ A @ O + A @ U
        assert np.array_equal(S256.reshape(-1), np.cumsum(A.reshape(-1)))
        # a non-strict L would count the own row twice
        assert not np.array_equal((np.tril(O) @ A @ O + A @ U).reshape(-1), np.cumsum(A.reshape(-1)))
    # a segment of 512 = two tiles: the second tile's scan continues with the first tile's total as carry
    A0, A1 = tiles[0], tiles[1]
    first = (L @ A0 @ O + A0 @ U).reshape(-1)
    second = (L @ A1 @ O + A1 @ U + first[-1] * O).reshape(-1)
    assert np.array_equal(np.r_[first, second], np.cumsum(np.r_[A0.reshape(-1), A1.reshape(-1)]))


def test_the_forms_with_the_tile_as_second_operand():
    """16x16x32 product D = M . X with the data X (32 x 16, column c = 32 consecutive elements, i.e. four chunks of 8)
    as the second operand: an all-ones M gives the column totals in every row, and the block upper-triangular U1 / U2
    (ones where k <= m inside the same chunk of 8, for chunks 0-1 and 2-3) give the inclusive prefix sums inside
    every chunk; the chunk totals are then carried across with an exclusive scan outside the product."""
    rng = np.random.default_rng(7)
    for _ in range(50):
        X = rng.integers(-9, 10, size=(32, 16)).astype(np.int64)
        ones = np.ones((16, 32), np.int64)
        assert np.array_equal((ones @ X)[3], X.sum(axis=0))
        m = np.arange(16)[:, None]
        k = np.arange(32)[None, :]
        U1 = ((k // 8 == m // 8) & (k <= m)).astype(np.int64)              # rows 0..15 <-> positions 0..15 of the column
        U2 = ((k // 8 == 2 + m // 8) & (k - 16 <= m)).astype(np.int64)     # rows 0..15 <-> positions 16..31
        D1, D2 = U1 @ X, U2 @ X
        for c in range(16):
            col = X[:, c]
            in_chunk = np.concatenate([np.cumsum(col[8 * q:8 * q + 8]) for q in range(4)])
            assert np.array_equal(np.r_[D1[:, c], D2[:, c]], in_chunk)
            chunk_totals = col.reshape(4, 8).sum(axis=1)
            carries = np.r_[0, np.cumsum(chunk_totals)[:-1]]
            assert np.array_equal(in_chunk + np.repeat(carries, 8), np.cumsum(col))
