"""Pins oracle.sgemm (Parboil SGEMM, src/ori_kernel/sgemm_kernel.cu:9-44).

The checks are formulations the C restatement does not share: a float64 matrix product in
numpy (tolerance), integer-valued operands (every product and sum exact in fp32, so the result must
equal an integer matrix product bit for bit -- a transposed operand, a wrong leading dimension, a
dropped alpha or beta fails here), a one-hot A (C = 2 C + 2 B[k]), the fused multiply-add per k
step against exact rational arithmetic rounded once, the known launch shapes the reference holds,
and the invariance of the result under any ascending tiling of the (blocks) x (k parts) position
grid."""
from fractions import Fraction

import numpy as np
import pytest

import oracle


def inputs(M, N, K, seed=3):
    rng = np.random.default_rng(seed)
    A = rng.uniform(0, 1, (K, M)).astype(np.float32)
    B = rng.uniform(0, 1, (K, N)).astype(np.float32)
    C0 = rng.uniform(-1, 1, (N, M)).astype(np.float32)
    return A, B, C0


def test_matches_a_float64_matrix_product():
    A, B, C0 = inputs(256, 48, 300)
    got = oracle.sgemm(A, B, C0)
    want = 2.0 * C0.astype(np.float64) + 2.0 * (B.astype(np.float64).T @ A.astype(np.float64))
    # 300 fused multiply-adds of values in [0,1): a few ulp of the sum
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-5)
    assert got.shape == (48, 256) and got.dtype == np.float32


def test_integer_operands_give_the_integer_product_exactly():
    rng = np.random.default_rng(4)
    M, N, K = 128, 32, 37                                   # K not a multiple of anything
    A = rng.integers(-8, 9, (K, M)).astype(np.float32)
    B = rng.integers(-8, 9, (K, N)).astype(np.float32)
    C0 = rng.integers(-100, 101, (N, M)).astype(np.float32)
    want = 2 * C0.astype(np.int64) + 2 * (B.astype(np.int64).T @ A.astype(np.int64))
    got = oracle.sgemm(A, B, C0)
    assert np.array_equal(got.astype(np.int64), want) and np.array_equal(got, want.astype(np.float32))
    # alpha and beta are both 2: C = 0 gives twice the product, A = 0 twice the old C
    assert np.array_equal(oracle.sgemm(A, B, np.zeros_like(C0)), (2 * (B.astype(np.int64).T @ A.astype(np.int64))))
    assert np.array_equal(oracle.sgemm(np.zeros_like(A), B, C0), 2 * C0)


def test_one_hot_rows_of_a_pick_rows_of_b():
    M, N, K = 128, 16, 20
    _, B, C0 = inputs(M, N, K, seed=5)
    A = np.zeros((K, M), np.float32)
    pick = np.arange(M) % K
    A[pick, np.arange(M)] = 1.0                              # row m of the product is B[pick[m]]
    got = oracle.sgemm(A, B, C0)
    want = C0 * np.float32(2) + np.float32(2) * B[pick].T    # one rounding: the sum
    assert np.array_equal(got, want)


def round_to_f32(x):
    """the float32 nearest to the rational x (no tie can occur for the inputs used here)"""
    guess = np.float32(float(x))
    best = min((guess, np.nextafter(guess, np.float32(np.inf)), np.nextafter(guess, np.float32(-np.inf))),
               key=lambda c: abs(Fraction(float(c)) - x))
    return np.float32(best)


def test_every_k_step_is_one_fused_multiply_add():
    # c = fl(a*b + c) with the product exact: restated with rationals; a separately rounded product differs
    M, N, K = 128, 16, 24
    A, B, C0 = inputs(M, N, K, seed=6)
    got = oracle.sgemm(A, B, C0)
    rows = (0, 57, 127)
    differs_from_unfused = False
    for m in rows:
        for n in (0, 9, 15):
            c = np.float32(0)
            u = np.float32(0)
            for k in range(K):
                c = round_to_f32(Fraction(float(A[k, m])) * Fraction(float(B[k, n])) + Fraction(float(c)))
                u = np.float32(u + np.float32(A[k, m] * B[k, n]))
            want = np.float32(np.float32(C0[n, m] * np.float32(2)) + np.float32(np.float32(2) * c))
            assert got[n, m] == want, (m, n)
            differs_from_unfused |= bool(u != c)
    assert differs_from_unfused                              # the test can tell the two apart


def test_launch_shapes_the_reference_holds():
    # grid (M/128, N/16) of blocks (16, 8): 4096 x 4128 -> 32 x 258 (src/ori_kernel/sgemm_kernel.cu:120-125);
    # kinfo's ori_blks 774 = 3 x 258, the M/10 run of fusion/code/kinfo.json
    assert oracle.sgemm_positions(4096, 4128, 4064, chunk=1 << 30) == 32 * 258
    assert oracle.sgemm_positions(384, 4128, 4064, chunk=1 << 30) == 774
    assert oracle.sgemm_positions(4096, 4128, 4064) == 32 * 258 * 64          # parts of 64 k steps


@pytest.mark.parametrize("K", [256, 300, 700, 64])
def test_any_ascending_tiling_of_the_position_grid_is_one_kernel(K):
    M, N = 256, 48
    A, B, C0 = inputs(M, N, K, seed=K)
    whole = oracle.sgemm(A, B, C0)
    total = oracle.sgemm_positions(M, N, K)
    assert total == 2 * 3 * -(-K // 64)
    assert np.array_equal(oracle.sgemm(A, B, C0, parts="chunks"), whole)
    rng = np.random.default_rng(K)
    for _ in range(4):
        cuts = sorted(set(rng.integers(0, total + 1, 3).tolist()) | {0, total})
        out, W = C0.copy(), np.full((N, M), np.nan, np.float32)      # whatever the workspace held before
        for a, b in zip(cuts, cuts[1:]):
            out = oracle.sgemm(A, B, out, start=a, end=b, parts="chunks", W=W)
        assert np.array_equal(out, whole), cuts
    # a range that runs past the grid wraps to block 0, part 0: with several parts only the workspace changes,
    # with one part the block is updated a second time
    twice = oracle.sgemm(A, B, C0, start=0, end=total + 1, parts="chunks")
    if K > oracle.SGEMM_K_CHUNK:
        assert np.array_equal(twice, whole)
    else:
        assert np.array_equal(twice, oracle.sgemm(A, B, whole, start=0, end=1))


def test_a_range_touches_only_its_blocks():
    M, N, K = 256, 48, 300
    A, B, C0 = inputs(M, N, K, seed=8)
    whole = oracle.sgemm(A, B, C0)
    part = oracle.sgemm(A, B, C0, start=1, end=4)             # blocks 1, 2, 3 of 6: (bx, by) = (1,0), (0,1), (1,1)
    for blk in range(6):
        bx, by = blk % 2, blk // 2
        rows, cols = slice(bx * 128, bx * 128 + 128), slice(by * 16, by * 16 + 16)
        want = whole if 1 <= blk < 4 else C0
        assert np.array_equal(part[cols, rows], want[cols, rows]), blk
