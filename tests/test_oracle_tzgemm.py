"""Pins oracle.tzgemm* without retyping it: closed forms, numpy float64 matmul,
known answers held by the reference, and the tile-map bijection."""
import numpy as np
import pytest

import oracle


def test_dims_known_answers_from_reference_files():
    # K keys of src/config/kinfo-vgg16.json:8-12 are the rounded K of VGG16's
    # convs: kh*kw*Cin = 27, 576, 1152, 2304, 4608.
    for k_in, k_out in [(27, 128), (576, 512), (1152, 1152), (2304, 2304), (4608, 4608)]:
        assert oracle.tzgemm_dims(128, 128, k_in)[2] == k_out
    # src/Creator.cu:255-261: OriTZGEMMKernel(12800, 512, 4096)
    assert oracle.tzgemm_dims(12800, 512, 4096) == [12800, 512, 4096, 200 * 8]
    # benchmark configuration 1: 1024^3 -> 256 CTA tiles of 64x64
    assert oracle.tzgemm_dims(1024, 1024, 1024) == [1024, 1024, 1024, 256]
    # floor, not round; minimum 128 (src/tzgemm_kernel.h:31-33)
    assert oracle.tzgemm_dims(3136, 64, 255) == [3072, 128, 128, 48 * 2]
    assert oracle.tzgemm_dims(1, 1, 1) == [128, 128, 128, 4]


@pytest.mark.parametrize("M,N", [(128, 128), (256, 128), (128, 384), (512, 256)])
def test_tile_map_is_a_bijection(M, N):
    tiles = (M // 64) * (N // 64)
    seen = set()
    for pos in range(tiles):
        r, c = oracle.tzgemm_tile_origin(pos, N)
        assert r % 64 == 0 and c % 64 == 0 and 0 <= r < M and 0 <= c < N
        seen.add((r, c))
    assert len(seen) == tiles
    # row-major over the 64x64 tile grid
    assert oracle.tzgemm_tile_origin(1, N) == ((0, 64) if N > 64 else (64, 0))
    assert oracle.tzgemm_tile_origin(N // 64, N) == (64, 0)


def test_identity_gives_scaled_transpose_exactly():
    rng = np.random.default_rng(1)
    K = 128
    A = np.eye(128, K, dtype=np.float16)
    B = rng.uniform(-1, 1, (256, K)).astype(np.float16)
    Cm = oracle.tzgemm(A, B)
    want = (B.astype(np.float32).T * np.float32(1.1)).astype(np.float32)
    assert np.array_equal(Cm, want)
    assert np.array_equal(oracle.tzgemm(A, B, f64=True), want)


def test_all_ones_gives_alpha_k():
    for K in (128, 256):
        A = np.ones((128, K), np.float16)
        B = np.ones((128, K), np.float16)
        assert np.all(oracle.tzgemm(A, B) == np.float32(K) * np.float32(1.1))


def test_against_numpy_float64_nonsquare_nonsymmetric():
    rng = np.random.default_rng(2)
    M, N, K = 128, 256, 384
    A = rng.uniform(-1, 1, (M, K)).astype(np.float16)
    B = rng.uniform(-1, 1, (N, K)).astype(np.float16)
    truth = float(np.float32(1.1)) * (A.astype(np.float64) @ B.astype(np.float64).T)
    c64 = oracle.tzgemm(A, B, f64=True)
    c32 = oracle.tzgemm(A, B)
    assert c64.shape == (M, N)
    np.testing.assert_allclose(c64, truth, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(c32, truth, rtol=1e-5, atol=5e-4)
    # alpha = 1 is the plain product
    np.testing.assert_allclose(oracle.tzgemm(A, B, alpha=1.0, f64=True),
                               A.astype(np.float64) @ B.astype(np.float64).T, rtol=1e-6, atol=1e-6)


def test_tile_range_writes_only_its_tiles():
    rng = np.random.default_rng(3)
    M, N, K = 256, 256, 128
    A = rng.uniform(-1, 1, (M, K)).astype(np.float16)
    B = rng.uniform(-1, 1, (N, K)).astype(np.float16)
    full = oracle.tzgemm(A, B)
    sentinel = np.full((M, N), -7.0, np.float32)
    part = oracle.tzgemm(A, B, C_init=sentinel, start=3, end=9)
    mask = np.zeros((M, N), bool)
    for pos in range(3, 9):
        r, c = oracle.tzgemm_tile_origin(pos, N)
        mask[r:r + 64, c:c + 64] = True
    assert np.array_equal(part[mask], full[mask])
    assert np.all(part[~mask] == -7.0)


def test_subnormal_and_special_halfs_convert_like_numpy():
    # every finite half bit pattern through A=diag trick is too slow; instead
    # multiply a column of all 2^16 patterns by one.
    bits = np.arange(0, 0x7c00, dtype=np.uint16)  # all non-negative finite halfs
    vals = bits.view(np.float16)
    n = 128 * 248  # 31744 = 0x7c00
    assert vals.size == n
    A = np.zeros((128, 128), np.float16)
    A[:, 0] = 1
    for chunk in range(0, n, 128):
        B = np.zeros((128, 128), np.float16)
        B[:, 0] = vals[chunk:chunk + 128]
        Cm = oracle.tzgemm(A, B, alpha=1.0)
        assert np.array_equal(Cm[0], vals[chunk:chunk + 128].astype(np.float32))
