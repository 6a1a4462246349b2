"""Pins oracle.mrif_rhophi and oracle.mrif (MRI-FHD, src/ori_kernel/mrif_kernel.cu:62-152).

The checks are formulations the C restatement does not share: complex arithmetic
in numpy (RhoPhi = conj(phi) * d; FhD = sum_k RhoPhi_k exp(i 2 pi k.x) as one
complex128 matrix product), closed forms (x = 0; a single sample on the real
axis), and the invariance of the result under any ascending tiling of the
(voxel blocks) x (k chunks) position grid."""
import numpy as np
import pytest

import oracle


def mrif_inputs(numK, numX, seed=13):
    rng = np.random.default_rng(seed)
    k = rng.uniform(-0.5, 0.5, (numK, 3)).astype(np.float32)
    phi = rng.uniform(0, 1, (2, numK)).astype(np.float32)
    d = rng.uniform(0, 1, (2, numK)).astype(np.float32)
    xyz = [rng.uniform(-0.5, 0.5, numX).astype(np.float32) for _ in range(3)]
    return k, phi, d, xyz


def table(k, phi, d):
    re, im = oracle.mrif_rhophi(phi[0], phi[1], d[0], d[1])
    return np.concatenate([k, re[:, None], im[:, None]], 1).astype(np.float32)


def test_rhophi_is_conj_phi_times_d():
    _, phi, d, _ = mrif_inputs(300, 256)
    re, im = oracle.mrif_rhophi(phi[0], phi[1], d[0], d[1])
    want = np.conj(phi[0].astype(np.float64) + 1j * phi[1]) * (d[0].astype(np.float64) + 1j * d[1])
    np.testing.assert_allclose(re, want.real, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(im, want.imag, rtol=1e-6, atol=1e-7)
    # conj(3 + 4i) * (1 + 2i) = 11 + 2i
    one = oracle.mrif_rhophi(*[np.array([v], np.float32) for v in (3, 4, 1, 2)])
    assert (one[0][0], one[1][0]) == (11.0, 2.0)


def test_x_zero_sums_the_table():
    k, phi, d, _ = mrif_inputs(128, 256)
    kv = table(k, phi, d)
    zero = np.zeros(256, np.float32)
    r, i = oracle.mrif(kv, zero, zero, zero, zero, zero)
    np.testing.assert_allclose(r, kv[:, 3].astype(np.float64).sum(), rtol=1e-5)
    np.testing.assert_allclose(i, kv[:, 4].astype(np.float64).sum(), rtol=1e-5)


def test_single_sample_rotates_rhophi():
    # one sample k = (1, 0, 0) with RhoPhi = 2 - 1i: FhD(x) = (2 - i) e^{i 2 pi x}
    kv = np.array([[1, 0, 0, 2, -1]], np.float32)
    x = np.linspace(-0.5, 0.5, 256, endpoint=False).astype(np.float32)
    zero = np.zeros(256, np.float32)
    r, i = oracle.mrif(kv, x, zero, zero, zero, zero)
    want = (2 - 1j) * np.exp(2j * np.pi * x.astype(np.float64))
    np.testing.assert_allclose(r, want.real, atol=2e-6)
    np.testing.assert_allclose(i, want.imag, atol=2e-6)
    # a quarter turn exchanges the parts with the sign a transposed product would get wrong:
    # (2 - i) * i = 1 + 2i
    q = np.full(256, 0.25, np.float32)
    r, i = oracle.mrif(kv, q, zero, zero, zero, zero)
    np.testing.assert_allclose(r, 1.0, atol=2e-6)
    np.testing.assert_allclose(i, 2.0, atol=2e-6)


@pytest.mark.parametrize("f64", [False, True])
def test_against_complex_matrix_product(f64):
    numK, numX = 200, 512
    k, phi, d, xyz = mrif_inputs(numK, numX)
    kv = table(k, phi, d)
    rng = np.random.default_rng(5)
    r0 = rng.uniform(-1, 1, numX).astype(np.float32)     # read-modify-write: starts from what is there
    i0 = rng.uniform(-1, 1, numX).astype(np.float32)
    r, i = oracle.mrif(kv, *xyz, r0, i0, f64=f64)
    X = np.stack(xyz, 1).astype(np.float64)
    phase = np.exp(2j * np.pi * (X @ kv[:, :3].astype(np.float64).T))
    want = (r0 + 1j * i0) + phase @ (kv[:, 3].astype(np.float64) + 1j * kv[:, 4])
    tol = dict(rtol=1e-6, atol=1e-6) if f64 else dict(rtol=1e-4, atol=1e-3)
    np.testing.assert_allclose(r, want.real, **tol)
    np.testing.assert_allclose(i, want.imag, **tol)


def test_positions_of_the_block_by_chunk_grid():
    numK, numX = 300, 768          # 3 voxel blocks x 3 chunks (128, 128, 44)
    k, phi, d, xyz = mrif_inputs(numK, numX)
    kv = table(k, phi, d)
    q0 = np.zeros(numX, np.float32)
    whole = oracle.mrif(kv, *xyz, q0, q0)
    grid = oracle.mrif(kv, *xyz, q0, q0, kchunk=128)
    assert np.array_equal(whole[0], grid[0]) and np.array_equal(whole[1], grid[1])
    for cuts in ([0, 1, 2, 9], [0, 4, 5, 9], [0, 3, 6, 9], [0, 7, 9]):
        r, i = q0, q0
        for a, b in zip(cuts, cuts[1:]):
            r, i = oracle.mrif(kv, *xyz, r, i, start=a, end=b, kchunk=128)
        assert np.array_equal(whole[0], r) and np.array_equal(whole[1], i)
    # one position = its voxel block with its record range, nothing else touched
    r, i = oracle.mrif(kv, *xyz, q0, q0, start=7, end=8, kchunk=128, f64=True)   # block 1, chunk 2
    assert not r[:256].any() and not r[512:].any()
    X = np.stack(xyz, 1).astype(np.float64)[256:512]
    want = np.exp(2j * np.pi * (X @ kv[256:, :3].astype(np.float64).T)) @ (kv[256:, 3].astype(np.float64) + 1j * kv[256:, 4])
    np.testing.assert_allclose(r[256:512], want.real, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(i[256:512], want.imag, rtol=1e-6, atol=1e-6)
