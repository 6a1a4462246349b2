"""Pins oracle.fft (Parboil's batched 256-point FFT, src/ori_kernel/fft_kernel.cu:11-61).

The C restatement walks the reference's eight radix-2 stages with their shared-memory exchanges.
The checks are formulations it does not share: the discrete Fourier transform in float64 (numpy's
FFT and, for a few bins, the defining sum), unit impulses (the transform of e_m is the m-th row of
the DFT matrix: a wrong sign of the angle, a wrong exchange index or bit-reversed output fails here),
pure tones (one non-zero bin), linearity, Parseval's identity, and the position bookkeeping of the
GPTB form (a position is a batch entry, positions past the batch wrap, the others are untouched)."""
import numpy as np

import oracle


def as_complex(a):
    return a[..., 0].astype(np.float64) + 1j * a[..., 1].astype(np.float64)


def batch(n, seed=5):
    rng = np.random.default_rng(seed)
    return rng.uniform(-1, 1, (n, 256, 2)).astype(np.float32)


def test_matches_the_float64_transform():
    d = batch(6)
    got = as_complex(oracle.fft(d))
    want = np.fft.fft(as_complex(d), axis=1)
    # eight stages of fp32 butterflies on sums of magnitude ~16: a few 1e-6
    assert np.abs(got - want).max() <= 2e-5
    assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 5e-7
    # the defining sum for three bins of one entry, no FFT involved
    x = as_complex(d[2])
    n = np.arange(256)
    for k in (0, 1, 37, 255):
        assert abs(got[2, k] - np.sum(x * np.exp(-2j * np.pi * k * n / 256))) <= 2e-5


def test_unit_impulses_give_the_rows_of_the_dft_matrix():
    ms = [0, 1, 2, 3, 64, 127, 128, 129, 200, 255]
    d = np.zeros((len(ms), 256, 2), np.float32)
    for i, m in enumerate(ms):
        d[i, m, 0] = 1.0
    got = as_complex(oracle.fft(d))
    k = np.arange(256)
    for i, m in enumerate(ms):
        assert np.abs(got[i] - np.exp(-2j * np.pi * k * m / 256)).max() <= 1e-6, m
    # an imaginary impulse: i times the row
    d = np.zeros((1, 256, 2), np.float32)
    d[0, 5, 1] = 1.0
    assert np.abs(as_complex(oracle.fft(d))[0] - 1j * np.exp(-2j * np.pi * k * 5 / 256)).max() <= 1e-6


def test_pure_tones_land_in_one_bin():
    n = np.arange(256)
    for f in (0, 1, 17, 128, 255):
        x = np.exp(2j * np.pi * f * n / 256)
        d = np.stack([x.real, x.imag], -1).astype(np.float32)[None]
        got = as_complex(oracle.fft(d))[0]
        assert abs(got[f] - 256) <= 1e-3
        others = np.delete(got, f)
        assert np.abs(others).max() <= 2e-4, f


def test_linearity_and_parseval():
    a, b = batch(3, 1), batch(3, 2)
    fa, fb = as_complex(oracle.fft(a)), as_complex(oracle.fft(b))
    fab = as_complex(oracle.fft((a + np.float32(0.5) * b).astype(np.float32)))
    assert np.abs(fab - (fa + 0.5 * fb)).max() <= 5e-5
    energy_in = np.sum(np.abs(as_complex(a)) ** 2, axis=1)
    energy_out = np.sum(np.abs(fa) ** 2, axis=1) / 256
    np.testing.assert_allclose(energy_out, energy_in, rtol=1e-6)


def test_positions_are_batch_entries_and_wrap():
    d = batch(5, 9)
    whole = oracle.fft(d)
    part = oracle.fft(d, 1, 3)
    assert np.array_equal(part[1:3], whole[1:3]) and np.array_equal(part[[0, 3, 4]], d[[0, 3, 4]])
    # positions 4, 5, 6 of a batch of 5: entries 4, 0, 1 (src/gptb_kernel/fft_kernel.cu:56: block_pos % grid_dimension_x)
    wrapped = oracle.fft(d, 4, 7)
    assert np.array_equal(wrapped[[4, 0, 1]], whole[[4, 0, 1]]) and np.array_equal(wrapped[[2, 3]], d[[2, 3]])
    # the transform is in place: a position served twice is transformed twice
    twice = oracle.fft(d, 0, 10)
    assert np.array_equal(twice, oracle.fft(whole))
    assert np.array_equal(oracle.fft(d, 2, 2), d)


def test_reference_input_stream():
    # srand(54321); rand() / (float)RAND_MAX * 2 - 1 (src/ori_kernel/fft_kernel.cu:93-103): the C library's
    # generator, the one the cp atoms come from as well
    s = oracle.fft_source(4)
    assert s.shape == (4, 256, 2) and s.dtype == np.float32
    assert -1.0 <= s.min() and s.max() <= 1.0 and abs(s.mean()) < 0.05
    assert np.array_equal(s, oracle.fft_source(4)) and np.array_equal(oracle.fft_source(2), s[:2])
    atoms = oracle.cp_initatoms(1, 4096, 4096, 1, 0.1)
    # the first draw of the same seeded stream: atom x = rand() / RAND_MAX * 409 (the size is held in an unsigned,
    # src/ori_kernel/cp_kernel.cu:186,197,203) against 2 * that - 1 here
    assert abs((s[0, 0, 0] + 1) / 2 * 409 - atoms.reshape(-1)[0]) <= 1e-4
