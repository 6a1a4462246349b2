"""GPU parity of the FFT partner (src/ori_kernel/fft_kernel.cu, src/gptb_kernel/fft_kernel.cu,
src/mix_kernel/tzgemm_fft.cu): against the oracle's walk through the reference's stages within
|d| <= 1e-4 + 1e-5 |ref| (the twiddles are table values here, cosf/sinf of a rounded angle there) and
against the float64 transform; the natural launch, the GPTB form over any tiling of its positions
and every fused variant give the same bits as each other."""
import numpy as np
import pytest
import torch

import oracle
import tacker_amd as ta
from gpu_util import dev, gemm_inputs, gemm_tolerance_ok, host, setup

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _init():
    setup()


def batch(n, seed=3):
    return np.random.default_rng(seed).uniform(-1, 1, (n, 256, 2)).astype(np.float32)


def close(got, want):
    return bool(np.all(np.abs(got.astype(np.float64) - want.astype(np.float64)) <= 1e-4 + 1e-5 * np.abs(want)))


def as_complex(a):
    return a[..., 0].astype(np.float64) + 1j * a[..., 1].astype(np.float64)


def bits(t):
    return host(t).view(np.uint32)


@pytest.mark.parametrize("n", [1, 7, 300])
def test_ori_and_gptb_forms_match_the_oracle_and_the_float64_transform(n):
    d = batch(n, seed=n)
    want = oracle.fft(d)
    d_ori, d_gptb, d_small = dev(d), dev(d), dev(d)
    ta.ori_fft(d_ori)
    ta.gptb_fft(d_gptb)
    ta.gptb_fft(d_small, launch_grid=3, launch_block=64)
    assert close(host(d_ori), want)
    truth = np.fft.fft(as_complex(d), axis=1)
    got = as_complex(host(d_ori))
    assert np.linalg.norm(got - truth) / np.linalg.norm(truth) <= 5e-7
    # one transform is one wavefront's work whatever the launch: the three forms agree bit for bit
    assert np.array_equal(bits(d_gptb), bits(d_ori)) and np.array_equal(bits(d_small), bits(d_ori))
    assert ta.spin_fail_flag() == 0


def test_impulses_and_tones():
    d = np.zeros((4, 256, 2), np.float32)
    d[0, 0, 0] = 1.0
    d[1, 3, 0] = 1.0
    d[2, 200, 1] = 1.0
    n = np.arange(256)
    tone = np.exp(2j * np.pi * 17 * n / 256)
    d[3, :, 0], d[3, :, 1] = tone.real, tone.imag
    t = dev(d)
    ta.gptb_fft(t)
    got = as_complex(host(t))
    assert np.abs(got[0] - 1).max() <= 1e-6
    assert np.abs(got[1] - np.exp(-2j * np.pi * n * 3 / 256)).max() <= 1e-6
    assert np.abs(got[2] - 1j * np.exp(-2j * np.pi * n * 200 / 256)).max() <= 1e-6
    assert abs(got[3, 17] - 256) <= 1e-3 and np.abs(np.delete(got[3], 17)).max() <= 2e-4


@pytest.mark.parametrize("seed", range(6))
def test_any_tiling_of_the_positions_gives_the_one_kernel(seed):
    rng = np.random.default_rng(700 + seed)
    n = int(rng.choice([5, 64, 257, 1000]))
    d = batch(n, seed=seed)
    whole = dev(d)
    ta.ori_fft(whole)
    cuts = sorted(set(rng.integers(0, n + 1, 4).tolist()) | {0, n})
    t = dev(d)
    for a, b in zip(cuts, cuts[1:]):
        ta.gptb_fft(t, a, b, launch_grid=int(rng.choice([1, 7, 64, 256])), launch_block=int(rng.choice([64, 128, 256])))
    assert np.array_equal(bits(t), bits(whole))
    # positions past the batch wrap (src/gptb_kernel/fft_kernel.cu:56); each is served once, by one wavefront
    if n >= 5:
        t = dev(d)
        ta.gptb_fft(t, n - 2, n + 3, launch_grid=2)
        want = oracle.fft(d, n - 2, n + 3)
        got = host(t)
        touched = [n - 2, n - 1, 0, 1, 2]
        assert close(got[touched], want[touched])
        rest = np.setdiff1d(np.arange(n), touched)
        assert np.array_equal(got[rest], d[rest])


@pytest.mark.parametrize("variant", [None, "wave_256", "wave_512", "wg_1_1", "wg_1_2"])
def test_mix_tzgemm_fft(variant):
    M, N, K = 256, 256, 256
    A, B = gemm_inputs(M, N, K, seed=21)
    d = batch(333, seed=22)
    solo_c = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dev(A), dev(B), solo_c)
    solo_d = dev(d)
    ta.gptb_fft(solo_d)
    mix_c = torch.zeros((M, N), device="cuda:0")
    mix_d = dev(d)
    ta.mix_tzgemm_fft(mix_d, dev(A), dev(B), mix_c, variant=variant)
    assert np.array_equal(host(mix_c), host(solo_c))
    assert np.array_equal(bits(mix_d), bits(solo_d))
    assert close(host(mix_d), oracle.fft(d))
    ok, fro, dmax = gemm_tolerance_ok(host(mix_c), oracle.tzgemm(A, B, f64=True), K)
    assert ok and fro <= 1e-5
    # a slice of the transforms rides with a slice of the tiles; the rest follows in a second fused launch
    mix_d = dev(d)
    mix_c.zero_()
    ta.mix_tzgemm_fft(mix_d, dev(A), dev(B), mix_c, be_start=0, be_end=100, tile_start=0, tile_end=5, variant=variant)
    ta.mix_tzgemm_fft(mix_d, dev(A), dev(B), mix_c, be_start=100, be_end=333, tile_start=5, tile_end=16, variant=variant)
    assert np.array_equal(bits(mix_d), bits(solo_d))
    assert np.array_equal(host(mix_c), host(solo_c))
    assert ta.spin_fail_flag() == 0


def test_creator_object_is_the_references_batch():
    # createKernel("fft"): 10240 transforms of rand() values after srand(54321) (src/ori_kernel/fft_kernel.cu:87-131)
    k = ta.create_kernel("fft")
    info = k.info()
    assert (info["ptb_start"], info["ptb_end"], info["ori_grid_x"]) == (0, 10240, 10240)
    src = oracle.fft_source(10240)
    size = src.size * 4
    assert ta.lib().tkMemcpy(k.param(0), src.ctypes.data, size, 1) == 0   # the object is memoised: start from its source
    k.execute()
    torch.cuda.synchronize()
    got = ta.device_to_host(k.param(0), (10240, 256, 2), np.float32)
    for first in (0, 5000, 10200):
        assert close(got[first:first + 40], oracle.fft(src[first:first + 40]))
    truth = np.fft.fft(as_complex(src[:512]), axis=1)
    assert np.linalg.norm(as_complex(got[:512]) - truth) / np.linalg.norm(truth) <= 5e-7
    assert ta.spin_fail_flag() == 0


def test_bad_arguments_are_refused():
    lib = ta.lib()
    t = dev(batch(2))
    assert lib.tacker_ori_fft(None, 2, None) == 1
    assert lib.tacker_gptb_fft(t.data_ptr(), 0, 0, 1, 0, 0, None) == 1
    assert lib.tacker_gptb_fft(t.data_ptr(), 2, 0, 2, 0, 100, None) == 1     # block not a multiple of 64
