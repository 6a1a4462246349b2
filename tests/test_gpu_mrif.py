"""GPU parity of MRI-FHD (mrif) in ori, GPTB and fused form against the CPU oracle, through
the C-ABI.

Bars: |d| <= 1e-3 + 1e-4|ref| against the fp64 oracle (hardware sine / cosine on the
phase in revolutions against libm on 2 pi phase; parity unpinned at the bit level, as for
mri-q); bit-exact between any two device forms of the same work: natural launch, any
ascending tiling of the position grid, any launch shape, fused and unfused.
"""
import numpy as np
import pytest
import torch

import oracle
import tacker_amd as ta
from gpu_util import dev, gemm_inputs, host, mrif_inputs, mrif_table, setup

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _init():
    setup()


def close(got, truth):
    return np.all(np.abs(got.astype(np.float64) - truth) <= 1e-3 + 1e-4 * np.abs(truth))


def same(a, b):
    return np.array_equal(host(a).view(np.uint32), host(b).view(np.uint32))


@pytest.mark.parametrize("numK,numX", [(64, 256), (1024, 1024), (2048, 512), (3, 256)])
def test_mrif_matches_fp64_oracle(numK, numX):
    k, phi, d, xyz = mrif_inputs(numK, numX)
    re, im = torch.zeros(numK, device="cuda:0"), torch.zeros(numK, device="cuda:0")
    ta.mrif_rhophi(dev(phi[0]), dev(phi[1]), dev(d[0]), dev(d[1]), re, im)
    want_re, want_im = oracle.mrif_rhophi(phi[0], phi[1], d[0], d[1])
    # one product of each sum is folded into it on the device: within an ulp of the sum
    np.testing.assert_allclose(host(re), want_re, rtol=3e-7, atol=1e-7)
    np.testing.assert_allclose(host(im), want_im, rtol=0, atol=1.5e-7)
    kv = np.concatenate([k, host(re)[:, None], host(im)[:, None]], 1).astype(np.float32)
    ta.mrif_set_kvalues(kv)
    x, y, z = dev(xyz[0]), dev(xyz[1]), dev(xyz[2])
    q0 = np.full(numX, 0.5, np.float32)
    tr, ti = oracle.mrif(kv, xyz[0], xyz[1], xyz[2], q0, q0, f64=True)
    outs = []
    for form in ("ori", "gptb"):
        outR, outI = dev(q0), dev(q0)
        if form == "ori":
            ta.ori_mrif(numK, x, y, z, outR, outI)
        else:
            ta.gptb_mrif(numK, x, y, z, outR, outI, launch_grid=3)
        assert close(host(outR), tr.astype(np.float64)) and close(host(outI), ti.astype(np.float64))
        outs.append((outR, outI))
    assert same(outs[0][0], outs[1][0]) and same(outs[0][1], outs[1][1])


def test_mrif_closed_forms():
    # x = 0: every voxel gets the sum of the table; one sample on the x axis rotates RhoPhi
    numK, numX = 300, 512
    k, phi, d, _ = mrif_inputs(numK, numX, seed=2)
    kv = mrif_table(k, phi, d)
    ta.mrif_set_kvalues(kv)
    zero = torch.zeros(numX, device="cuda:0")
    outR, outI = torch.zeros(numX, device="cuda:0"), torch.zeros(numX, device="cuda:0")
    ta.gptb_mrif(numK, zero, zero, zero, outR, outI)
    np.testing.assert_allclose(host(outR), kv[:, 3].astype(np.float64).sum(), rtol=1e-5)
    np.testing.assert_allclose(host(outI), kv[:, 4].astype(np.float64).sum(), rtol=1e-5)
    ta.mrif_set_kvalues(np.array([[1, 0, 0, 2, -1]], np.float32))
    xs = np.linspace(-0.5, 0.5, numX, endpoint=False).astype(np.float32)
    outR.zero_(); outI.zero_()
    ta.ori_mrif(1, dev(xs), zero, zero, outR, outI)
    want = (2 - 1j) * np.exp(2j * np.pi * xs.astype(np.float64))
    np.testing.assert_allclose(host(outR), want.real, atol=1e-5)
    np.testing.assert_allclose(host(outI), want.imag, atol=1e-5)


def test_mrif_block_positions_are_voxel_blocks_by_k_chunks():
    numK, numX = 300, 1024          # 4 voxel blocks x 3 chunks (128, 128, 44)
    k, phi, d, xyz = mrif_inputs(numK, numX, seed=5)
    kv = mrif_table(k, phi, d)
    ta.mrif_set_kvalues(kv)
    assert ta.mrif_blocks(numK, numX) == 12 and ta.mrif_blocks(0, numX) == 4 and ta.mrif_blocks(128, numX) == 4
    x, y, z = dev(xyz[0]), dev(xyz[1]), dev(xyz[2])
    q0 = np.zeros(numX, np.float32)
    refR, refI = dev(q0), dev(q0)
    ta.ori_mrif(numK, x, y, z, refR, refI)
    for cuts, kw in [([0, 12], {}), ([0, 1, 2, 12], dict(launch_grid=2)), ([0, 5, 6, 12], dict(launch_grid=1)),
                     ([0, 4, 8, 12], dict(launch_grid=7)), ([0, 11, 12], {})]:
        outR, outI = dev(q0), dev(q0)
        for a, b in zip(cuts, cuts[1:]):
            ta.gptb_mrif(numK, x, y, z, outR, outI, start=a, end=b, **kw)
        assert same(outR, refR) and same(outI, refI), cuts
    # one position: voxel block 2, chunk 1 -- nothing else is touched
    outR, outI = dev(q0), dev(q0)
    ta.gptb_mrif(numK, x, y, z, outR, outI, start=6, end=7)
    tr, ti = oracle.mrif(kv, xyz[0], xyz[1], xyz[2], q0, q0, start=6, end=7, kchunk=128, f64=True)
    assert close(host(outR), tr.astype(np.float64)) and close(host(outI), ti.astype(np.float64))
    assert not host(outR)[:512].any() and not host(outR)[768:].any() and host(outR)[512:768].any()


@pytest.mark.parametrize("seed", range(8))
def test_mrif_random_position_ranges_and_launch_shapes(seed):
    rng = np.random.default_rng(3000 + seed)
    numK = int(rng.integers(1, 420))
    numX = int(rng.choice([256, 512, 1024, 1536]))
    k, phi, d, xyz = mrif_inputs(numK, numX, seed=seed)
    kv = mrif_table(k, phi, d)
    ta.mrif_set_kvalues(kv)
    x, y, z = dev(xyz[0]), dev(xyz[1]), dev(xyz[2])
    total = ta.mrif_blocks(numK, numX)
    q0 = rng.uniform(-1, 1, numX).astype(np.float32)
    a = int(rng.integers(0, total + 1))
    b = int(rng.integers(a, 2 * total + 1))                       # may run past the grid and wrap
    mid = int(rng.integers(a, b + 1))
    grid = int(rng.choice([1, 2, 3, 5, 8, 40, 0]))
    outR, outI = dev(q0), dev(q0)
    ta.gptb_mrif(numK, x, y, z, outR, outI, start=a, end=b, launch_grid=grid)
    tr, ti = oracle.mrif(kv, xyz[0], xyz[1], xyz[2], q0, q0, start=a, end=b, kchunk=128, f64=True)
    tol = lambda got, want: np.all(np.abs(got.astype(np.float64) - want) <= 2e-3 + 2e-4 * np.abs(want))
    assert tol(host(outR), tr.astype(np.float64)) and tol(host(outI), ti.astype(np.float64)), (numK, numX, a, b, grid)
    # the same range cut in two, with another launch shape: the same bits
    pR, pI = dev(q0), dev(q0)
    other = int(rng.choice([1, 3, 7, 16, 0]))
    ta.gptb_mrif(numK, x, y, z, pR, pI, start=a, end=mid, launch_grid=other)
    ta.gptb_mrif(numK, x, y, z, pR, pI, start=mid, end=b, launch_grid=grid)
    assert same(pR, outR) and same(pI, outI), (numK, numX, a, mid, b, grid, other)


@pytest.mark.parametrize("variant", [None, "wave_256", "wave_512", "wg_1_1", "wg_1_2"])
def test_mix_tzgemm_mrif(variant):
    M, N, K = 256, 256, 256
    A, B = gemm_inputs(M, N, K, seed=10)
    numK, numX = 256, 2048
    k, phi, d, xyz = mrif_inputs(numK, numX)
    kv = mrif_table(k, phi, d)
    ta.mrif_set_kvalues(kv)
    x, y, z = dev(xyz[0]), dev(xyz[1]), dev(xyz[2])
    soloR, soloI = torch.zeros(numX, device="cuda:0"), torch.zeros(numX, device="cuda:0")
    ta.gptb_mrif(numK, x, y, z, soloR, soloI)
    solo_c = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dev(A), dev(B), solo_c)
    mix_c = torch.zeros((M, N), device="cuda:0")
    outR, outI = torch.zeros(numX, device="cuda:0"), torch.zeros(numX, device="cuda:0")
    ta.mix_tzgemm_mrif(numK, x, y, z, outR, outI, dev(A), dev(B), mix_c, variant=variant)
    assert same(mix_c, solo_c)
    assert same(outR, soloR) and same(outI, soloI)
    zq = np.zeros(numX, np.float32)
    tr, ti = oracle.mrif(kv, xyz[0], xyz[1], xyz[2], zq, zq, f64=True)
    assert close(host(outR), tr.astype(np.float64)) and close(host(outI), ti.astype(np.float64))


def test_creator_mrif_and_named_mixes():
    # createKernel("mrif") owns seeded buffers; the reference's mix names with mrif resolve
    g = ta.create_kernel("mrif")
    g.execute()
    for name in ("lbm_mrif", "mrif_stencil", "cp_mrif", "mrif_mriq"):
        ta.create_mix_kernel(name).execute()
    torch.cuda.synchronize()
    assert ta.spin_fail_flag() == 0
