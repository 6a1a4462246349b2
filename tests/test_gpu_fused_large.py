"""GPU parity of the 512-thread fused form whose GEMM role takes 256 x 128 tiles (variant
wave_256_large; csrc/kernels/tzgemm_large.h, tzgemm_role_large_rot): C bit for bit against the plain
GEMM kernel (128 x 128 tiles: every element is one fp32 accumulator over ascending steps of 32 k in
both) and against the fp64 oracle within the tzgemm tolerance, the partner's output bit for bit against
its own launch, over whole and partial ranges of both roles -- the checks the reference's generated
tests apply to every fused kernel (fusion/code/gen_test.py: fused vs unfused outputs)."""
import numpy as np
import pytest
import torch

import oracle
import tacker_amd as ta
from gpu_util import C0, C1, dev, gemm_inputs, gemm_tolerance_ok, host, lbm_inputs, setup, stencil_inputs

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _init():
    setup()


def stencil_partner(nz=10, ny=32, nx=256, seed=5):
    a0 = dev(stencil_inputs(nz, ny, nx, seed))
    out = a0.clone()
    return ta.ori_stencil_create(C0, C1, a0, out), ta.stencil_blocks(nx, ny, nz), out


def lbm_partner(sx=120, sy=6, sz=5, seed=7):
    src = dev(lbm_inputs(sx, sy, sz, seed))
    dst = torch.zeros_like(src)
    return ta.ori_lbm_create(src, dst, sx, sy, sz), sy * sz, dst, (src, dst)


# K = 128: only the tail of the K loop (two pairs of chunks); 256: one round of the steady loop; 384, 640, 1152:
# more rounds, whole and half; shapes with one tile, with fewer tiles than workgroups, with several rounds of
# tiles in a small launch, with a tile for every CU.  (768, 384, 640) is a K-split shape: there the kernel
# takes the 128 x 128 role's K-split form, as the plain kernel does.
@pytest.mark.parametrize("M,N,K,grid", [(256, 128, 128, 0), (512, 256, 256, 0), (768, 384, 640, 0),
                                        (1024, 1152, 640, 0), (1024, 512, 384, 8), (1280, 1024, 1152, 16),
                                        (2048, 4096, 128, 0)])
def test_gemm_role_with_256x128_tiles_gives_the_plain_kernels_bits(M, N, K, grid):
    assert M % 256 == 0 and N % 128 == 0 and K % 128 == 0
    A, B = gemm_inputs(M, N, K, seed=M + 3 * N + K)
    dA, dB = dev(A), dev(B)
    tiles = (M // 64) * (N // 64)
    plain = torch.full((M, N), -7.0, device="cuda:0")
    ta.gptb_tzgemm(dA, dB, plain)
    st_ori, blocks, st_out = stencil_partner()
    fresh = st_out.clone()
    st = ta.gptb_create(st_ori, 0, 0, 0, blocks)
    st.execute()
    want_st = host(st_out).copy()
    st_out.copy_(fresh)
    fused_c = torch.full((M, N), -7.0, device="cuda:0")
    tz = ta.gptb_create(ta.ori_tzgemm_create(dA, dB, fused_c), 0, 0, 0, tiles)
    mix = ta.mix_create(st, tz, 0, blocks, 0, tiles, variant="wave_256_large", launch_grid=grid)
    assert mix.info()["block"] == 512
    mix.execute()
    got, plain = host(fused_c), host(plain)
    assert np.array_equal(got.view(np.uint32), plain.view(np.uint32))
    if M * N * K <= 1024 * 1152 * 640:
        ok, fro, dmax = gemm_tolerance_ok(got, oracle.tzgemm(A, B, f64=True), K)
        assert ok and fro <= 1e-5, (fro, dmax)
    assert np.array_equal(host(st_out).view(np.uint32), want_st.view(np.uint32))
    assert ta.spin_fail_flag() == 0


@pytest.mark.parametrize("tile_range,be_range", [((0, 0), (0, None)), ((5, 23), (3, 40)), ((17, 18), (0, 0)),
                                                 ((0, 96), (7, 8)), ((40, 96), (0, None)), ((31, 65), (10, 11))])
def test_ranges_of_both_roles(tile_range, be_range):
    """[start, end) still counts the reference's 64 x 64 tiles: exactly those are written, whichever 256 x 128
    tile they lie in; the partner's blocks outside its range stay untouched"""
    M, N, K = 512, 768, 384
    A, B = gemm_inputs(M, N, K, seed=11)
    dA, dB = dev(A), dev(B)
    full = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dA, dB, full)
    full = host(full)
    lbm_ori, rows, lbm_dst, keep = lbm_partner()
    lo, hi = be_range[0], rows if be_range[1] is None else be_range[1]
    before = lbm_dst.clone()
    be = ta.gptb_create(lbm_ori, 0, 0, lo, hi)
    be.execute()
    want_lbm = host(lbm_dst).copy()
    lbm_dst.copy_(before)
    Cd = torch.full((M, N), -7.0, device="cuda:0")
    tz = ta.gptb_create(ta.ori_tzgemm_create(dA, dB, Cd), 0, 0, tile_range[0], tile_range[1])
    mix = ta.mix_create(be, tz, lo, hi, tile_range[0], tile_range[1], variant="wave_256_large")
    mix.execute()
    got = host(Cd)
    cols = N // 64
    for pos in range((M // 64) * cols):
        r, c = pos // cols, pos % cols
        tile = got[64 * r:64 * r + 64, 64 * c:64 * c + 64]
        if tile_range[0] <= pos < tile_range[1]:
            assert np.array_equal(tile.view(np.uint32), full[64 * r:64 * r + 64, 64 * c:64 * c + 64].view(np.uint32)), pos
        else:
            assert (tile == -7.0).all(), pos
    assert np.array_equal(host(lbm_dst).view(np.uint32), want_lbm.view(np.uint32))
    assert ta.spin_fail_flag() == 0


def test_a_shape_the_large_tiles_do_not_divide_takes_the_128x128_form_in_the_same_kernel():
    for M, N, K in [(384, 256, 384), (256, 256, 4608), (128, 128, 128)]:   # the second: reductions shared by workgroups
        A, B = gemm_inputs(M, N, K, seed=M + K)
        dA, dB = dev(A), dev(B)
        tiles = (M // 64) * (N // 64)
        plain = torch.zeros((M, N), device="cuda:0")
        ta.gptb_tzgemm(dA, dB, plain)
        st_ori, blocks, st_out = stencil_partner(seed=M)
        st = ta.gptb_create(st_ori, 0, 0, 0, blocks)
        Cd = torch.full((M, N), -7.0, device="cuda:0")
        tz = ta.gptb_create(ta.ori_tzgemm_create(dA, dB, Cd), 0, 0, 0, tiles)
        ta.mix_create(st, tz, 0, blocks, 0, tiles, variant="wave_256_large").execute()
        assert np.array_equal(host(Cd).view(np.uint32), host(plain).view(np.uint32)), (M, N, K)
    assert ta.spin_fail_flag() == 0


def test_the_host_picks_the_form_by_shape_where_kinfo_names_one():
    """createTzgemmMix without a variant: the pair's default form, except for a GEMM with a 256 x 128 tile for
    every CU when kinfo holds large_gemm_variant for the pair (lbm does, the stencil does not)"""
    lbm_ori, rows, _, keep = lbm_partner()
    st_ori, blocks, _ = stencil_partner()
    lbm = ta.gptb_create(lbm_ori, 0, 0, 0, rows)
    st = ta.gptb_create(st_ori, 0, 0, 0, blocks)

    def gemm(M, N, K):
        A = torch.zeros((M, K), dtype=torch.float16, device="cuda:0")
        B = torch.zeros((N, K), dtype=torch.float16, device="cuda:0")
        Cm = torch.zeros((M, N), device="cuda:0")
        return ta.gptb_create(ta.ori_tzgemm_create(A, B, Cm), 0, 0, 0, (M // 64) * (N // 64)), (A, B, Cm)

    big, hold1 = gemm(2048, 4096, 128)       # 8 x 32 = 256 tiles of 256 x 128
    small, hold2 = gemm(2048, 2048, 128)     # 128 of them: half the CUs would idle
    assert ta.mix_create(lbm, big, 0, rows, 0, 2048).info()["block"] == 512
    assert ta.mix_create(lbm, small, 0, rows, 0, 1024).info()["block"] == 768
    assert ta.mix_create(st, big, 0, blocks, 0, 2048).info()["block"] == 768
    assert ta.mix_create(lbm, big, 0, rows, 0, 2048, variant="wave_512").info()["block"] == 768
