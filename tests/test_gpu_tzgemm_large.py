"""GPU parity of the large-tile build of general_ptb_tzgemm (256 x 256 macro tiles): against the
fp64 oracle within the tzgemm tolerance, and bit for bit against the 128 x 128 form, which every
fused kernel uses -- launched by key at small shapes (the host only picks it for shapes with a
tile for every CU) and through tacker_gptb_tzgemm at a shape it is picked for."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
import tacker_amd as ta
from gpu_util import dev, gemm_inputs, gemm_tolerance_ok, host, launch, setup

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _init():
    setup()


def launch_large(dA, dB, dC, M, N, K, start, end, grid):
    i, p = C.c_int, lambda t: C.c_void_p(t.data_ptr())
    tiles = (M // 64) * (N // 64)
    # general_ptb_tzgemm's list: A, B, C, M, N, K, 6 dims, start, step, end, thread_base
    launch("gptb_tzgemm@large", grid, 256,
           [p(dA), p(dB), p(dC), i(M), i(N), i(K), i(tiles), i(1), i(1), i(256), i(1), i(1), i(start), i(grid),
            i(end), i(0)])


# K = 128 runs only the tail of the K loop (4 chunks of 32), 256 one round of the steady loop, 1152 many
@pytest.mark.parametrize("M,N,K,grid", [(256, 256, 128, 1), (512, 768, 256, 6), (768, 512, 1152, 3),
                                        (1024, 1024, 640, 16), (512, 512, 4096, 4), (1280, 1024, 640, 7)])
def test_large_form_matches_oracle_and_the_small_form_bit_for_bit(M, N, K, grid):
    A, B = gemm_inputs(M, N, K, seed=M + N + K)
    dA, dB = dev(A), dev(B)
    small = torch.full((M, N), -7.0, device="cuda:0")
    ta.gptb_tzgemm(dA, dB, small)           # shapes below a tile per CU: the 128 x 128 or K-split form
    got = torch.full((M, N), -7.0, device="cuda:0")
    launch_large(dA, dB, got, M, N, K, 0, (M // 64) * (N // 64), grid)
    got, small = host(got), host(small)
    ok, fro, dmax = gemm_tolerance_ok(got, oracle.tzgemm(A, B, f64=True), K)
    assert ok and fro <= 1e-5, (fro, dmax)
    if ta.tzgemm_parts(M, N, K) == 1 and not ((M // 128) * (N // 128) <= 64 and K >= 512):
        # same order of additions per element as the macro-tile form (the K-split form adds in parts)
        assert np.array_equal(got.view(np.uint32), small.view(np.uint32))


@pytest.mark.parametrize("start,end,grid", [(0, 5, 2), (3, 9, 1), (17, 18, 6), (0, 0, 1), (0, 96, 4), (40, 96, 5)])
def test_large_form_tile_range_writes_only_its_reference_tiles(start, end, grid):
    M, N, K = 512, 768, 384
    A, B = gemm_inputs(M, N, K, seed=11)
    dA, dB = dev(A), dev(B)
    full = torch.zeros((M, N), device="cuda:0")
    launch_large(dA, dB, full, M, N, K, 0, 96, 6)
    full = host(full)
    Cd = torch.full((M, N), -7.0, device="cuda:0")
    launch_large(dA, dB, Cd, M, N, K, start, end, grid)
    got = host(Cd)
    want = oracle.tzgemm(A, B, C_init=np.full((M, N), -7.0, np.float32), start=start, end=end)
    mask = want != -7.0
    assert np.array_equal(got[~mask], want[~mask])       # untouched outside the range
    assert np.array_equal(got[mask], full[mask])         # same values as the full launch


def test_large_form_is_what_a_shape_with_a_tile_per_cu_runs_and_equals_the_fused_role():
    # 4096 x 4096: 256 tiles of 256 x 256.  The stand-alone launch (large form) against the GEMM
    # role of a fused launch (128 x 128 form) with no best-effort block in it: same bits; and
    # against the fp64 oracle on the first and last 128 rows.
    M, N, K = 4096, 4096, 512
    A, B = gemm_inputs(M, N, K, seed=7)
    dA, dB = dev(A), dev(B)
    alone = torch.full((M, N), -7.0, device="cuda:0")
    ta.gptb_tzgemm(dA, dB, alone)
    fused = torch.full((M, N), -7.0, device="cuda:0")
    grid = torch.zeros((8, 32, 128), device="cuda:0")
    out = grid.clone()
    ta.mix_tzgemm_stencil(1 / 6, 1 / 36, grid, out, dA, dB, fused, be_start=0, be_end=0)
    alone, fused = host(alone), host(fused)
    assert np.array_equal(alone.view(np.uint32), fused.view(np.uint32))
    for rows in (slice(0, 128), slice(M - 128, M)):
        ok, fro, dmax = gemm_tolerance_ok(alone[rows], oracle.tzgemm(A[rows], B, f64=True), K)
        assert ok and fro <= 1e-5, (fro, dmax)
    # a tile range through the same entry point
    part = torch.full((M, N), -7.0, device="cuda:0")
    ta.gptb_tzgemm(dA, dB, part, tile_start=100, tile_end=3000, launch_grid=64)
    part = host(part)
    pos = (np.arange(M)[:, None] // 64) * (N // 64) + np.arange(N)[None, :] // 64
    inside = (pos >= 100) & (pos < 3000)
    assert np.array_equal(part[inside], alone[inside]) and np.all(part[~inside] == -7.0)
    assert ta.spin_fail_flag() == 0
