"""GPU parity: every kernel of the path, in ori, GPTB and fused form, against the
CPU oracle on the same seeded inputs, through the C-ABI.

Bars: bit-exact for stencil, lbm, cp (ordered fp32, contraction off on both
sides), for all [start,end) bookkeeping, and for fused-vs-unfused device output;
tzgemm |d| <= 5e-3 + 1e-5|ref| and rel-Frobenius <= 1e-5 against the fp64 oracle;
mri-q |d| <= 1e-3 + 1e-4|ref| against the fp64 oracle.
"""
import numpy as np
import pytest
import torch

import oracle
import tacker_amd as ta
from gpu_util import (C0, C1, dev, gemm_inputs, gemm_tolerance_ok, host, lbm_inputs, mrif_inputs, mrif_table,
                      mriq_inputs, setup, stencil_inputs)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _init():
    setup()


# ------------------------------------------------------------------ tzgemm
# shapes with at most 64 macro tiles and K >= 512 take the K-split form of the kernel (one
# reference tile per workgroup, K cut over its waves), the others the macro-tile form
@pytest.mark.parametrize("M,N,K", [(128, 128, 128), (256, 384, 128), (1024, 1024, 1024), (384, 128, 640),
                                   (128, 512, 4608), (128, 256, 25088), (1152, 1024, 512), (256, 128, 576 + 64)])
def test_gptb_tzgemm_matches_fp64_oracle(M, N, K):
    A, B = gemm_inputs(M, N, K)
    Cd = torch.full((M, N), -7.0, device="cuda:0")
    ta.gptb_tzgemm(dev(A), dev(B), Cd)
    got = host(Cd)
    truth = oracle.tzgemm(A, B, f64=True)
    ok, fro, dmax = gemm_tolerance_ok(got, truth, K)
    assert ok and fro <= 1e-5, (fro, dmax)


def test_tzgemm_closed_forms():
    K = 256
    A = np.eye(128, K, dtype=np.float16)
    rng = np.random.default_rng(3)
    B = rng.uniform(-1, 1, (256, K)).astype(np.float16)
    Cd = torch.zeros((128, 256), device="cuda:0")
    ta.gptb_tzgemm(dev(A), dev(B), Cd)
    assert np.array_equal(host(Cd), B.astype(np.float32).T[:128] * np.float32(1.1))
    ones = np.ones((128, K), np.float16)
    Cd2 = torch.zeros((128, 128), device="cuda:0")
    ta.gptb_tzgemm(dev(ones), dev(ones), Cd2)
    assert np.all(host(Cd2) == np.float32(K) * np.float32(1.1))


@pytest.mark.parametrize("K", [128, 768])          # macro-tile form, K-split form
@pytest.mark.parametrize("start,end,grid", [(0, 5, 0), (3, 9, 8), (7, 8, 16), (0, 0, 0), (0, 24, 3)])
def test_tzgemm_tile_range_writes_only_its_tiles(start, end, grid, K):
    M, N = 256, 384
    A, B = gemm_inputs(M, N, K, seed=5)
    full = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dev(A), dev(B), full)
    full = host(full)
    Cd = torch.full((M, N), -7.0, device="cuda:0")
    ta.gptb_tzgemm(dev(A), dev(B), Cd, tile_start=start, tile_end=end, launch_grid=grid)
    got = host(Cd)
    want = oracle.tzgemm(A, B, C_init=np.full((M, N), -7.0, np.float32), start=start, end=end)
    mask = want != -7.0
    assert np.array_equal(got[~mask], want[~mask])       # untouched outside the range
    assert np.array_equal(got[mask], full[mask])         # same values as the full launch


# A workgroup with several macro tiles refills its LDS ring for each of them.  Few workgroups, K just
# above and well above the ring depth (4 chunks of 64), ranges with holes: same bits as one tile per
# workgroup.
@pytest.mark.parametrize("M,N,K", [(256, 384, 384), (1152, 1024, 512), (1280, 1024, 640), (1152, 1024, 1280)])
def test_tzgemm_several_tiles_per_workgroup_equal_one_tile_per_workgroup(M, N, K):
    assert (M // 128) * (N // 128) > 64 or K < 512          # shapes of the macro-tile form
    A, B = gemm_inputs(M, N, K, seed=M + N + K)
    dA, dB = dev(A), dev(B)
    tiles = (M // 64) * (N // 64)
    ref = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dA, dB, ref, launch_grid=256)             # at most one macro tile per workgroup
    ref = host(ref)
    ok, fro, dmax = gemm_tolerance_ok(ref, oracle.tzgemm(A, B, f64=True), K)
    assert ok and fro <= 1e-5, (fro, dmax)
    for grid in (1, 2, 3, 5, 8):
        Cd = torch.full((M, N), -7.0, device="cuda:0")
        ta.gptb_tzgemm(dA, dB, Cd, launch_grid=grid)
        assert np.array_equal(host(Cd).view(np.uint32), ref.view(np.uint32)), grid
    # ranges that skip macro tiles between the ones a workgroup takes
    for start, end, grid in ((0, tiles // 2, 2), (tiles // 3, tiles, 1), (5, tiles - 7, 3)):
        Cd = torch.full((M, N), -7.0, device="cuda:0")
        ta.gptb_tzgemm(dA, dB, Cd, tile_start=start, tile_end=end, launch_grid=grid)
        want = oracle.tzgemm(A, B, C_init=np.full((M, N), -7.0, np.float32), start=start, end=end)
        mask = want != -7.0
        got = host(Cd)
        assert np.array_equal(got[~mask], want[~mask]) and np.array_equal(got[mask], ref[mask]), (start, end, grid)


# Shapes whose tiles are so few that the reduction of one tile is shared by several workgroups (the
# batch-1 layers of VGG16: conv5, conv4, fc2, fc3 with 8, 2, 2, 8 parts).  Who stores C is decided by
# arrival order, what is stored is not: every launch -- whatever its grid, however its range is cut --
# must give the same bits, and the arrival counters must be back at zero for the next one.
@pytest.mark.parametrize("M,N,K", [(256, 512, 4608), (896, 512, 4608), (4096, 128, 4096), (1024, 128, 4096),
                                   (128, 4096, 4096), (128, 1024, 4096)])
def test_tzgemm_reduction_shared_by_workgroups(M, N, K):
    parts = ta.tzgemm_parts(M, N, K)
    assert parts > 1 and ta.tzgemm_workspace_bytes(M, N, K) >= (M // 64) * (N // 64) * parts * 64 * 64 * 4
    A, B = gemm_inputs(M, N, K, seed=M + K)
    dA, dB = dev(A), dev(B)
    Cd = torch.full((M, N), -7.0, device="cuda:0")
    ta.gptb_tzgemm(dA, dB, Cd)
    first = host(Cd).copy()
    ok, fro, dmax = gemm_tolerance_ok(first, oracle.tzgemm(A, B, f64=True), K)
    assert ok and fro <= 1e-5, (fro, dmax)
    tiles = (M // 64) * (N // 64)
    for grid in (0, 8, 17, 64, 256, 300):
        Cd.fill_(-7.0)
        ta.gptb_tzgemm(dA, dB, Cd, launch_grid=grid)
        assert np.array_equal(host(Cd).view(np.uint32), first.view(np.uint32)), grid
    # the range cut into three launches, the middle one first
    cuts = [0, tiles // 3 + 1, tiles - 5, tiles]
    Cd.fill_(-7.0)
    for i in (1, 0, 2):
        ta.gptb_tzgemm(dA, dB, Cd, tile_start=cuts[i], tile_end=cuts[i + 1], launch_grid=(0, 40, 256)[i])
    assert np.array_equal(host(Cd).view(np.uint32), first.view(np.uint32))
    # a range of one tile leaves the others alone
    Cd.fill_(-7.0)
    ta.gptb_tzgemm(dA, dB, Cd, tile_start=3, tile_end=4)
    got = host(Cd)
    want = oracle.tzgemm(A, B, C_init=np.full((M, N), -7.0, np.float32), start=3, end=4)
    mask = want != -7.0
    assert np.array_equal(got[~mask], want[~mask]) and np.array_equal(got[mask], first[mask])


def test_tzgemm_shared_reduction_never_reads_a_previous_launch():
    # the workspace keeps the partial tiles of the last launch; a launch on other operands must not
    # see any of them (they were written and are read across the XCDs' separate L2s).  The witnesses
    # are first launches into output buffers of their own: their workspaces are new and zeroed.
    M, N, K = 256, 512, 4608
    ta.tzgemm_release_workspaces()
    dev_pairs = [tuple(dev(x) for x in gemm_inputs(M, N, K, seed=900 + i)) for i in range(4)]
    witnesses = []
    for dA, dB in dev_pairs:
        out = torch.zeros((M, N), device="cuda:0")      # kept alive: four different addresses
        ta.gptb_tzgemm(dA, dB, out)
        witnesses.append(out)
    want = [host(w).view(np.uint32).copy() for w in witnesses]
    assert not np.array_equal(want[0], want[1])
    used = torch.zeros((M, N), device="cuda:0")
    for rounds in range(3):
        for i, (dA, dB) in enumerate(dev_pairs):
            ta.gptb_tzgemm(dA, dB, used, launch_grid=(0, 64, 256)[rounds])
            assert np.array_equal(host(used).view(np.uint32), want[i]), (rounds, i)


@pytest.mark.parametrize("M,N,K", [(256, 512, 4608), (128, 4096, 4096)])
def test_tzgemm_shared_reduction_under_traffic(M, N, K):
    # changing operands, launch grids, ranges cut in three, fused launches, and a sweep of the stencil on
    # another stream keeping HBM and the L2s busy: every result equals the witness of its operands
    rng = np.random.default_rng(M + N)
    ta.tzgemm_release_workspaces()
    pairs = [tuple(dev(x) for x in gemm_inputs(M, N, K, seed=50 + i)) for i in range(3)]
    witnesses = []
    for dA, dB in pairs:
        out = torch.zeros((M, N), device="cuda:0")
        ta.gptb_tzgemm(dA, dB, out)
        witnesses.append(out)
    torch.cuda.synchronize()
    A0 = dev(stencil_inputs(64, 256, 512, seed=2))
    A1 = A0.clone()
    side = torch.cuda.Stream(device="cuda:0")
    used = torch.zeros((M, N), device="cuda:0")
    tiles = (M // 64) * (N // 64)
    for it in range(48):
        i = int(rng.integers(0, 3))
        grid = int(rng.choice([0, 8, 40, 96, 256, 304]))
        dA, dB = pairs[i]
        if it % 3 == 0:
            ta.gptb_stencil(C0, C1, A0, A1, stream=side)
        if it % 4 == 1:
            t0 = int(rng.integers(0, tiles))
            t1 = int(rng.integers(t0, tiles + 1))
            used.fill_(0)
            ta.gptb_tzgemm(dA, dB, used, tile_start=0, tile_end=t0, launch_grid=grid)
            ta.gptb_tzgemm(dA, dB, used, tile_start=t1, tile_end=tiles, launch_grid=grid)
            ta.gptb_tzgemm(dA, dB, used, tile_start=t0, tile_end=t1, launch_grid=grid)
        elif it % 4 == 2:
            ta.mix_tzgemm_stencil(C0, C1, A0, A1, dA, dB, used, be_start=0, be_end=int(rng.integers(0, 256)))
        else:
            ta.gptb_tzgemm(dA, dB, used, launch_grid=grid)
        assert torch.equal(used.view(torch.int32), witnesses[i].view(torch.int32)), (it, i, grid)
    torch.cuda.synchronize()
    assert ta.spin_fail_flag() == 0


def test_tzgemm_shared_reductions_on_two_streams_do_not_meet():
    # each output buffer has a workspace of its own, so GEMMs of the same shape that run at the same
    # time on different streams cannot draw each other's tickets
    M, N, K = 256, 512, 4608
    inputs = [gemm_inputs(M, N, K, seed=70 + i) for i in range(2)]
    dev_in = [(dev(A), dev(B)) for A, B in inputs]
    want = []
    for dA, dB in dev_in:
        Cd = torch.zeros((M, N), device="cuda:0")
        ta.gptb_tzgemm(dA, dB, Cd)
        want.append(host(Cd).copy())
    assert not np.array_equal(want[0], want[1])
    streams = [torch.cuda.Stream(device="cuda:0") for _ in range(2)]
    outs = [torch.zeros((M, N), device="cuda:0") for _ in range(2)]
    torch.cuda.synchronize()
    for _ in range(20):
        for (dA, dB), Cd, st in zip(dev_in, outs, streams):
            ta.gptb_tzgemm(dA, dB, Cd, launch_grid=96, stream=st)
    torch.cuda.synchronize()
    for Cd, w in zip(outs, want):
        assert np.array_equal(host(Cd).view(np.uint32), w.view(np.uint32))


def test_tzgemm_on_the_global_operand_buffers():
    # OriTZGEMMKernel(id, m, n, k) of the reference works on process-wide buffers; here they grow with
    # the largest shape seen, and the workspace of the shared reductions is a fourth one beside A, B, C.
    # A shape without a workspace first, then two that need one (the second one larger): each result is
    # the GEMM of what the buffers hold, and equals the launch on caller-owned copies bit for bit.
    for (m, n, k) in [(256, 256, 128), (256, 512, 4608), (128, 4096, 4096)]:
        ori = ta.ori_tzgemm_create(None, None, None, m, n, k)
        g = ta.gptb_create(ori, 0, 0, 0, (m // 64) * (n // 64))
        for _ in range(2):
            g.execute()
        torch.cuda.synchronize()
        pa, pb, pc, sizes = ta.global_gemm_buffers()
        assert sizes[0] >= 2 * m * k and sizes[1] >= 2 * n * k and sizes[2] >= 4 * m * n
        A = ta.device_to_host(pa, (m, k), np.float16)
        B = ta.device_to_host(pb, (n, k), np.float16)
        got = ta.device_to_host(pc, (m, n), np.float32)
        ok, fro, dmax = gemm_tolerance_ok(got, oracle.tzgemm(A, B, f64=True), k)
        assert ok and fro <= 1e-5, (m, n, k, fro, dmax)
        own = torch.zeros((m, n), device="cuda:0")
        ta.gptb_tzgemm(dev(A), dev(B), own)
        assert np.array_equal(host(own).view(np.uint32), got.view(np.uint32))


def test_a_larger_workspace_replaces_the_bound_one_while_launches_are_queued():
    # an allocator hands an output address out again for another shape: the workspace bound to it is too
    # small, a larger one replaces it while launches on the old one are still queued (the old one stays
    # allocated until the workspaces are released), and both shapes keep giving their own bits
    ta.tzgemm_release_workspaces()
    buf = torch.zeros(128 * 8192, device="cuda:0")
    shapes = [(128, 128, 1024), (256, 512, 4608), (128, 8192, 1024)]
    assert [ta.tzgemm_workspace_bytes(*s_) for s_ in shapes] == sorted(ta.tzgemm_workspace_bytes(*s_) for s_ in shapes)
    ops, wants, kernels = [], [], []
    for i, (M, N, K) in enumerate(shapes):
        A, B = gemm_inputs(M, N, K, seed=60 + i)
        ops.append((dev(A), dev(B)))
        own = torch.zeros((M, N), device="cuda:0")
        ta.gptb_tzgemm(ops[-1][0], ops[-1][1], own)
        wants.append(host(own))
    torch.cuda.synchronize()
    for i, (M, N, K) in enumerate(shapes):
        Cv = buf[:M * N].view(M, N)
        assert Cv.data_ptr() == buf.data_ptr()
        ori = ta.ori_tzgemm_create(ops[i][0], ops[i][1], Cv)      # binds, or replaces, the workspace of this address
        g = ta.gptb_create(ori, 0, 0, 0, (M // 64) * (N // 64))
        kernels.append((ori, g))
        for _ in range(20):
            g.execute()                                            # left queued: no synchronisation before the next shape
    torch.cuda.synchronize()
    assert np.array_equal(host(buf[:128 * 8192].view(128, 8192)).view(np.uint32), wants[2].view(np.uint32))
    # the objects of the smaller shapes still work: they find the replacement through the table
    for i in (0, 1, 2, 0):
        M, N, K = shapes[i]
        kernels[i][1].execute()
        torch.cuda.synchronize()
        assert np.array_equal(host(buf[:M * N].view(M, N)).view(np.uint32), wants[i].view(np.uint32)), shapes[i]
    assert ta.spin_fail_flag() == 0
    ta.tzgemm_release_workspaces()


def test_tzgemm_shared_reduction_fused_equals_unfused():
    # conv5's shape with a best-effort kernel in the same launch: same bits as the GEMM alone
    M, N, K = 256, 512, 4608
    A, B = gemm_inputs(M, N, K, seed=41)
    dA, dB = dev(A), dev(B)
    solo = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dA, dB, solo)
    A0 = stencil_inputs(16, 64, 256, seed=9)
    a0 = dev(A0)
    want_s = oracle.stencil(C0, C1, A0, A0)
    for variant in ("wave_512", "wave_256", "wg_1_1"):
        for _ in range(2):
            mix_c = torch.full((M, N), -7.0, device="cuda:0")
            mix_s = a0.clone()
            ta.mix_tzgemm_stencil(C0, C1, a0, mix_s, dA, dB, mix_c, variant=variant)
            assert np.array_equal(host(mix_c).view(np.uint32), host(solo).view(np.uint32)), variant
            assert np.array_equal(host(mix_s), want_s)
    assert ta.spin_fail_flag() == 0


# ------------------------------------------------------------------ stencil
# widths that are multiples of 4 take the float4 (quad of blocks) form of the GPTB role, the
# others the one-block-per-wave form; 3 planes is the smallest grid with an interior
@pytest.mark.parametrize("shape", [(8, 8, 64), (6, 10, 70), (5, 7, 130), (4, 9, 33), (64, 64, 128),
                                   (12, 9, 260), (3, 5, 4), (11, 6, 516), (20, 13, 1028), (10, 4, 200)])
def test_stencil_ori_and_gptb_bit_exact(shape):
    A0 = stencil_inputs(*shape)
    want = oracle.stencil(C0, C1, A0, A0)
    a0 = dev(A0)
    out = a0.clone()
    ta.ori_stencil(C0, C1, a0, out)
    assert np.array_equal(host(out), want)
    out2 = a0.clone()
    ta.gptb_stencil(C0, C1, a0, out2)
    assert np.array_equal(host(out2), want)
    out3 = a0.clone()
    ta.gptb_stencil(C0, C1, a0, out3, launch_grid=3, launch_block=128)
    assert np.array_equal(host(out3), want)


def test_stencil_gptb_ranges_and_wrap():
    A0 = stencil_inputs(5, 12, 130)
    nblk = ta.stencil_blocks(130, 12)
    a0 = dev(A0)
    acc = torch.full_like(a0, -3.0)
    want = np.full_like(A0, -3.0)
    for s, e in [(0, 2), (2, 7), (7, nblk)]:
        ta.gptb_stencil(C0, C1, a0, acc, start=s, end=e, launch_grid=2, launch_block=64)
        want = oracle.stencil_gptb(C0, C1, A0, want, s, e)
        assert np.array_equal(host(acc), want)
    ta.gptb_stencil(C0, C1, a0, acc, start=nblk, end=2 * nblk)      # wraps: same cells again
    assert np.array_equal(host(acc), want)
    ta.gptb_stencil(C0, C1, a0, acc, start=4, end=4)                # empty range
    assert np.array_equal(host(acc), want)


@pytest.mark.parametrize("nx", [520, 200])
def test_stencil_wide_form_ranges_and_wrap(nx):
    # block rows are 9 (520) or 4 (200) blocks wide: quads of 4 blocks are ragged at the row
    # end, ranges start and end inside quads and inside either of the two runs of 8 centre
    # planes a block column of 13 planes has, and positions past the grid wrap onto it
    A0 = stencil_inputs(13, 10, nx)
    nblk = ta.stencil_blocks(nx, 10)
    npos = ta.stencil_blocks(nx, 10, 13)
    assert npos == 2 * nblk
    a0 = dev(A0)
    acc = torch.full_like(a0, -3.0)
    want = np.full_like(A0, -3.0)
    cuts = [0, 1, 3, 6, 11, 13, nblk - 2, nblk + 5, npos - 3, npos]
    for s, e in zip(cuts[:-1], cuts[1:]):
        if e <= s:
            continue
        ta.gptb_stencil(C0, C1, a0, acc, start=s, end=e, launch_grid=1, launch_block=128)   # 2 waves: the march
        want = oracle.stencil_gptb(C0, C1, A0, want, s, e, gdz="runs")
        assert np.array_equal(host(acc), want), (s, e)
    assert np.array_equal(want, oracle.stencil(C0, C1, A0, np.full_like(A0, -3.0)))
    acc2 = torch.full_like(a0, -3.0)
    ta.gptb_stencil(C0, C1, a0, acc2, start=npos + 2, end=2 * npos - 1, launch_grid=2)   # wraps onto 2 .. npos-2
    assert np.array_equal(host(acc2), oracle.stencil_gptb(C0, C1, A0, np.full_like(A0, -3.0), 2, npos - 1, gdz="runs"))


@pytest.mark.parametrize("shape", [(30, 20, 260), (27, 9, 130), (64, 24, 512)])
@pytest.mark.parametrize("grid", [1, 7, 256])
def test_stencil_any_tiling_of_the_position_grid_is_one_sweep(shape, grid):
    # positions = blocks x runs of 8 centre planes; few workgroups march quads of blocks plane by
    # plane, many (every wave at most two runs) issue all loads of a run at once: same bits
    nz, ny, nx = shape
    A0 = stencil_inputs(*shape, seed=nz + nx)
    npos = ta.stencil_blocks(nx, ny, nz)
    assert npos == ta.stencil_blocks(nx, ny) * -(-(nz - 2) // 8)
    want = oracle.stencil(C0, C1, A0, np.full_like(A0, -3.0))
    a0 = dev(A0)
    rng = np.random.default_rng(grid + nz)
    cuts = sorted(set([0, npos] + list(rng.integers(1, npos, 9))))
    acc = torch.full_like(a0, -3.0)
    ranges = list(zip(cuts[:-1], cuts[1:]))
    for i in rng.permutation(len(ranges)):            # in any order
        ta.gptb_stencil(C0, C1, a0, acc, start=int(ranges[i][0]), end=int(ranges[i][1]), launch_grid=grid)
    assert np.array_equal(host(acc), want)
    # one range alone writes exactly what the oracle's restatement of the position grid writes
    s, e = int(cuts[1]), int(cuts[3])
    one = torch.full_like(a0, -3.0)
    ta.gptb_stencil(C0, C1, a0, one, start=s, end=e, launch_grid=grid)
    assert np.array_equal(host(one), oracle.stencil_gptb(C0, C1, A0, np.full_like(A0, -3.0), s, e, gdz="runs"))


@pytest.mark.parametrize("ny,grid", [(256, 8), (256, 64), (128, 16), (192, 32)])
def test_stencil_slab_numbering_of_the_wide_form_is_one_sweep(ny, grid):
    # ranges long enough for the plane-by-plane march: with 64 or 32 quad rows the tasks are numbered by
    # XCD slabs (256 rows: for 4 and for 8 waves a workgroup; 128 rows: for 4 only), with 48 in the plain
    # order; any tiling by ranges, in any order, gives the bits of one sweep, alone and fused
    nz, nx = (66 if ny > 128 else 130), 512
    A0 = stencil_inputs(nz, ny, nx, seed=ny + grid)
    npos = ta.stencil_blocks(nx, ny, nz)
    assert npos == 8 * (ny // 4) * ((nz - 2) // 8) and npos > 2048
    want = oracle.stencil(C0, C1, A0, np.full_like(A0, -3.0))
    a0 = dev(A0)
    rng = np.random.default_rng(ny + grid)
    cuts = sorted(set([0, npos] + [int(c) for c in rng.integers(1, npos, 3)]))
    ranges = list(zip(cuts[:-1], cuts[1:]))
    acc = torch.full_like(a0, -3.0)
    for i in rng.permutation(len(ranges)):
        ta.gptb_stencil(C0, C1, a0, acc, start=ranges[i][0], end=ranges[i][1], launch_grid=grid)
    assert np.array_equal(host(acc), want)
    whole = torch.full_like(a0, -3.0)
    ta.gptb_stencil(C0, C1, a0, whole, launch_grid=grid)
    assert np.array_equal(host(whole), want)
    # the same ranges riding with a GEMM (8 best-effort waves a workgroup)
    gA, gB = gemm_inputs(256, 256, 256, 5)
    dA, dB = dev(gA), dev(gB)
    Cm = torch.zeros((256, 256), device="cuda:0")
    fused = torch.full_like(a0, -3.0)
    for i in rng.permutation(len(ranges)):
        ta.mix_tzgemm_stencil(C0, C1, a0, fused, dA, dB, Cm, be_start=ranges[i][0], be_end=ranges[i][1],
                              variant="wave_512", launch_grid=grid)
    assert np.array_equal(host(fused), want)
    assert ta.spin_fail_flag() == 0


def test_stencil_iterations_ping_pong():
    A0 = stencil_inputs(6, 16, 128)
    a, b = dev(A0), dev(A0)
    ha, hb = A0.copy(), A0.copy()
    for _ in range(5):
        ta.gptb_stencil(C0, C1, a, b)
        hb = oracle.stencil(C0, C1, ha, hb)
        a, b = b, a
        ha, hb = hb, ha
    assert np.array_equal(host(a), ha)


# ------------------------------------------------------------------ lbm
# even row lengths take the two-cells-per-lane form, odd ones one cell per lane; 300 is longer than one wave of pairs
@pytest.mark.parametrize("dims", [(4, 4, 4), (12, 5, 6), (64, 3, 5), (120, 6, 4), (128, 4, 4), (200, 3, 3),
                                  (7, 5, 4), (121, 4, 3), (2, 3, 5), (300, 3, 3), (1, 4, 4)])
def test_lbm_ori_and_gptb_bit_exact(dims):
    sx, sy, sz = dims
    src = lbm_inputs(sx, sy, sz, obstacle_p=0.2, accel_p=0.1)
    dst0 = np.full_like(src, -5.0)
    want = oracle.lbm(src, dst0, sx, sy, sz)
    s = dev(src)
    d = dev(dst0)
    ta.ori_lbm(s, d, sx, sy, sz)
    assert np.array_equal(host(d).view(np.uint32), want.view(np.uint32))
    d2 = dev(dst0)
    ta.gptb_lbm(s, d2, sx, sy, sz)
    assert np.array_equal(host(d2).view(np.uint32), want.view(np.uint32))
    d3 = dev(dst0)
    ta.gptb_lbm(s, d3, sx, sy, sz, launch_grid=2, launch_block=64)
    assert np.array_equal(host(d3).view(np.uint32), want.view(np.uint32))


def test_lbm_ranges():
    sx, sy, sz = 16, 4, 3
    src = lbm_inputs(sx, sy, sz)
    s = dev(src)
    d = torch.zeros_like(s)
    want = np.zeros_like(src)
    for a, b in [(0, 5), (5, 6), (6, 12)]:
        ta.gptb_lbm(s, d, sx, sy, sz, start=a, end=b)
        want = oracle.lbm(src, want, sx, sy, sz, a, b)
        assert np.array_equal(host(d), want)


# ------------------------------------------------------------------ mri-q
def mriq_close(got, truth):
    return np.all(np.abs(got.astype(np.float64) - truth) <= 1e-3 + 1e-4 * np.abs(truth))


@pytest.mark.parametrize("numK,numX", [(64, 256), (1024, 1024), (2048, 512), (3, 256)])
def test_mriq_matches_fp64_oracle(numK, numX):
    k, phiR, phiI, xyz = mriq_inputs(numK, numX)
    pm = torch.zeros(numK, device="cuda:0")
    ta.mriq_phimag(dev(phiR), dev(phiI), pm)
    phimag = host(pm)
    assert np.array_equal(phimag, oracle.mriq_phimag(phiR, phiI))
    kv = np.concatenate([k, phimag[:, None]], 1).astype(np.float32)
    ta.mriq_set_kvalues(kv)
    x, y, z = dev(xyz[0]), dev(xyz[1]), dev(xyz[2])
    q0 = np.full(numX, 0.5, np.float32)
    tr, ti = oracle.mriq(kv, xyz[0], xyz[1], xyz[2], q0, q0, f64=True)
    for form in ("ori", "gptb"):
        Qr, Qi = dev(q0), dev(q0)
        if form == "ori":
            ta.ori_mriq(numK, x, y, z, Qr, Qi)
        else:
            ta.gptb_mriq(numK, x, y, z, Qr, Qi, launch_grid=3)
        assert mriq_close(host(Qr), tr.astype(np.float64)) and mriq_close(host(Qi), ti.astype(np.float64))


def test_mriq_closed_forms_and_ranges():
    numK, numX = 128, 1024
    k, phiR, phiI, xyz = mriq_inputs(numK, numX, seed=2)
    kv = np.concatenate([k, oracle.mriq_phimag(phiR, phiI)[:, None]], 1).astype(np.float32)
    ta.mriq_set_kvalues(kv)
    zero = torch.zeros(numX, device="cuda:0")
    Qr, Qi = torch.zeros(numX, device="cuda:0"), torch.zeros(numX, device="cuda:0")
    ta.gptb_mriq(numK, zero, zero, zero, Qr, Qi)
    np.testing.assert_allclose(host(Qr), kv[:, 3].astype(np.float64).sum(), rtol=1e-5)
    assert np.all(host(Qi) == 0)
    x, y, z = dev(xyz[0]), dev(xyz[1]), dev(xyz[2])
    full_r = torch.zeros(numX, device="cuda:0")
    full_i = torch.zeros(numX, device="cuda:0")
    ta.gptb_mriq(numK, x, y, z, full_r, full_i)
    pr, pi = torch.zeros(numX, device="cuda:0"), torch.zeros(numX, device="cuda:0")
    ta.gptb_mriq(numK, x, y, z, pr, pi, start=1, end=3)
    pr, fr = host(pr), host(full_r)
    assert np.array_equal(pr[256:768], fr[256:768]) and np.all(pr[:256] == 0) and np.all(pr[768:] == 0)


def test_mriq_block_positions_are_voxel_blocks_by_k_chunks():
    # numK 300 -> chunks of 128, 128 and 44 records; 4 voxel blocks -> 12 block positions
    numK, numX = 300, 1024
    k, phiR, phiI, xyz = mriq_inputs(numK, numX, seed=5)
    kv = np.concatenate([k, oracle.mriq_phimag(phiR, phiI)[:, None]], 1).astype(np.float32)
    ta.mriq_set_kvalues(kv)
    assert ta.mriq_blocks(numK, numX) == 12 and ta.mriq_blocks(0, numX) == 4 and ta.mriq_blocks(128, numX) == 4
    x, y, z = dev(xyz[0]), dev(xyz[1]), dev(xyz[2])
    q0 = np.linspace(-1, 1, numX).astype(np.float32)

    def run(ranges, **kw):
        Qr, Qi = dev(q0), dev(q0)
        for a, b in ranges:
            ta.gptb_mriq(numK, x, y, z, Qr, Qi, start=a, end=b, **kw)
        return host(Qr), host(Qi)

    Qr, Qi = dev(q0), dev(q0)
    ta.ori_mriq(numK, x, y, z, Qr, Qi)
    ori = host(Qr), host(Qi)
    # the whole grid in one launch, for several launch shapes (3 workgroups: owners hold two
    # voxel blocks; 7: more workgroups than voxel blocks), equals the natural kernel bit for bit
    for kw in ({}, {"launch_grid": 3}, {"launch_grid": 7}, {"launch_grid": 1}):
        got = run([(0, 12)], **kw)
        assert np.array_equal(got[0], ori[0]) and np.array_equal(got[1], ori[1]), kw
    # so does any tiling of it by ascending ranges: inside a row, across a row end, whole rows
    for tiling in ([(0, 3), (3, 5), (5, 11), (11, 12)], [(0, 4), (4, 8), (8, 12)], [(0, 1), (1, 12)],
                   [(0, 6), (6, 12)], [(i, i + 1) for i in range(12)]):
        got = run(tiling, launch_grid=3)
        assert np.array_equal(got[0], ori[0]) and np.array_equal(got[1], ori[1]), tiling
    # partial ranges against the oracle's restatement of the position grid (float64 truth)
    for a, b in ((5, 7), (2, 11), (11, 12), (3, 4), (7, 17)):
        got = run([(a, b)], launch_grid=3)
        tr, ti = oracle.mriq(kv, xyz[0], xyz[1], xyz[2], q0, q0, start=a, end=b, kchunk=128, f64=True)
        assert mriq_close(got[0], tr.astype(np.float64)) and mriq_close(got[1], ti.astype(np.float64)), (a, b)
        same = tr == q0                                     # voxels the range does not touch
        assert np.array_equal(got[0][same], q0[same]) and np.array_equal(got[1][same], q0[same]), (a, b)
    # positions 5 and 6 alone: chunk 1 (records 128..255) onto voxel blocks 1 and 2
    got = run([(5, 7)])
    sel = slice(256, 768)
    tr, ti = oracle.mriq(kv[128:256], xyz[0][sel], xyz[1][sel], xyz[2][sel], q0[sel], q0[sel], f64=True)
    assert mriq_close(got[0][sel], tr.astype(np.float64)) and mriq_close(got[1][sel], ti.astype(np.float64))
    assert np.array_equal(got[0][:256], q0[:256]) and np.array_equal(got[0][768:], q0[768:])
    assert np.array_equal(got[1][:256], q0[:256]) and np.array_equal(got[1][768:], q0[768:])
    # positions past the grid wrap as the reference's index arithmetic does (block p % x, chunk
    # (p / x) % y): [0, 24) adds every chunk twice, [10, 14) = last chunk of blocks 2,3 then first of 0,1
    twice = run([(0, 24)], launch_grid=3)
    again = run([(0, 12), (0, 12)], launch_grid=5)
    assert np.array_equal(twice[0], again[0]) and np.array_equal(twice[1], again[1])
    wrap = run([(10, 14)])
    split = run([(10, 12), (0, 2)])
    assert np.array_equal(wrap[0], split[0]) and np.array_equal(wrap[1], split[1])


# ------------------------------------------------------------------ cp
def cp_atoms():
    atoms = ta.cp_initatoms(4000)
    assert np.array_equal(atoms, oracle.cp_initatoms(4000))
    return atoms[1:65]


@pytest.mark.parametrize("shape", [(8, 128), (24, 384), (64, 1024)])
def test_cp_bit_exact(shape):
    atoms = cp_atoms()
    ta.cp_set_atoms(atoms, 0.0)
    info = oracle.cp_atoms_to_const(atoms, 0.0)
    rng = np.random.default_rng(4)
    g0 = rng.uniform(-1, 1, shape).astype(np.float32)
    want = oracle.cp(info, g0)
    g = dev(g0)
    ta.ori_cp(64, 0.1, g)
    assert np.array_equal(host(g).view(np.uint32), want.view(np.uint32))
    g2 = dev(g0)
    ta.gptb_cp(64, 0.1, g2, launch_grid=5)
    assert np.array_equal(host(g2).view(np.uint32), want.view(np.uint32))
    g3 = dev(g0)
    nblk = ta.cp_blocks(shape[1], shape[0])
    assert nblk == (shape[1] // 128) * (shape[0] // 8) * 4
    want3 = g0
    for s, e in [(0, 1), (1, nblk)]:
        ta.gptb_cp(64, 0.1, g3, start=s, end=e, launch_block=256)
        want3 = oracle.cp(info, want3, start=s, end=e, parts=4)
    assert np.array_equal(host(g3).view(np.uint32), want3.view(np.uint32))
    assert np.array_equal(want3, want)


def test_cp_block_positions_are_blocks_by_x_parts():
    atoms = cp_atoms()
    ta.cp_set_atoms(atoms, 0.0)
    info = oracle.cp_atoms_to_const(atoms, 0.0)
    H, Wd = 24, 384                                    # 3 x 3 blocks x 4 parts = 36 positions
    g0 = np.random.default_rng(9).uniform(-1, 1, (H, Wd)).astype(np.float32)
    whole = oracle.cp(info, g0)
    assert ta.cp_blocks(Wd, H) == 36

    def run(ranges, **kw):
        g = dev(g0)
        for a, b in ranges:
            ta.gptb_cp(64, 0.1, g, start=a, end=b, **kw)
        return host(g)

    same = lambda a, b: np.array_equal(a.view(np.uint32), b.view(np.uint32))
    for kw in ({}, {"launch_grid": 1}, {"launch_grid": 2, "launch_block": 256}, {"launch_grid": 5}, {"launch_grid": 40}):
        assert same(run([(0, 36)], **kw), whole), kw
    for tiling in ([(0, 5), (5, 11), (11, 30), (30, 36)], [(0, 9), (9, 18), (18, 27), (27, 36)],
                   [(i, i + 1) for i in range(36)], [(20, 36), (0, 20)], [(0, 10), (10, 36)]):
        assert same(run(tiling, launch_grid=2), whole), tiling
    # partial ranges against the oracle's restatement of the position grid, bit for bit
    for a, b in ((5, 7), (3, 31), (35, 36), (9, 18), (8, 28), (17, 19)):
        for kw in ({"launch_grid": 2}, {}):
            assert same(run([(a, b)], **kw), oracle.cp(info, g0, start=a, end=b, parts=4)), (a, b, kw)
    # past the grid the positions come round again: every point gets its sum a second time, after the first
    assert same(run([(0, 72)], launch_grid=2), oracle.cp(info, whole))
    assert same(run([(30, 42)], launch_grid=3), oracle.cp(info, g0, start=30, end=42, parts=4))


def test_cp_short_inverse_square_root_is_the_ieee_one_on_its_whole_range():
    # every float in [2^-20, 2^20): 335 544 320 values, each compared bitwise with 1.0f / sqrtf(x)
    assert ta.cp_inv_sqrt_selftest() == 0
    # the check itself can fail: just below the range the short form is not exact everywhere
    assert ta.cp_inv_sqrt_selftest(0x00800000, 0x35800000) > 0


def test_cp_points_on_and_next_to_atoms_take_the_general_path():
    # atoms exactly on grid points (r2 = 0 -> inf, as IEEE says), within 2^-10 of a grid row, and far away:
    # the wave-level range guard must send the close ones through sqrtf / divide
    atoms = np.array([[1.6, 0.8, 0.0, 1.0],        # on the point (16, 8)
                      [3.2005, 1.6003, 0.0, -0.5], # dy = 0.0003 from row 16: dyz2 below 2^-20
                      [7.3, 2.29, 0.0, 0.25],
                      [0.0, 0.0, 0.0, 2.0]], np.float32)
    ta.cp_set_atoms(atoms, 0.0)
    info = oracle.cp_atoms_to_const(atoms, 0.0)
    g0 = np.zeros((32, 256), np.float32)
    want = oracle.cp(info, g0)
    assert np.isinf(want).sum() >= 1
    for kw in ({}, {"launch_grid": 3}):
        g = dev(g0)
        ta.gptb_cp(4, 0.1, g, **kw)
        assert np.array_equal(host(g).view(np.uint32), want.view(np.uint32))
    g = dev(g0)
    ta.ori_cp(4, 0.1, g)
    assert np.array_equal(host(g).view(np.uint32), want.view(np.uint32))
    g = dev(g0)
    for a, b in ((0, 5), (5, 23), (23, ta.cp_blocks(256, 32))):
        ta.gptb_cp(4, 0.1, g, start=a, end=b)
    assert np.array_equal(host(g).view(np.uint32), want.view(np.uint32))


def test_cp_fewer_atoms():
    atoms = cp_atoms()[:7]
    ta.cp_set_atoms(atoms, 0.5)
    info = oracle.cp_atoms_to_const(atoms, 0.5)
    g = torch.zeros((16, 256), device="cuda:0")
    ta.gptb_cp(7, 0.1, g)
    assert np.array_equal(host(g), oracle.cp(info, np.zeros((16, 256), np.float32)))


# ------------------------------------------------------------------ fused
VARIANTS = [None, "wave_256", "wave_512", "wg_1_1", "wg_1_2"]


@pytest.mark.parametrize("variant", VARIANTS)
def test_mix_tzgemm_stencil(variant):
    M, N, K = 256, 384, 256
    A, B = gemm_inputs(M, N, K, seed=7)
    A0 = stencil_inputs(6, 20, 200)
    a0 = dev(A0)
    solo_c = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dev(A), dev(B), solo_c)
    solo_s = a0.clone()
    ta.gptb_stencil(C0, C1, a0, solo_s)
    mix_c = torch.full((M, N), -7.0, device="cuda:0")
    mix_s = a0.clone()
    ta.mix_tzgemm_stencil(C0, C1, a0, mix_s, dev(A), dev(B), mix_c, variant=variant)
    assert np.array_equal(host(mix_c), host(solo_c))             # fused == unfused, bit-exact
    assert np.array_equal(host(mix_s), host(solo_s))
    assert np.array_equal(host(mix_s), oracle.stencil(C0, C1, A0, A0))
    ok, fro, _ = gemm_tolerance_ok(host(mix_c), oracle.tzgemm(A, B, f64=True), K)
    assert ok and fro <= 1e-5
    assert ta.spin_fail_flag() == 0          # no role-local barrier gave up waiting


def test_mix_tzgemm_stencil_partial_ranges():
    M, N, K = 256, 256, 128
    A, B = gemm_inputs(M, N, K, seed=8)
    A0 = stencil_inputs(5, 12, 130)
    a0 = dev(A0)
    mix_c = torch.full((M, N), -7.0, device="cuda:0")
    mix_s = torch.full_like(a0, -3.0)
    ta.mix_tzgemm_stencil(C0, C1, a0, mix_s, dev(A), dev(B), mix_c, be_start=2, be_end=7, tile_start=3, tile_end=11)
    assert np.array_equal(host(mix_s), oracle.stencil_gptb(C0, C1, A0, np.full_like(A0, -3.0), 2, 7))
    want_c = oracle.tzgemm(A, B, C_init=np.full((M, N), -7.0, np.float32), start=3, end=11)
    got_c = host(mix_c)
    assert np.array_equal(got_c == -7.0, want_c == -7.0)
    ta.mix_tzgemm_stencil(C0, C1, a0, mix_s, dev(A), dev(B), mix_c, be_start=0, be_end=0, tile_start=0, tile_end=0)
    assert np.array_equal(host(mix_c), got_c)


@pytest.mark.parametrize("variant", VARIANTS)
def test_mix_tzgemm_lbm(variant):
    M, N, K = 256, 256, 256
    A, B = gemm_inputs(M, N, K, seed=9)
    sx, sy, sz = 120, 6, 5
    src = lbm_inputs(sx, sy, sz)
    s = dev(src)
    solo_c = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dev(A), dev(B), solo_c)
    mix_c = torch.zeros((M, N), device="cuda:0")
    d = torch.zeros_like(s)
    ta.mix_tzgemm_lbm(s, d, sx, sy, sz, dev(A), dev(B), mix_c, variant=variant)
    assert np.array_equal(host(mix_c), host(solo_c))
    want = oracle.lbm(src, np.zeros_like(src), sx, sy, sz)
    assert np.array_equal(host(d).view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("variant", VARIANTS)
def test_mix_tzgemm_mriq(variant):
    M, N, K = 256, 256, 256
    A, B = gemm_inputs(M, N, K, seed=10)
    numK, numX = 256, 2048
    k, phiR, phiI, xyz = mriq_inputs(numK, numX)
    kv = np.concatenate([k, oracle.mriq_phimag(phiR, phiI)[:, None]], 1).astype(np.float32)
    ta.mriq_set_kvalues(kv)
    x, y, z = dev(xyz[0]), dev(xyz[1]), dev(xyz[2])
    solo_r, solo_i = torch.zeros(numX, device="cuda:0"), torch.zeros(numX, device="cuda:0")
    ta.gptb_mriq(numK, x, y, z, solo_r, solo_i)
    solo_c = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dev(A), dev(B), solo_c)
    mix_c = torch.zeros((M, N), device="cuda:0")
    Qr, Qi = torch.zeros(numX, device="cuda:0"), torch.zeros(numX, device="cuda:0")
    ta.mix_tzgemm_mriq(numK, x, y, z, Qr, Qi, dev(A), dev(B), mix_c, variant=variant)
    assert np.array_equal(host(mix_c), host(solo_c))
    assert np.array_equal(host(Qr), host(solo_r)) and np.array_equal(host(Qi), host(solo_i))
    zq = np.zeros(numX, np.float32)
    tr, ti = oracle.mriq(kv, xyz[0], xyz[1], xyz[2], zq, zq, f64=True)
    assert mriq_close(host(Qr), tr.astype(np.float64)) and mriq_close(host(Qi), ti.astype(np.float64))


@pytest.mark.parametrize("variant", VARIANTS)
def test_mix_tzgemm_cp(variant):
    M, N, K = 256, 256, 256
    A, B = gemm_inputs(M, N, K, seed=11)
    atoms = cp_atoms()
    ta.cp_set_atoms(atoms, 0.0)
    info = oracle.cp_atoms_to_const(atoms, 0.0)
    solo_c = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dev(A), dev(B), solo_c)
    mix_c = torch.zeros((M, N), device="cuda:0")
    g = torch.zeros((32, 512), device="cuda:0")
    ta.mix_tzgemm_cp(64, 0.1, g, dev(A), dev(B), mix_c, variant=variant)
    assert np.array_equal(host(mix_c), host(solo_c))
    assert np.array_equal(host(g).view(np.uint32), oracle.cp(info, np.zeros((32, 512), np.float32)).view(np.uint32))


# ------------------------------------------------------------------ randomised ranges of the position grids
@pytest.mark.parametrize("seed", range(12))
def test_mriq_random_position_ranges_and_launch_shapes(seed):
    rng = np.random.default_rng(1000 + seed)
    numK = int(rng.integers(1, 420))
    numX = int(rng.choice([256, 512, 1024, 1536]))
    k, phiR, phiI, xyz = mriq_inputs(numK, numX, seed=seed)
    kv = np.concatenate([k, oracle.mriq_phimag(phiR, phiI)[:, None]], 1).astype(np.float32)
    ta.mriq_set_kvalues(kv)
    x, y, z = dev(xyz[0]), dev(xyz[1]), dev(xyz[2])
    total = ta.mriq_blocks(numK, numX)
    q0 = rng.uniform(-1, 1, numX).astype(np.float32)
    a = int(rng.integers(0, total + 1))
    b = int(rng.integers(a, 2 * total + 1))                       # may run past the grid and wrap
    mid = int(rng.integers(a, b + 1))
    grid = int(rng.choice([1, 2, 3, 5, 8, 40, 0]))
    Qr, Qi = dev(q0), dev(q0)
    ta.gptb_mriq(numK, x, y, z, Qr, Qi, start=a, end=b, launch_grid=grid)
    tr, ti = oracle.mriq(kv, xyz[0], xyz[1], xyz[2], q0, q0, start=a, end=b, kchunk=128, f64=True)
    tol = lambda got, want: np.all(np.abs(got.astype(np.float64) - want) <= 2e-3 + 2e-4 * np.abs(want))
    assert tol(host(Qr), tr.astype(np.float64)) and tol(host(Qi), ti.astype(np.float64)), (numK, numX, a, b, grid)
    # the same range cut in two, with another launch shape: the same bits
    Pr, Pi = dev(q0), dev(q0)
    other = int(rng.choice([1, 3, 7, 16, 0]))
    ta.gptb_mriq(numK, x, y, z, Pr, Pi, start=a, end=mid, launch_grid=other)
    ta.gptb_mriq(numK, x, y, z, Pr, Pi, start=mid, end=b, launch_grid=grid)
    assert np.array_equal(host(Pr), host(Qr)) and np.array_equal(host(Pi), host(Qi)), (numK, numX, a, mid, b, grid, other)


@pytest.mark.parametrize("seed", range(12))
def test_cp_random_position_ranges_and_launch_shapes(seed):
    rng = np.random.default_rng(2000 + seed)
    H, Wd = [(8, 128), (16, 256), (24, 384), (40, 128), (8, 640)][int(rng.integers(0, 5))]
    natoms = int(rng.integers(1, 65))
    atoms = cp_atoms()[:natoms].copy()
    atoms[:, :2] *= np.float32(0.1)                               # bring some atoms into the small volume
    zplane = float(rng.choice([0.0, 0.3]))
    ta.cp_set_atoms(atoms, zplane)
    info = oracle.cp_atoms_to_const(atoms, zplane)
    g0 = rng.uniform(-1, 1, (H, Wd)).astype(np.float32)
    total = ta.cp_blocks(Wd, H)
    a = int(rng.integers(0, total + 1))
    b = int(rng.integers(a, 2 * total + 1))
    grid = int(rng.choice([1, 2, 3, 5, 8, 40, 0]))
    block = int(rng.choice([128, 256]))
    g = dev(g0)
    ta.gptb_cp(natoms, 0.1, g, start=a, end=b, launch_grid=grid, launch_block=block)
    want = oracle.cp(info, g0, start=a, end=b, parts=4)
    assert np.array_equal(host(g).view(np.uint32), want.view(np.uint32)), (H, Wd, natoms, a, b, grid, block)


# ------------------------------------------------------------------ best-effort x best-effort pairs
def _small_be(name):
    """(ori kernel, blocks, output tensors, snapshot of the outputs before any launch)"""
    if name == "stencil":
        A0 = stencil_inputs(6, 20, 200, seed=31)
        a0 = dev(A0)
        out = a0.clone()
        return ta.ori_stencil_create(C0, C1, a0, out), ta.stencil_blocks(200, 20), [out]
    if name == "lbm":
        src = dev(lbm_inputs(120, 6, 5, seed=32))
        dst = torch.zeros_like(src)
        return ta.ori_lbm_create(src, dst, 120, 6, 5), 30, [dst]
    if name == "mriq":
        k, phiR, phiI, xyz = mriq_inputs(256, 2048, seed=33)
        kv = np.concatenate([k, oracle.mriq_phimag(phiR, phiI)[:, None]], 1).astype(np.float32)
        ta.mriq_set_kvalues(kv)
        Qr, Qi = torch.zeros(2048, device="cuda:0"), torch.zeros(2048, device="cuda:0")
        return (ta.ori_mriq_create(256, dev(xyz[0]), dev(xyz[1]), dev(xyz[2]), Qr, Qi), ta.mriq_blocks(256, 2048),
                [Qr, Qi])
    if name == "mrif":
        k, phi, d, xyz = mrif_inputs(256, 2048, seed=34)
        ta.mrif_set_kvalues(mrif_table(k, phi, d))
        outR, outI = torch.zeros(2048, device="cuda:0"), torch.zeros(2048, device="cuda:0")
        return (ta.ori_mrif_create(256, dev(xyz[0]), dev(xyz[1]), dev(xyz[2]), outR, outI), ta.mrif_blocks(256, 2048),
                [outR, outI])
    if name == "sgemm":
        sA, sB, sC0 = sgemm_inputs()
        sC = dev(sC0)
        return ta.ori_sgemm_create(dev(sA), dev(sB), sC), ta.sgemm_blocks(256, 48, 700), [sC]
    if name == "fft":
        data = dev(fft_inputs())
        return ta.ori_fft_create(data), data.shape[0], [data]
    if name == "cutcp":
        inp = ta.CutcpInput(cutcp_atoms(), (0, 0, 0), 24, 16, 16, 0.5, 12.0)
        return ta.ori_cutcp_create(inp, 144.0, 0.006944), inp.blocks(), [inp.energies]
    ta.cp_set_atoms(cp_atoms(), 0.0)
    g = torch.zeros((32, 512), device="cuda:0")
    return ta.ori_cp_create(64, 0.1, g), ta.cp_blocks(512, 32), [g]


def cutcp_atoms():
    rng = np.random.default_rng(37)
    a = np.empty((300, 4), np.float32)
    a[:, :3] = rng.uniform(0, 7.5, (300, 3))
    a[:, 3] = rng.uniform(0.1, 1, 300) * rng.choice([-1, 1], 300)
    return a


def fft_inputs():
    return np.random.default_rng(36).uniform(-1, 1, (50, 256, 2)).astype(np.float32)


def fft_close(got, want):
    """|d| <= 1e-4 + 1e-5 |ref|: eight stages of fp32 butterflies on inputs in [-1, 1] (sums up to ~40) with
    twiddles that differ from the C library's in the last place"""
    return bool(np.all(np.abs(got.astype(np.float64) - want) <= 1e-4 + 1e-5 * np.abs(want)))


def sgemm_inputs():
    rng = np.random.default_rng(35)
    return (rng.uniform(0, 1, (700, 256)).astype(np.float32), rng.uniform(0, 1, (700, 48)).astype(np.float32),
            rng.uniform(-1, 1, (48, 256)).astype(np.float32))


BE_PAIRS = [("cp", "lbm"), ("cp", "mriq"), ("cp", "stencil"), ("lbm", "mriq"), ("lbm", "stencil"), ("mriq", "stencil"),
            ("cp", "mrif"), ("lbm", "mrif"), ("mrif", "mriq"), ("mrif", "stencil"), ("cp", "sgemm"), ("lbm", "sgemm"),
            ("mrif", "sgemm"), ("mriq", "sgemm"), ("sgemm", "stencil"), ("cp", "fft"), ("fft", "lbm"), ("fft", "mrif"),
            ("fft", "mriq"), ("fft", "sgemm"), ("fft", "stencil"), ("cp", "cutcp"), ("cutcp", "fft"), ("cutcp", "lbm"),
            ("cutcp", "mrif"), ("cutcp", "mriq"), ("cutcp", "sgemm"), ("cutcp", "stencil")]


@pytest.mark.parametrize("first,second", BE_PAIRS)
@pytest.mark.parametrize("variant", [None, "wg_1_2", "wg_2_1", "ord_1_1", "ord_1_2"])
def test_best_effort_pairs_fused_equals_unfused(first, second, variant):
    ori1, n1, outs1 = _small_be(first)
    ori2, n2, outs2 = _small_be(second)
    outs = outs1 + outs2
    before = [o.clone() for o in outs]
    r1 = (1, n1 - 1) if n1 > 2 else (0, n1)          # a partial range of the first kernel
    if first == "sgemm":
        r1 = (0, n1 - 1)    # its later k parts continue from the workspace, which only part 0 resets: start there
    g1 = ta.gptb_create(ori1, 0, 0, r1[0], r1[1])
    g2 = ta.gptb_create(ori2, 0, 0, 0, n2)
    g1.execute()
    g2.execute()
    want = [host(o).copy() for o in outs]
    for o, b in zip(outs, before):
        o.copy_(b)
    mix = ta.be_pair_create(ta.gptb_create(ori1, 0, 0, 0, n1), g2, r1[0], r1[1], 0, n2, variant=variant, launch_grid=48)
    mix.execute()
    for o, w in zip(outs, want):
        assert np.array_equal(host(o).view(np.uint32), w.view(np.uint32))


def _small_be_matches_oracle(name, outs):
    """the outputs of _small_be(name) after one full pass, against the oracle on the same seeded inputs:
    bit-exact for stencil, lbm, cp and sgemm, the float tolerances for the two MRI kernels and the FFT"""
    if name == "stencil":
        A0 = stencil_inputs(6, 20, 200, seed=31)
        return np.array_equal(host(outs[0]).view(np.uint32), oracle.stencil(C0, C1, A0, A0).view(np.uint32))
    if name == "lbm":
        src = lbm_inputs(120, 6, 5, seed=32)
        want = oracle.lbm(src, np.zeros_like(src), 120, 6, 5)
        return np.array_equal(host(outs[0]).view(np.uint32), want.view(np.uint32))
    zq = np.zeros(2048, np.float32)
    if name == "mriq":
        k, phiR, phiI, xyz = mriq_inputs(256, 2048, seed=33)
        kv = np.concatenate([k, oracle.mriq_phimag(phiR, phiI)[:, None]], 1).astype(np.float32)
        tr, ti = oracle.mriq(kv, xyz[0], xyz[1], xyz[2], zq, zq, f64=True)
        return mriq_close(host(outs[0]), tr.astype(np.float64)) and mriq_close(host(outs[1]), ti.astype(np.float64))
    if name == "mrif":
        k, phi, d, xyz = mrif_inputs(256, 2048, seed=34)
        tr, ti = oracle.mrif(mrif_table(k, phi, d), xyz[0], xyz[1], xyz[2], zq, zq, f64=True)
        return mriq_close(host(outs[0]), tr.astype(np.float64)) and mriq_close(host(outs[1]), ti.astype(np.float64))
    if name == "sgemm":
        return np.array_equal(host(outs[0]).view(np.uint32), oracle.sgemm(*sgemm_inputs()).view(np.uint32))
    if name == "fft":
        return fft_close(host(outs[0]), oracle.fft(fft_inputs()).astype(np.float64))
    if name == "cutcp":
        prep = oracle.cutcp_prepare(cutcp_atoms(), (0, 0, 0), 24, 16, 16, 0.5, 12.0)
        want = oracle.cutcp(prep, 0.5, 144.0, 0.006944, (3, 2, 2)).astype(np.float64)
        return bool(np.all(np.abs(host(outs[0]) - want) <= 2e-4 + 2e-5 * np.abs(want)))
    want = oracle.cp(oracle.cp_atoms_to_const(cp_atoms(), 0.0), np.zeros((32, 512), np.float32))
    return np.array_equal(host(outs[0]).view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("first,second", BE_PAIRS)
def test_best_effort_pairs_full_ranges_match_the_oracle(first, second):
    ori1, n1, outs1 = _small_be(first)
    ori2, n2, outs2 = _small_be(second)
    g1, g2 = ta.gptb_create(ori1, 0, 0, 0, n1), ta.gptb_create(ori2, 0, 0, 0, n2)
    ta.be_pair_create(g1, g2, 0, n1, 0, n2, launch_grid=48).execute()
    assert _small_be_matches_oracle(first, outs1), first
    assert _small_be_matches_oracle(second, outs2), second
    assert ta.spin_fail_flag() == 0


@pytest.mark.parametrize("variant", VARIANTS)
def test_mix_with_a_k_split_gemm_shape(variant):
    # 256 x 384 x 1024: 6 macro tiles, K >= 512 -> the GEMM role takes its K-split form,
    # whose workgroup-level reduction runs on the role barrier of the fused kernel
    M, N, K = 256, 384, 1024
    A, B = gemm_inputs(M, N, K, seed=17)
    A0 = stencil_inputs(6, 20, 200, seed=5)
    a0 = dev(A0)
    solo_c = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dev(A), dev(B), solo_c)
    mix_c = torch.full((M, N), -7.0, device="cuda:0")
    mix_s = a0.clone()
    ta.mix_tzgemm_stencil(C0, C1, a0, mix_s, dev(A), dev(B), mix_c, variant=variant, tile_start=2, tile_end=19)
    got = host(mix_c)
    full = host(solo_c)
    want = oracle.tzgemm(A, B, C_init=np.full((M, N), -7.0, np.float32), start=2, end=19)
    mask = want != -7.0
    assert np.array_equal(got[~mask], want[~mask]) and np.array_equal(got[mask], full[mask])
    ok, fro, dmax = gemm_tolerance_ok(full, oracle.tzgemm(A, B, f64=True), K)
    assert ok and fro <= 1e-5, (fro, dmax)
    assert np.array_equal(host(mix_s), oracle.stencil(C0, C1, A0, A0))
    assert ta.spin_fail_flag() == 0


@pytest.mark.parametrize("seed", range(16))
def test_random_fused_launches_equal_the_two_kernels_alone(seed):
    # random GEMM shape (both forms of the role), tile range, best-effort kernel, block range (may wrap),
    # variant and launch grid: the fused launch must leave exactly what the two GPTB kernels leave
    rng = np.random.default_rng(3000 + seed)
    name = ["stencil", "lbm", "mriq", "cp"][seed % 4]
    M, N, K = [(256, 384, 256), (256, 384, 1024), (128, 128, 640), (384, 256, 128), (512, 128, 2048)][int(rng.integers(0, 5))]
    A, B = gemm_inputs(M, N, K, seed=seed)
    dA, dB = dev(A), dev(B)
    tiles = (M // 64) * (N // 64)
    t0 = int(rng.integers(0, tiles))
    t1 = int(rng.integers(t0, tiles + 1))
    ori, nblk, outs = _small_be(name)
    wrap_ok = name in ("mriq", "cp")                     # accumulating kernels: a second pass adds again, in order
    b0 = int(rng.integers(0, nblk))
    b1 = int(rng.integers(b0, (2 * nblk if wrap_ok else nblk) + 1))
    variant = [None, "wave_256", "wave_512", "wg_1_1", "wg_1_2"][int(rng.integers(0, 5))]
    before = [o.clone() for o in outs]
    solo_c = torch.full((M, N), -3.0, device="cuda:0")
    tz_ori = ta.ori_tzgemm_create(dA, dB, solo_c)
    ta.gptb_create(ori, 0, 0, b0, b1).execute()
    ta.gptb_create(tz_ori, 0, 0, t0, t1).execute()
    want = [host(o).copy() for o in outs] + [host(solo_c).copy()]
    for o, keep in zip(outs, before):
        o.copy_(keep)
    solo_c.fill_(-3.0)
    be_full = ta.gptb_create(ori, 0, 0, 0, nblk)
    tz_full = ta.gptb_create(tz_ori, 0, 0, 0, tiles)
    ta.mix_create(be_full, tz_full, b0, b1, t0, t1, variant=variant).execute()
    got = [host(o) for o in outs] + [host(solo_c)]
    for g, w in zip(got, want):
        assert np.array_equal(g.view(np.uint32), w.view(np.uint32)), (name, (M, N, K), (t0, t1), (b0, b1), variant)
    assert ta.spin_fail_flag() == 0


@pytest.mark.parametrize("variant", ["wave_256", "wave_512"])
def test_gemm_role_barrier_hands_over_to_the_hardware_barrier_at_any_point(variant):
    # In a wave-split kernel the GEMM role synchronises on an LDS arrival counter while best-effort waves run
    # and on the hardware barrier once they have ended.  The change-over falls wherever the best-effort
    # work happens to end: before the first tile (no blocks), in the middle of a tile, between tiles of a
    # workgroup that has several (few workgroups launched), inside a shared reduction, or never (best-effort
    # work that outlasts the GEMM).  Whatever the point, the GEMM's bits are those of the kernel alone.
    for (M, N, K), grid in [((512, 512, 2048), 4), ((512, 512, 2048), 0), ((256, 384, 1024), 0), ((128, 128, 4608), 0)]:
        A, B = gemm_inputs(M, N, K, seed=M + K)
        dA, dB = dev(A), dev(B)
        tiles = (M // 64) * (N // 64)
        solo = torch.zeros((M, N), device="cuda:0")
        ta.gptb_tzgemm(dA, dB, solo)
        want_c = host(solo).view(np.uint32)
        numK, numX = 512, 8192
        k, phiR, phiI, xyz = mriq_inputs(numK, numX, seed=44)
        ta.mriq_set_kvalues(np.concatenate([k, oracle.mriq_phimag(phiR, phiI)[:, None]], 1).astype(np.float32))
        dx, dy, dz = (dev(v) for v in xyz)
        nblk = ta.mriq_blocks(numK, numX)
        ref_q = [torch.zeros(numX, device="cuda:0") for _ in range(2)]
        ta.gptb_mriq(numK, dx, dy, dz, ref_q[0], ref_q[1])
        for blocks in (0, 1, 3, nblk // 8, nblk // 2, nblk):
            c = torch.full((M, N), -9.0, device="cuda:0")
            q = [torch.zeros(numX, device="cuda:0") for _ in range(2)]
            ta.mix_tzgemm_mriq(numK, dx, dy, dz, q[0], q[1], dA, dB, c, be_end=blocks, variant=variant, launch_grid=grid)
            assert np.array_equal(host(c).view(np.uint32), want_c), ((M, N, K), grid, blocks)
            if blocks == nblk:
                assert np.array_equal(host(q[0]).view(np.uint32), host(ref_q[0]).view(np.uint32))
                assert np.array_equal(host(q[1]).view(np.uint32), host(ref_q[1]).view(np.uint32))
    assert ta.spin_fail_flag() == 0
