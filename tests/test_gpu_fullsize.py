"""GPU parity at the benchmark's full sizes (configs 2 to 5), through the C-ABI.

The oracle runs where it finishes in seconds (stencil sweeps, one lbm step, row samples of
the GEMM, voxel samples of mri-q); what it cannot cover is checked through properties that
do not depend on size: fused output == unfused output bit for bit, a checksum of checksums
for the GEMM (column sums of C against 1.1 * (column sums of A) * B^T in float64), mass
conservation of the lbm step, linearity of the stencil sweep.
"""
import numpy as np
import pytest
import torch

import oracle
import tacker_amd as ta
from gpu_util import (C0, C1, dev, gemm_inputs, host, lbm_inputs, mriq_inputs, setup, stencil_inputs)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _init():
    setup()


def gemm_sample_ok(got, A, B, rows):
    """rows of C against a float64 product of the fp16 operands, tolerance of the GEMM bar"""
    truth = np.float64(np.float32(1.1)) * (A[rows].astype(np.float64) @ B.astype(np.float64).T)
    d = np.abs(got[rows].astype(np.float64) - truth)
    return bool(np.all(d <= 5e-3 + 1e-5 * np.abs(truth))), float(d.max())


def gemm_checksum_ok(got, A, B):
    """sum over rows of C = 1.1 * (sum over rows of A) * B^T: one float64 vector per side"""
    lhs = got.astype(np.float64).sum(axis=0)
    rhs = np.float64(np.float32(1.1)) * (A.astype(np.float64).sum(axis=0) @ B.astype(np.float64).T)
    scale = np.abs(A.astype(np.float64)).sum(axis=0) @ np.abs(B.astype(np.float64)).T
    return bool(np.all(np.abs(lhs - rhs) <= 1e-6 * scale + 1e-3))


def test_config2_tzgemm_2048_and_stencil_512x512x64_fused_equals_unfused_equals_oracle():
    M = N = K = 2048
    A, B = gemm_inputs(M, N, K)
    A0 = stencil_inputs(64, 512, 512)
    dA, dB, a0 = dev(A), dev(B), dev(A0)
    solo_c = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dA, dB, solo_c)
    solo_s = a0.clone()
    ta.gptb_stencil(C0, C1, a0, solo_s)
    mix_c = torch.zeros((M, N), device="cuda:0")
    mix_s = a0.clone()
    ta.mix_tzgemm_stencil(C0, C1, a0, mix_s, dA, dB, mix_c)
    got_c, got_s = host(mix_c), host(mix_s)
    assert np.array_equal(got_c, host(solo_c))
    assert np.array_equal(got_s, host(solo_s))
    assert np.array_equal(got_s, oracle.stencil(C0, C1, A0, A0))        # bit-exact, 16.7 M points
    rows = np.random.default_rng(0).choice(M, 48, replace=False)
    ok, dmax = gemm_sample_ok(got_c, A, B, rows)
    assert ok, dmax
    assert gemm_checksum_ok(got_c, A, B)
    assert ta.spin_fail_flag() == 0


def test_config2_ten_sweeps_with_pointer_swap_track_the_oracle():
    A0 = stencil_inputs(64, 512, 512, seed=2)
    a, b = dev(A0), dev(A0)
    ha, hb = A0.copy(), A0.copy()
    for _ in range(10):
        ta.gptb_stencil(C0, C1, a, b)
        hb = oracle.stencil(C0, C1, ha, hb)
        a, b = b, a
        ha, hb = hb, ha
    assert np.array_equal(host(a), ha)


def test_stencil_full_size_is_linear_in_its_input():
    # sweep(2^-3 * A) == 2^-3 * sweep(A) exactly: scaling by a power of two commutes with
    # every rounding of the expression (no subnormals at these magnitudes)
    A0 = stencil_inputs(64, 512, 512, seed=3)
    a0 = dev(A0)
    out = a0.clone()
    ta.gptb_stencil(C0, C1, a0, out)
    a1 = dev(A0 * np.float32(0.125))
    out1 = a1.clone()
    ta.gptb_stencil(C0, C1, a1, out1)
    assert np.array_equal(host(out1), host(out) * np.float32(0.125))


def test_config3_tzgemm_4096x4096x1024_and_lbm_120x120x150():
    M, N, K = 4096, 4096, 1024
    A, B = gemm_inputs(M, N, K, seed=21)
    sx, sy, sz = 120, 120, 150
    src = lbm_inputs(sx, sy, sz)
    s = dev(src)
    dA, dB = dev(A), dev(B)
    solo_c = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dA, dB, solo_c)
    solo_d = torch.zeros_like(s)
    ta.gptb_lbm(s, solo_d, sx, sy, sz)
    mix_c = torch.zeros((M, N), device="cuda:0")
    mix_d = torch.zeros_like(s)
    ta.mix_tzgemm_lbm(s, mix_d, sx, sy, sz, dA, dB, mix_c)
    got_c, got_d = host(mix_c), host(mix_d)
    assert np.array_equal(got_c, host(solo_c))
    assert np.array_equal(got_d.view(np.uint32), host(solo_d).view(np.uint32))
    want = oracle.lbm(src, np.zeros_like(src), sx, sy, sz)               # one step, 2.16 M cells
    assert np.array_equal(got_d.view(np.uint32), want.view(np.uint32))
    rows = np.random.default_rng(1).choice(M, 32, replace=False)
    ok, dmax = gemm_sample_ok(got_c, A, B, rows)
    assert ok, dmax
    assert gemm_checksum_ok(got_c, A, B)
    # collision conserves mass cell by cell and streaming only moves it; the only mass that
    # disappears is what the bottom plane sends down and the top plane sends up (5 of the 19
    # directions each, about 1/6 of a cell's mass): a loss of about (2/sz)/6 of the total
    cells = sx * sy * sz
    m_in = src.reshape(20, cells)[:19].astype(np.float64).sum()
    m_out = got_d.reshape(20, cells)[:19].astype(np.float64).sum()
    loss = (m_in - m_out) / m_in
    assert 0.5 * (2.0 / sz) / 6 <= loss <= 1.5 * (2.0 / sz) / 6, loss


def test_config3_ten_lbm_steps_with_grid_swap_track_the_oracle_step_by_step():
    # both grids start as the same lattice (obstacle and accelerated cells marked in both, as the
    # benchmark's loader leaves them); after each step source and destination change places
    sx, sy, sz = 120, 120, 150
    src = lbm_inputs(sx, sy, sz, seed=77, accel_p=0.01)
    a, b = dev(src), dev(src)
    ha, hb = src.copy(), src.copy()
    k = ta.ori_lbm_create(a, b, sx, sy, sz)
    g = ta.gptb_create(k, 0, 0, 0, sy * sz)
    for step in range(10):
        g.execute()                                              # the object follows the swap below
        hb = oracle.lbm(ha, hb, sx, sy, sz)
        k.swap_buffers()
        a, b = b, a
        ha, hb = hb, ha
        torch.cuda.synchronize()
        assert np.array_equal(host(a).view(np.uint32), ha.view(np.uint32)), step
    assert np.isfinite(ha.reshape(20, -1)[:19]).all()
    g.close()
    k.close()


def test_config4_tzgemm_2048_and_mriq_2048x262144():
    M = N = K = 2048
    A, B = gemm_inputs(M, N, K, seed=22)
    numK, numX = 2048, 262144
    k, phiR, phiI, xyz = mriq_inputs(numK, numX)
    kv = np.concatenate([k, oracle.mriq_phimag(phiR, phiI)[:, None]], 1).astype(np.float32)
    ta.mriq_set_kvalues(kv)
    x, y, z = dev(xyz[0]), dev(xyz[1]), dev(xyz[2])
    dA, dB = dev(A), dev(B)
    solo_r, solo_i = torch.zeros(numX, device="cuda:0"), torch.zeros(numX, device="cuda:0")
    ta.gptb_mriq(numK, x, y, z, solo_r, solo_i)
    solo_c = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dA, dB, solo_c)
    mix_c = torch.zeros((M, N), device="cuda:0")
    Qr, Qi = torch.zeros(numX, device="cuda:0"), torch.zeros(numX, device="cuda:0")
    ta.mix_tzgemm_mriq(numK, x, y, z, Qr, Qi, dA, dB, mix_c)
    assert np.array_equal(host(mix_c), host(solo_c))
    got_r, got_i = host(Qr), host(Qi)
    assert np.array_equal(got_r, host(solo_r)) and np.array_equal(got_i, host(solo_i))
    # float64 truth on a sample of voxels (numpy, independent of the oracle's loop)
    pick = np.random.default_rng(2).choice(numX, 512, replace=False)
    phase = 2.0 * np.pi * (kv[:, 0:1].astype(np.float64) * xyz[0][pick] + kv[:, 1:2].astype(np.float64) * xyz[1][pick]
                           + kv[:, 2:3].astype(np.float64) * xyz[2][pick])
    tr = (kv[:, 3:4].astype(np.float64) * np.cos(phase)).sum(axis=0)
    ti = (kv[:, 3:4].astype(np.float64) * np.sin(phase)).sum(axis=0)
    assert np.all(np.abs(got_r[pick] - tr) <= 1e-3 + 1e-4 * np.abs(tr))
    assert np.all(np.abs(got_i[pick] - ti) <= 1e-3 + 1e-4 * np.abs(ti))
    ok, dmax = gemm_sample_ok(host(mix_c), A, B, np.arange(0, M, 97))
    assert ok, dmax
    assert ta.spin_fail_flag() == 0


def test_config4_mriq_spread_over_nine_fused_launches_equals_one_launch():
    # the co-location pattern of benchmark configuration 4: the k-chunk x voxel-block grid of mri-q is cut
    # into 9 consecutive slices, each riding with one GEMM launch; Q must come out bit-identical to the kernel
    # run alone (a float carried through memory between chunks is the float the one k loop keeps in a register)
    M = N = K = 2048
    A, B = gemm_inputs(M, N, K, seed=23)
    numK, numX = 2048, 262144
    k, phiR, phiI, xyz = mriq_inputs(numK, numX, seed=4)
    kv = np.concatenate([k, oracle.mriq_phimag(phiR, phiI)[:, None]], 1).astype(np.float32)
    ta.mriq_set_kvalues(kv)
    x, y, z = dev(xyz[0]), dev(xyz[1]), dev(xyz[2])
    dA, dB = dev(A), dev(B)
    solo_r, solo_i = torch.zeros(numX, device="cuda:0"), torch.zeros(numX, device="cuda:0")
    ta.ori_mriq(numK, x, y, z, solo_r, solo_i)
    solo_c = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dA, dB, solo_c)
    Qr, Qi = torch.zeros(numX, device="cuda:0"), torch.zeros(numX, device="cuda:0")
    mix_c = torch.zeros((M, N), device="cuda:0")
    total = ta.mriq_blocks(numK, numX)
    assert total == 1024 * 16
    n = 9
    for i in range(n):
        ta.mix_tzgemm_mriq(numK, x, y, z, Qr, Qi, dA, dB, mix_c, be_start=total * i // n, be_end=total * (i + 1) // n)
    assert np.array_equal(host(Qr), host(solo_r)) and np.array_equal(host(Qi), host(solo_i))
    assert np.array_equal(host(mix_c), host(solo_c))
    assert ta.spin_fail_flag() == 0


def test_mrif_2048x262144_spread_over_ten_fused_launches_equals_one_launch():
    # mri-fhd at mri-q's benchmark size (the reference's tzgemm_mrif mix): the position grid cut into 10
    # consecutive slices, each riding with one 2048^3 GEMM launch, gives the bits of the natural launch; a
    # sample of voxels is checked against a complex128 matrix product in numpy
    from gpu_util import mrif_inputs, mrif_table
    M = N = K = 2048
    A, B = gemm_inputs(M, N, K, seed=24)
    numK, numX = 2048, 262144
    k, phi, d, xyz = mrif_inputs(numK, numX, seed=6)
    kv = mrif_table(k, phi, d)
    ta.mrif_set_kvalues(kv)
    x, y, z = dev(xyz[0]), dev(xyz[1]), dev(xyz[2])
    dA, dB = dev(A), dev(B)
    solo_r, solo_i = torch.zeros(numX, device="cuda:0"), torch.zeros(numX, device="cuda:0")
    ta.ori_mrif(numK, x, y, z, solo_r, solo_i)
    solo_c = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dA, dB, solo_c)
    outR, outI = torch.zeros(numX, device="cuda:0"), torch.zeros(numX, device="cuda:0")
    mix_c = torch.zeros((M, N), device="cuda:0")
    total = ta.mrif_blocks(numK, numX)
    assert total == 1024 * 16
    n = 10
    for i in range(n):
        ta.mix_tzgemm_mrif(numK, x, y, z, outR, outI, dA, dB, mix_c, be_start=total * i // n, be_end=total * (i + 1) // n)
    got_r, got_i = host(outR), host(outI)
    assert np.array_equal(got_r, host(solo_r)) and np.array_equal(got_i, host(solo_i))
    assert np.array_equal(host(mix_c), host(solo_c))
    pick = np.random.default_rng(3).choice(numX, 512, replace=False)
    X = np.stack([xyz[0][pick], xyz[1][pick], xyz[2][pick]], 1).astype(np.float64)
    want = np.exp(2j * np.pi * (X @ kv[:, :3].astype(np.float64).T)) @ (kv[:, 3].astype(np.float64) + 1j * kv[:, 4])
    assert np.all(np.abs(got_r[pick] - want.real) <= 1e-3 + 1e-4 * np.abs(want.real))
    assert np.all(np.abs(got_i[pick] - want.imag) <= 1e-3 + 1e-4 * np.abs(want.imag))
    assert ta.spin_fail_flag() == 0


def test_config5_vgg16_224_colocated_queries_equal_the_solo_query():
    # VGG16 batch 1 at 224x224 under TaskManager, with the reference's always-fuse policy and the kinfo
    # block counts (mri-q, then the stencil), then with calibrated counts and mri-q: whatever rides along, the logits are the solo query's bit for bit, no role barrier was
    # abandoned, and the latencies are inside the budget.  The deep layers take the shared-reduction
    # form of the GEMM here (conv4, conv5, fc: 2 to 8 workgroups per tile).
    task = ta.LcTask("vgg16")
    shapes = [k["args"] for k in task.kernels() if k["mixable"]]
    assert len(shapes) == 16
    assert ta.tzgemm_parts(14 * 14, 512, 9 * 512) == 8 and ta.tzgemm_parts(128, 4096, 25088) == 4
    task.execute()
    torch.cuda.synchronize()
    p, stride, n = task.logits()
    solo = ta.device_to_host(p, (n, stride), np.float32)[:, 0].copy()
    assert np.isfinite(solo).all() and np.abs(solo).max() > 0
    for _ in range(3):                                   # the query is reproducible
        task.execute()
    torch.cuda.synchronize()
    assert np.array_equal(ta.device_to_host(p, (n, stride), np.float32)[:, 0], solo)

    for be in ("mriq", "stencil"):
        tm = ta.TaskManager(task, be, "lbm")
        tm.configure(qos_budget_ms=50.0, guard_ms=4.0, warmup=2, profile=5, queries=20, verbose=0)
        tm.set_fusion_strikes(0)                         # the reference's loop: fuse whenever the budget allows
        rep = tm.run("aker", second_stage=False)
        torch.cuda.synchronize()
        if be == "mriq":                                 # its kinfo table has blocks for every layer's K
            assert rep["mix_times"] > 0 and rep["be_blocks_executed"] > 0
        assert np.array_equal(ta.device_to_host(p, (n, stride), np.float32)[:, 0], solo)
        assert all(0 < v < 50.0 for v in tm.latencies())
        tm.close()

    tm = ta.TaskManager(task, "mriq", "lbm")
    tm.configure(qos_budget_ms=50.0, guard_ms=4.0, warmup=2, profile=5, queries=20, verbose=0)
    tm.set_calibration(True, 0.10)
    rep = tm.run("aker", second_stage=False)
    torch.cuda.synchronize()
    assert len(tm.calibrated_blocks()) >= 16
    assert np.array_equal(ta.device_to_host(p, (n, stride), np.float32)[:, 0], solo)
    assert all(0 < v < 50.0 for v in tm.latencies())
    assert ta.spin_fail_flag() == 0
    tm.close()

    # a budget for the whole query, both forms of the fused kernel, the stencil's large slices allowed:
    # what the pass chooses stays inside the budget by its own figures, and the logits do not move
    tm = ta.TaskManager(task, "stencil", "lbm")
    tm.configure(qos_budget_ms=50.0, guard_ms=4.0, warmup=2, profile=20, queries=20, verbose=0)
    tm.set_calibration(True, 1.5)
    tm.set_calibration_budget(0.15, 2)
    tm.set_calibration_variants(("default", "wave_256"))
    tm.set_end_to_end(10)
    rep = tm.run("aker", second_stage=False)
    torch.cuda.synchronize()
    blocks = tm.calibrated_blocks()
    assert len(blocks) >= 16 and all(0 <= b <= 8192 for b in blocks)
    assert all(v in ("", "wave_256") for v in tm.calibrated_variants())
    assert np.array_equal(ta.device_to_host(p, (n, stride), np.float32)[:, 0], solo)
    assert all(0 < v < 50.0 for v in tm.latencies())
    solo_e2e = np.median(tm.latencies(kind="e2e_solo"))
    assert np.median(tm.latencies(kind="e2e_colocated")) < 1.5 * solo_e2e
    assert ta.spin_fail_flag() == 0
    tm.close()
    task.close()
