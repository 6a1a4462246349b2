"""Committed golden vectors (tests/golden/kernels_small.npz, kernels_partners.npz): the oracle must
keep reproducing them (CPU), and the HIP path must match them (GPU)."""
import os

import numpy as np
import pytest

import oracle

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kernels_small.npz"))
P = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kernels_partners.npz"))
C0, C1 = np.float32(1 / 6), np.float32(1 / 36)


def test_oracle_reproduces_golden_vectors():
    assert np.array_equal(oracle.tzgemm(G["gemm_A"], G["gemm_B"], f64=True), G["gemm_C64"])
    assert np.array_equal(oracle.tzgemm(G["gemm_A"], G["gemm_B"]), G["gemm_C32"])
    a, b = G["stencil_A0"].copy(), G["stencil_A0"].copy()
    for _ in range(3):
        b = oracle.stencil(C0, C1, a, b)
        a, b = b, a
    assert np.array_equal(a, G["stencil_after3"])
    sx, sy, sz = (int(v) for v in G["lbm_dims"])
    d1 = oracle.lbm(G["lbm_src"], G["lbm_src"].copy(), sx, sy, sz)
    assert np.array_equal(d1, G["lbm_step1"])
    assert np.array_equal(oracle.lbm(d1, G["lbm_src"].copy(), sx, sy, sz), G["lbm_step2"])
    z = np.zeros(512, np.float32)
    qr, qi = oracle.mriq(G["mriq_kvals"], *G["mriq_xyz"], z, z, f64=True)
    assert np.array_equal(qr, G["mriq_Qr"]) and np.array_equal(qi, G["mriq_Qi"])
    assert np.array_equal(oracle.cp_initatoms(70)[1:65], G["cp_atoms"])
    assert np.array_equal(oracle.cp(oracle.cp_atoms_to_const(G["cp_atoms"], 0.0), np.zeros((16, 256), np.float32)),
                          G["cp_grid"])
    assert np.array_equal(oracle.im2col(G["im2col_im"], (3, 3), (1, 1), (1, 1)), G["im2col_col"])
    re, im = oracle.mrif_rhophi(G["mrif_phi"][0], G["mrif_phi"][1], G["mrif_d"][0], G["mrif_d"][1])
    assert np.array_equal(re, G["mrif_kvals"][:, 3]) and np.array_equal(im, G["mrif_kvals"][:, 4])
    fr, fi = oracle.mrif(G["mrif_kvals"], *G["mrif_xyz"], z, z, f64=True)
    assert np.array_equal(fr, G["mrif_outR"]) and np.array_equal(fi, G["mrif_outI"])


@pytest.mark.gpu
def test_hip_path_matches_golden_vectors():
    import torch
    import tacker_amd as ta
    from gpu_util import dev, host, setup
    setup()
    Cd = torch.zeros((128, 256), device="cuda:0")
    ta.gptb_tzgemm(dev(G["gemm_A"]), dev(G["gemm_B"]), Cd)
    d = np.abs(host(Cd).astype(np.float64) - G["gemm_C64"])
    assert np.all(d <= 5e-3 + 1e-5 * np.abs(G["gemm_C64"]))
    a, b = dev(G["stencil_A0"]), dev(G["stencil_A0"])
    for _ in range(3):
        ta.gptb_stencil(float(C0), float(C1), a, b)
        a, b = b, a
    assert np.array_equal(host(a), G["stencil_after3"])
    sx, sy, sz = (int(v) for v in G["lbm_dims"])
    s, d1, d2 = dev(G["lbm_src"]), dev(G["lbm_src"]), dev(G["lbm_src"])
    ta.gptb_lbm(s, d1, sx, sy, sz)
    ta.gptb_lbm(d1, d2, sx, sy, sz)
    assert np.array_equal(host(d1).view(np.uint32), G["lbm_step1"].view(np.uint32))
    assert np.array_equal(host(d2).view(np.uint32), G["lbm_step2"].view(np.uint32))
    pm = torch.zeros(96, device="cuda:0")
    ta.mriq_phimag(dev(G["mriq_phiR"]), dev(G["mriq_phiI"]), pm)
    assert np.array_equal(host(pm), G["mriq_kvals"][:, 3])
    ta.mriq_set_kvalues(G["mriq_kvals"])
    Qr, Qi = torch.zeros(512, device="cuda:0"), torch.zeros(512, device="cuda:0")
    x, y, z = (dev(v) for v in G["mriq_xyz"])
    ta.gptb_mriq(96, x, y, z, Qr, Qi)
    for got, want in ((host(Qr), G["mriq_Qr"]), (host(Qi), G["mriq_Qi"])):
        assert np.all(np.abs(got.astype(np.float64) - want) <= 1e-3 + 1e-4 * np.abs(want))
    ta.cp_set_atoms(G["cp_atoms"], 0.0)
    g = torch.zeros((16, 256), device="cuda:0")
    ta.gptb_cp(64, 0.1, g)
    assert np.array_equal(host(g).view(np.uint32), G["cp_grid"].view(np.uint32))
    col = torch.zeros(G["im2col_col"].shape, device="cuda:0")
    ta.im2col(dev(G["im2col_im"]), (3, 3), (1, 1), (1, 1), (1, 1), col)
    assert np.array_equal(host(col), G["im2col_col"])
    ta.mrif_set_kvalues(G["mrif_kvals"])
    outR, outI = torch.zeros(512, device="cuda:0"), torch.zeros(512, device="cuda:0")
    x, y, z = (dev(v) for v in G["mrif_xyz"])
    ta.gptb_mrif(96, x, y, z, outR, outI)
    for got, want in ((host(outR), G["mrif_outR"]), (host(outI), G["mrif_outI"])):
        assert np.all(np.abs(got.astype(np.float64) - want) <= 1e-3 + 1e-4 * np.abs(want))


def test_oracle_reproduces_the_partners_golden_vectors():
    assert np.array_equal(oracle.sgemm(P["sgemm_A"], P["sgemm_B"], P["sgemm_C0"]), P["sgemm_C"])
    assert np.array_equal(oracle.fft(P["fft_in"]), P["fft_out"])
    prep = oracle.cutcp_prepare(P["cutcp_atoms"], (0, 0, 0), 16, 16, 8, 0.5, 12.0)
    assert np.array_equal(oracle.cutcp(prep, 0.5, 144.0, 0.006944, (2, 2, 1)), P["cutcp_energies"])
    assert np.array_equal(oracle.nn(P["nn_locations"], 30.0, 90.0), P["nn_distances"])
    t1 = oracle.hot3d(P["hot3d_power"], P["hot3d_t0"])
    assert np.array_equal(t1, P["hot3d_t1"]) and np.array_equal(oracle.hot3d(P["hot3d_power"], t1), P["hot3d_t2"])
    assert np.array_equal(oracle.path(40, P["path_wall"], P["path_src"]), P["path_result"])
    assert np.array_equal(oracle.lava(0.5, 2, P["lava_rv"], P["lava_qv"]), P["lava_fv"])


@pytest.mark.gpu
def test_hip_path_matches_the_partners_golden_vectors():
    import torch
    import tacker_amd as ta
    from gpu_util import dev, host, setup
    setup()

    def close(got, want, atol, rtol):
        return bool(np.all(np.abs(got.astype(np.float64) - want.astype(np.float64)) <= atol + rtol * np.abs(want)))

    c = dev(P["sgemm_C0"])
    ta.gptb_sgemm(dev(P["sgemm_A"]), dev(P["sgemm_B"]), c)
    assert np.array_equal(host(c).view(np.uint32), P["sgemm_C"].view(np.uint32))
    d = dev(P["fft_in"])
    ta.gptb_fft(d)
    assert close(host(d), P["fft_out"], 1e-4, 1e-5)
    inp = ta.CutcpInput(P["cutcp_atoms"], (0, 0, 0), 16, 16, 8, 0.5, 12.0)
    ta.gptb_cutcp(inp, 144.0, 0.006944)
    assert close(host(inp.energies), P["cutcp_energies"], 2e-4, 2e-5)
    dist = torch.zeros(700, device="cuda:0")
    ta.gptb_nn(dev(P["nn_locations"]), dist, 30.0, 90.0)
    assert np.array_equal(host(dist).view(np.uint32), P["nn_distances"].view(np.uint32))
    t1, t2 = torch.zeros((4, 8, 64), device="cuda:0"), torch.zeros((4, 8, 64), device="cuda:0")
    ta.gptb_hot3d(dev(P["hot3d_power"]), dev(P["hot3d_t0"]), t1)
    ta.gptb_hot3d(dev(P["hot3d_power"]), t1, t2)
    assert np.array_equal(host(t1).view(np.uint32), P["hot3d_t1"].view(np.uint32))
    assert np.array_equal(host(t2).view(np.uint32), P["hot3d_t2"].view(np.uint32))
    res = torch.zeros(300, dtype=torch.int32, device="cuda:0")
    ta.gptb_path(40, dev(P["path_wall"]), dev(P["path_src"]), res)
    assert np.array_equal(host(res), P["path_result"])
    fv = torch.zeros((800, 4), device="cuda:0")
    ta.gptb_lava(0.5, dev(P["lava_rv"]), dev(P["lava_qv"]), fv)
    assert close(host(fv), P["lava_fv"], 2e-3, 2e-5)
    assert ta.spin_fail_flag() == 0
