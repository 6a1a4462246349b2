"""GPU parity of the cutoff Coulomb potential partner (src/ori_kernel/cutcp_kernel.cu,
src/gptb_kernel/cutcp_kernel.cu, src/mix_kernel/tzgemm_cutcp.cu): against the oracle's walk through the
bins within |d| <= 2e-4 + 2e-5 |ref| (the hardware's reciprocal square root here, 1 / sqrtf there, CUDA's
rsqrtf in the reference: approximations of an ulp each, summed over hundreds of atoms) and against the
float64 sum over the atom list; the natural launch, the GPTB form over any tiling of its positions and
every fused variant give the same bits as each other (positions = regions x parts of the neighbour list); the host's binning equals the oracle's exactly."""
import numpy as np
import pytest
import torch

import oracle
import tacker_amd as ta
from gpu_util import dev, gemm_inputs, gemm_tolerance_ok, host, setup

pytestmark = pytest.mark.gpu
H, CUTOFF = 0.5, 12.0
C2, INV_C2 = 144.0, 0.006944            # as the reference types them (src/ori_kernel/cutcp_kernel.cu:226-227)


@pytest.fixture(scope="module", autouse=True)
def _init():
    setup()


def atoms_in_box(n, box, seed):
    rng = np.random.default_rng(seed)
    a = np.empty((n, 4), np.float32)
    a[:, :3] = rng.uniform(0, box, (n, 3))
    a[:, 3] = rng.uniform(-1, 1, n)
    a[a[:, 3] == 0, 3] = 0.5
    return a


def close(got, want):
    return bool(np.all(np.abs(got.astype(np.float64) - want.astype(np.float64)) <= 2e-4 + 2e-5 * np.abs(want)))


def bits(t):
    return host(t).view(np.uint32)


def case(points=(24, 24, 16), natoms=500, seed=4):
    nx, ny, nz = points
    atoms = atoms_in_box(natoms, (min(points) - 1) * H, seed)
    inp = ta.CutcpInput(atoms, (0, 0, 0), nx, ny, nz, H, CUTOFF)
    prep = oracle.cutcp_prepare(atoms, (0, 0, 0), nx, ny, nz, H, CUTOFF)
    return atoms, inp, prep


def test_host_binning_equals_the_oracles():
    atoms = atoms_in_box(5000, 19.5, seed=8)          # dense: some bins overflow
    atoms[3, 3] = 0.0
    inp = ta.CutcpInput(atoms, (0.25, -0.5, 0.0), 40, 40, 40, H, CUTOFF)
    prep = oracle.cutcp_prepare(atoms, (0.25, -0.5, 0.0), 40, 40, 40, H, CUTOFF)
    assert inp.binDim == prep["binDim"] and inp.padding == prep["padding"]
    assert np.array_equal(inp.host_bins, prep["bins"]) and np.array_equal(inp.nbr, prep["nbr"])
    assert (inp.extra, inp.excluded) == (prep["extra"], prep["excluded"]) and inp.extra > 0 and inp.excluded >= 1


def test_ori_and_gptb_forms_match_the_oracle_and_the_float64_sum():
    atoms, inp, prep = case()
    want = oracle.cutcp(prep, H, C2, INV_C2, inp.regions)
    e_ori, e_gptb, e_small = (torch.zeros_like(inp.energies) for _ in range(3))
    ta.ori_cutcp(inp, C2, INV_C2, e_ori)
    ta.gptb_cutcp(inp, C2, INV_C2, e_gptb)
    ta.gptb_cutcp(inp, C2, INV_C2, e_small, launch_grid=3, launch_block=64)
    assert close(host(e_ori), want) and np.abs(want).max() > 1.0
    assert np.array_equal(bits(e_gptb), bits(e_ori)) and np.array_equal(bits(e_small), bits(e_ori))
    # float64, no bins: every binned atom against every lattice point
    b = prep["bins"].reshape(-1, 4)
    b = b[b[:, 3] != 0].astype(np.float64)
    rx, ry, rz = inp.regions
    zs, ys, xs = np.arange(8 * rz) * H, np.arange(8 * ry) * H, np.arange(8 * rx) * H
    pot = np.zeros((8 * rz, 8 * ry, 8 * rx))
    for ax, ay, az, q in b:
        r2 = (az - zs)[:, None, None] ** 2 + (ay - ys)[None, :, None] ** 2 + (ax - xs)[None, None, :] ** 2
        with np.errstate(divide="ignore", invalid="ignore"):
            pot += np.where(r2 < C2, q / np.sqrt(r2) * (1.0 - r2 * INV_C2) ** 2, 0.0)
    truth = pot.reshape(rz, 8, ry, 8, rx, 8).transpose(0, 2, 4, 1, 3, 5)
    assert close(host(e_ori), truth)
    assert ta.spin_fail_flag() == 0


@pytest.mark.parametrize("seed", range(4))
def test_any_tiling_of_the_positions_gives_the_one_kernel(seed):
    rng = np.random.default_rng(800 + seed)
    atoms, inp, prep = case(points=[(24, 16, 16), (16, 24, 8), (8, 8, 40), (32, 16, 16)][seed], natoms=300, seed=seed)
    whole = torch.zeros_like(inp.energies)
    ta.ori_cutcp(inp, C2, INV_C2, whole)
    n = inp.blocks()
    cuts = sorted(set(rng.integers(0, n + 1, 3).tolist()) | {0, n})
    e = torch.full_like(inp.energies, -3.0)
    for a, b in zip(cuts, cuts[1:]):
        ta.gptb_cutcp(inp, C2, INV_C2, e, a, b, launch_grid=int(rng.choice([1, 5, 64, 256])),
                      launch_block=int(rng.choice([64, 128, 256])))
    assert np.array_equal(bits(e), bits(whole))
    assert n == oracle.cutcp_positions(inp.regions, len(inp.nbr)) == inp.regions[0] * inp.regions[1] * inp.regions[2] * 11
    # a partial range touches its regions only, in the reference's position order (x slowest); positions 1 and 2
    # are the first part of the neighbour list (entries 0, 11, 22, ...) of regions 1 and 2
    e = torch.full_like(inp.energies, -3.0)
    ta.gptb_cutcp(inp, C2, INV_C2, e, 1, 3)
    want = oracle.cutcp(prep, H, C2, INV_C2, inp.regions, 1, 3, out=np.full(tuple(e.shape), -3.0, np.float32),
                        parts="chunks")
    got = host(e)
    assert np.array_equal(got == -3.0, want == -3.0) and close(got, want)


@pytest.mark.parametrize("variant", [None, "wave_128", "wave_256", "wave_512", "wg_1_1", "wg_1_2"])
def test_mix_tzgemm_cutcp(variant):
    M, N, K = 256, 256, 256
    A, B = gemm_inputs(M, N, K, seed=31)
    atoms, inp, prep = case(natoms=400, seed=6)
    solo_c = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dev(A), dev(B), solo_c)
    solo_e = torch.zeros_like(inp.energies)
    ta.gptb_cutcp(inp, C2, INV_C2, solo_e)
    mix_c = torch.zeros((M, N), device="cuda:0")
    mix_e = torch.zeros_like(inp.energies)
    ta.mix_tzgemm_cutcp(inp, C2, INV_C2, dev(A), dev(B), mix_c, mix_e, variant=variant)
    assert np.array_equal(host(mix_c), host(solo_c))
    assert np.array_equal(bits(mix_e), bits(solo_e))
    assert close(host(mix_e), oracle.cutcp(prep, H, C2, INV_C2, inp.regions))
    ok, fro, dmax = gemm_tolerance_ok(host(mix_c), oracle.tzgemm(A, B, f64=True), K)
    assert ok and fro <= 1e-5
    n = inp.blocks()
    mix_e.zero_()
    mix_c.zero_()
    ta.mix_tzgemm_cutcp(inp, C2, INV_C2, dev(A), dev(B), mix_c, mix_e, be_start=0, be_end=5, tile_start=0, tile_end=5,
                        variant=variant)
    ta.mix_tzgemm_cutcp(inp, C2, INV_C2, dev(A), dev(B), mix_c, mix_e, be_start=5, be_end=n, tile_start=5, tile_end=16,
                        variant=variant)
    assert np.array_equal(bits(mix_e), bits(solo_e)) and np.array_equal(host(mix_c), host(solo_c))
    assert ta.spin_fail_flag() == 0


def test_creator_object_is_the_references_instance_on_seeded_atoms():
    # createKernel("cutcp"): 208^3 lattice points, spacing 0.5, cutoff 12, bins 32 x 32, grid (26, 26, 2)
    # (src/ori_kernel/cutcp_kernel.cu:181-263)
    k = ta.create_kernel("cutcp")
    info = k.info()
    assert (info["ptb_start"], info["ptb_end"], info["ori_grid_x"], info["ori_grid_y"]) == (0, 26 * 26 * 2 * 11, 26, 26)
    assert (k.param(0, "int"), k.param(1, "int")) == (32, 32)
    assert abs(k.param(3, "float") - 0.5) < 1e-7 and abs(k.param(4, "float") - 144.0) < 1e-4
    assert abs(k.param(5, "float") - 0.006944) < 1e-8
    k.execute()
    torch.cuda.synchronize()
    bins = ta.device_to_host(k.param(2) - (((3 * 32 + 3) * 32 + 3) * 32) * 4, (32, 32, 32, 8, 4), np.float32)
    assert 60000 < np.count_nonzero(bins[..., 3]) <= 70000
    got = ta.device_to_host(k.param(6), (2, 26, 26, 8, 8, 8), np.float32)
    prep = {"bins": bins, "padding": 3, "binDim": (32, 32, 32),
            "nbr": oracle.cutcp_prepare(np.zeros((0, 4), np.float32), (0, 0, 0), 208, 208, 208, H, CUTOFF)["nbr"]}
    for pos in (0, 700, 1351):                                   # x slowest: region (pos // 52, (pos // 2) % 26, pos % 2)
        want = oracle.cutcp(prep, H, C2, INV_C2, (26, 26, 2), pos, pos + 1)
        x, y, z = pos // 52, (pos // 2) % 26, pos % 2
        assert close(got[z, y, x], want[z, y, x]) and np.abs(want[z, y, x]).max() > 0.1
    assert ta.spin_fail_flag() == 0


def test_bad_arguments_are_refused():
    lib = ta.lib()
    atoms, inp, prep = case(natoms=10)
    a = inp.args(C2, INV_C2)
    assert lib.tacker_ori_cutcp(*((a[0], a[1], None) + a[3:]), None) == 1
    assert lib.tacker_gptb_cutcp(*(a[:7] + (0, 2, 2)), 0, 1, 0, 0, None) == 1
    assert lib.tacker_cutcp_set_neighbours(None, 5) == 1 and lib.tacker_cutcp_set_neighbours(inp.nbr.ctypes.data, 2000) == 1
    inp.load_neighbours()
