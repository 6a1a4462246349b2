"""GPU tests of the ModuleCenter path (src/ModuleCenter.cu of the reference): the library's device
code loaded as gfx950 code objects, kernel objects switched to lmode DRIVER_LAUNCH, and their
results bit for bit those of the registry launches -- including kernels that read device symbols
the host fills by name, whose copies inside a code object have to follow the library's."""
import numpy as np
import pytest
import torch

import oracle
import tacker_amd as ta
from gpu_util import C0, C1, dev, gemm_inputs, gemm_tolerance_ok, host, setup, stencil_inputs

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _init():
    setup()
    ta.register_module("kernels", ta.CODE_OBJECT_PATH)
    ta.register_module("kernels_large", ta.CODE_OBJECT_LARGE_PATH)


def bits(t):
    return host(t).view(np.uint32)


def test_modules_hold_the_device_functions_by_name():
    for name in ("general_ptb_stencil", "general_ptb_lbm", "g_general_ptb_mriq", "g_general_ptb_cp", "general_ptb_mrif",
                 "general_ptb_tzgemm", "stencil_tzgemm_mix_wave_512", "ori_stencil"):
        assert ta.module_has_function("kernels", name), name
    assert ta.module_has_function("kernels_large", "general_ptb_tzgemm_large")
    assert not ta.module_has_function("kernels", "general_ptb_tzgemm_large")
    assert not ta.module_has_function("kernels", "no_such_kernel")
    with pytest.raises(ta.TackerError):
        ta.register_module("broken", __file__)                      # not a code object


def test_stencil_launched_from_the_code_object_equals_the_registry_launch():
    A0 = stencil_inputs(10, 36, 200, seed=51)
    a0 = dev(A0)
    want, got = a0.clone(), a0.clone()
    blocks = ta.stencil_blocks(200, 36, 10)
    g = ta.gptb_create(ta.ori_stencil_create(C0, C1, a0, want), 0, 0, 0, blocks)
    g.execute()
    m = ta.gptb_create(ta.ori_stencil_create(C0, C1, a0, got), 0, 0, 0, blocks)
    with pytest.raises(ta.TackerError):
        m.use_module("kernels", "no_such_kernel")
    m.use_module("kernels", "general_ptb_stencil")
    m.execute()
    assert np.array_equal(bits(got), bits(want))
    assert np.array_equal(bits(got), oracle.stencil(C0, C1, A0, A0).view(np.uint32))
    # a part of the position grid through the driver launch
    got.copy_(a0)
    m.set_range(3, blocks - 2)
    m.execute()
    assert np.array_equal(bits(got), oracle.stencil_gptb(C0, C1, A0, A0, start=3, end=blocks - 2, gdz="runs").view(np.uint32))


def test_cp_from_the_code_object_sees_the_atoms_set_before_and_after_it_was_loaded():
    atoms = ta.cp_initatoms(4000)
    first, second = atoms[1:65], atoms[101:165]
    ta.cp_set_atoms(first, 0.0)
    ta.register_module("kernels_loaded_later", ta.CODE_OBJECT_PATH)       # its table is filled at load
    for name, table in (("kernels_loaded_later", first), ("kernels_loaded_later", second), ("kernels", second)):
        ta.cp_set_atoms(table, 0.0)                                       # ... and follows later writes
        g = torch.zeros((32, 512), device="cuda:0")
        k = ta.gptb_create(ta.ori_cp_create(64, 0.1, g), 0, 0, 0, ta.cp_blocks(512, 32))
        k.use_module(name, "g_general_ptb_cp")
        k.execute()
        want = oracle.cp(oracle.cp_atoms_to_const(table, 0.0), np.zeros((32, 512), np.float32))
        assert np.array_equal(bits(g), want.view(np.uint32)), name


def test_k_split_gemm_from_the_code_object_finds_its_workspace():
    # 256 x 384 x 1024: workgroups share reductions through a workspace found in a device table keyed by C;
    # the code object has a table of its own, which the runtime's writes have to reach
    M, N, K = 256, 384, 1024
    A, B = gemm_inputs(M, N, K, seed=52)
    dA, dB = dev(A), dev(B)
    want = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dA, dB, want)
    got = torch.full((M, N), -7.0, device="cuda:0")
    tiles = ta.tzgemm_grid_dim(M, N, K)[3]
    g = ta.gptb_create(ta.ori_tzgemm_create(dA, dB, got), 0, 0, 0, tiles)
    g.use_module("kernels", "general_ptb_tzgemm")
    g.execute()
    assert np.array_equal(bits(got), bits(want))
    ok, fro, dmax = gemm_tolerance_ok(host(got), oracle.tzgemm(A, B, f64=True), K)
    assert ok and fro <= 1e-5, (fro, dmax)
    assert ta.spin_fail_flag() == 0


def test_large_tile_gemm_and_a_fused_kernel_from_code_objects():
    M, N, K = 4096, 4096, 256
    A, B = gemm_inputs(M, N, K, seed=53)
    dA, dB = dev(A), dev(B)
    want = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dA, dB, want)                                          # the host picks the large-tile build
    got = torch.full((M, N), -7.0, device="cuda:0")
    tiles = ta.tzgemm_grid_dim(M, N, K)[3]
    tz = ta.gptb_create(ta.ori_tzgemm_create(dA, dB, got), 0, 0, 0, tiles)
    tz.use_module("kernels_large", "general_ptb_tzgemm_large")
    tz.execute()
    assert np.array_equal(bits(got), bits(want))
    # fused: tzgemm + stencil from the code object against the same pair from the registry
    A0 = stencil_inputs(10, 36, 200, seed=54)
    a0 = dev(A0)
    s_want, s_got = a0.clone(), a0.clone()
    blocks = ta.stencil_blocks(200, 36, 10)
    c_want, c_got = torch.zeros((M, N), device="cuda:0"), torch.zeros((M, N), device="cuda:0")
    for c, s, module in ((c_want, s_want, None), (c_got, s_got, "kernels")):
        st = ta.gptb_create(ta.ori_stencil_create(C0, C1, a0, s), 0, 0, 0, blocks)
        tzk = ta.gptb_create(ta.ori_tzgemm_create(dA, dB, c), 0, 0, 0, tiles)
        mix = ta.mix_create(st, tzk, 0, blocks, 0, tiles, variant="wave_512")
        if module:
            mix.use_module(module, "stencil_tzgemm_mix_wave_512")
        mix.execute()
    assert np.array_equal(bits(c_got), bits(c_want)) and np.array_equal(bits(s_got), bits(s_want))
    assert np.array_equal(bits(s_got), oracle.stencil(C0, C1, A0, A0).view(np.uint32))
    assert np.array_equal(bits(c_got), bits(want))
    assert ta.spin_fail_flag() == 0


def test_cutcp_and_fft_from_the_code_object():
    # cutcp reads its neighbour list from two device symbols (NbrListLen, NbrList): the copies inside a code
    # object follow the library's, whether the list was loaded before the object or after; fft carries its
    # twiddle table in the object itself
    rng = np.random.default_rng(61)
    atoms = np.empty((300, 4), np.float32)
    atoms[:, :3] = rng.uniform(0, 7.5, (300, 3))
    atoms[:, 3] = rng.uniform(0.1, 1, 300)
    inp = ta.CutcpInput(atoms, (0, 0, 0), 16, 16, 16, 0.5, 12.0)          # loads the list: the modules are already there
    want = torch.zeros_like(inp.energies)
    ta.gptb_cutcp(inp, 144.0, 0.006944, want)
    for name in ("kernels", "kernels_after_cutcp"):
        if name != "kernels":
            ta.register_module(name, ta.CODE_OBJECT_PATH)                 # loaded after the list: filled at load
        got = torch.full_like(inp.energies, -1.0)
        k = ta.gptb_create(ta.ori_cutcp_create(inp, 144.0, 0.006944, got), 0, 0, 0, inp.blocks())
        k.use_module(name, "general_ptb_cutcp")
        k.execute()
        assert np.array_equal(bits(got), bits(want)), name
    d = rng.uniform(-1, 1, (70, 256, 2)).astype(np.float32)
    a, b = dev(d), dev(d)
    ta.gptb_fft(a)
    k = ta.gptb_create(ta.ori_fft_create(b), 0, 0, 0, 70)
    k.use_module("kernels", "g_general_ptb_fft")
    k.execute()
    assert np.array_equal(bits(a), bits(b))
    assert ta.spin_fail_flag() == 0


def test_the_rodinia_kernels_from_the_code_object():
    # cuModuleGetFunction + cuLaunchKernel (src/ModuleCenter.cu) with structs passed by value (lavaMD's par_str,
    # dim_str): the driver-style launch from the code object gives the registry launch's bits
    rng = np.random.default_rng(62)
    loc = dev(rng.uniform(0, 90, (3000, 2)).astype(np.float32))
    want, got = torch.zeros(3000, device="cuda:0"), torch.full((3000,), -1.0, device="cuda:0")
    ta.gptb_nn(loc, want, 30.0, 90.0)
    k = ta.gptb_create(ta.ori_nn_create(loc, got, 30.0, 90.0), 0, 0, 0, ta.nn_blocks(3000))
    k.use_module("kernels", "general_ptb_nn")
    k.execute()
    assert np.array_equal(bits(got), bits(want))
    p, t = dev(rng.uniform(0, 0.01, (4, 8, 128)).astype(np.float32)), dev(rng.uniform(320, 340, (4, 8, 128)).astype(np.float32))
    want, got = torch.zeros((4, 8, 128), device="cuda:0"), torch.full((4, 8, 128), -1.0, device="cuda:0")
    ta.gptb_hot3d(p, t, want)
    k = ta.gptb_create(ta.ori_hot3d_create(p, t, got), 0, 0, 0, ta.hot3d_blocks(128, 8))
    k.use_module("kernels", "general_ptb_hot3d")
    k.execute()
    assert np.array_equal(bits(got), bits(want))
    wall, src = dev(rng.integers(0, 10, (50, 900), dtype=np.int32)), dev(rng.integers(0, 10, 900, dtype=np.int32))
    want = torch.zeros(900, dtype=torch.int32, device="cuda:0")
    got = torch.full((900,), -1, dtype=torch.int32, device="cuda:0")
    ta.gptb_path(50, wall, src, want)
    k = ta.gptb_create(ta.ori_path_create(50, wall, src, got), 0, 0, 0, ta.path_blocks(900, 50))
    k.use_module("kernels", "general_ptb_path")
    k.execute()
    assert np.array_equal(host(got), host(want))
    rv = dev((rng.integers(1, 11, (800, 4)) / 10.0).astype(np.float32))
    qv = dev((rng.integers(1, 11, 800) / 10.0).astype(np.float32))
    want, got = torch.zeros((800, 4), device="cuda:0"), torch.zeros((800, 4), device="cuda:0")
    ta.gptb_lava(0.5, rv, qv, want)
    k = ta.gptb_create(ta.ori_lava_create(0.5, rv, qv, got), 0, 0, 0, ta.lava_blocks(2))
    k.use_module("kernels", "general_ptb_lava")
    k.execute()
    assert np.array_equal(bits(got), bits(want))
    assert ta.spin_fail_flag() == 0
