"""GPU parity of the Rodinia partners nn, hotspot3D, pathfinder and lavaMD
(src/ori_kernel/{nn,hot3d,path,lava}_kernel.cu, src/gptb_kernel/*, src/mix_kernel/tzgemm_{nn,hot3d,path,lava}.cu,
hot3d_nn.cu, hot3d_path.cu, nn_path.cu, hot3d_lava.cu, lava_nn.cu, lava_path.cu): bit for bit against the oracle
-- fp32 in the reference's operation order for nn and hot3d, integers for path -- and within
|d| <= 2e-3 + 2e-5 |ref| for lavaMD (the hardware's exponential against the C library's), for the natural
launch, the GPTB form over any tiling of its positions, every fused variant with tzgemm and every fused pair
among the four; every device form of the same lavaMD work gives the same bits as every other."""
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


def bits(t):
    return host(t).view(np.uint32)


# ----------------------------------------------------------------------------- inputs
def nn_inputs(n, seed=1):
    return np.random.default_rng(seed).uniform(0, 90, (n, 2)).astype(np.float32)


def hot3d_inputs(nx, ny, nz, seed=2):
    rng = np.random.default_rng(seed)
    return (rng.uniform(0, 0.01, (nz, ny, nx)).astype(np.float32), rng.uniform(320, 340, (nz, ny, nx)).astype(np.float32))


def path_inputs(cols, rows, seed=3):
    rng = np.random.default_rng(seed)
    return rng.integers(0, 10, (rows - 1, cols), dtype=np.int32), rng.integers(0, 10, cols, dtype=np.int32)


# ----------------------------------------------------------------------------- nn
@pytest.mark.parametrize("n", [1, 255, 256, 1000, 256 * 300 + 17])
def test_nn_forms_match_the_oracle(n):
    loc = nn_inputs(n, seed=n)
    want = oracle.nn(loc, 30.0, 90.0)
    d_loc = dev(loc)
    out = [torch.full((n,), -1.0, device="cuda:0") for _ in range(3)]
    ta.ori_nn(d_loc, out[0], 30.0, 90.0)
    ta.gptb_nn(d_loc, out[1], 30.0, 90.0)
    ta.gptb_nn(d_loc, out[2], 30.0, 90.0, launch_grid=3, launch_block=128)
    for o in out:
        assert np.array_equal(bits(o), want.view(np.uint32))
    assert ta.nn_blocks(n) == oracle.nn_blocks(n)


@pytest.mark.parametrize("seed", range(4))
def test_nn_any_tiling_of_the_positions(seed):
    rng = np.random.default_rng(100 + seed)
    n = int(rng.choice([700, 5000, 256 * 64]))
    loc = nn_inputs(n, seed=seed)
    blocks = ta.nn_blocks(n)
    cuts = sorted(set(rng.integers(0, blocks + 1, 3).tolist()) | {0, blocks})
    d_loc, out = dev(loc), torch.full((n,), -1.0, device="cuda:0")
    for a, b in zip(cuts, cuts[1:]):
        ta.gptb_nn(d_loc, out, 12.5, 40.25, a, b, launch_grid=int(rng.choice([1, 5, 64])),
                   launch_block=int(rng.choice([64, 128, 256])))
    assert np.array_equal(bits(out), oracle.nn(loc, 12.5, 40.25).view(np.uint32))
    # one position alone touches its 256 records only
    if blocks >= 3:
        out = torch.full((n,), -1.0, device="cuda:0")
        ta.gptb_nn(d_loc, out, 12.5, 40.25, 1, 2)
        want = oracle.nn(loc, 12.5, 40.25, out=np.full(n, -1.0, np.float32), start=1, end=2)
        assert np.array_equal(bits(out), want.view(np.uint32))


# ----------------------------------------------------------------------------- hot3d
@pytest.mark.parametrize("shape", [(64, 4, 2), (128, 8, 8), (192, 20, 5), (512, 64, 8)])
def test_hot3d_forms_match_the_oracle(shape):
    nx, ny, nz = shape
    p, t = hot3d_inputs(nx, ny, nz, seed=nx + ny)
    want = oracle.hot3d(p, t)
    k_dev, k_orc = ta.hot3d_coefficients(nx, ny, nz), oracle.hot3d_coefficients(nx, ny, nz)
    assert all(np.float32(k_dev[n]) == k_orc[n] for n in k_orc)
    d_p, d_t = dev(p), dev(t)
    out = [torch.full((nz, ny, nx), -1.0, device="cuda:0") for _ in range(3)]
    ta.ori_hot3d(d_p, d_t, out[0])
    ta.gptb_hot3d(d_p, d_t, out[1])
    ta.gptb_hot3d(d_p, d_t, out[2], launch_grid=5, launch_block=128)
    for o in out:
        assert np.array_equal(bits(o), want.view(np.uint32))


@pytest.mark.parametrize("seed", range(4))
def test_hot3d_any_tiling_of_the_positions(seed):
    rng = np.random.default_rng(200 + seed)
    nx, ny, nz = int(rng.choice([64, 256])), int(rng.choice([8, 36])), int(rng.choice([2, 3, 8]))
    p, t = hot3d_inputs(nx, ny, nz, seed=seed)
    blocks = ta.hot3d_blocks(nx, ny)
    cuts = sorted(set(rng.integers(0, blocks + 1, 3).tolist()) | {0, blocks})
    d_p, d_t, out = dev(p), dev(t), torch.full((nz, ny, nx), -1.0, device="cuda:0")
    for a, b in zip(cuts, cuts[1:]):
        ta.gptb_hot3d(d_p, d_t, out, a, b, launch_grid=int(rng.choice([1, 7, 64])),
                      launch_block=int(rng.choice([64, 128, 256])))
    assert np.array_equal(bits(out), oracle.hot3d(p, t).view(np.uint32))
    out = torch.full((nz, ny, nx), -1.0, device="cuda:0")
    ta.gptb_hot3d(d_p, d_t, out, blocks - 1, blocks)
    want = oracle.hot3d(p, t, out=np.full((nz, ny, nx), -1.0, np.float32), start=blocks - 1, end=blocks)
    assert np.array_equal(bits(out), want.view(np.uint32))


def test_hot3d_steps_with_exchanged_arrays():
    nx, ny, nz = 128, 16, 8
    p, t = hot3d_inputs(nx, ny, nz, seed=77)
    d_p, a, b = dev(p), dev(t), torch.zeros((nz, ny, nx), device="cuda:0")
    ref = t
    for step in range(5):
        ta.gptb_hot3d(d_p, a, b)
        ref = oracle.hot3d(p, ref)
        assert np.array_equal(bits(b), ref.view(np.uint32)), step
        a, b = b, a


# ----------------------------------------------------------------------------- path
@pytest.mark.parametrize("cols,iteration", [(1200, 125), (300, 20), (256, 127), (7, 3), (1, 1), (431, 100), (5000, 64)])
def test_path_forms_match_the_oracle(cols, iteration):
    wall, src = path_inputs(cols, iteration + 3, seed=cols)
    want = oracle.path(iteration, wall, src)
    d_w, d_s = dev(wall), dev(src)
    out = [torch.full((cols,), -1, dtype=torch.int32, device="cuda:0") for _ in range(3)]
    ta.ori_path(iteration, d_w, d_s, out[0])
    ta.gptb_path(iteration, d_w, d_s, out[1])
    ta.gptb_path(iteration, d_w, d_s, out[2], launch_grid=2, launch_block=128)
    for o in out:
        assert np.array_equal(host(o), want)
    later = torch.full((cols,), -1, dtype=torch.int32, device="cuda:0")
    ta.gptb_path(iteration, d_w, d_s, later, start_step=2)
    assert np.array_equal(host(later), oracle.path(iteration, wall, src, start_step=2))
    assert ta.path_blocks(cols, iteration) == oracle.path_blocks(cols, iteration)


@pytest.mark.parametrize("seed", range(4))
def test_path_any_tiling_of_the_positions(seed):
    rng = np.random.default_rng(300 + seed)
    cols, iteration = int(rng.choice([900, 2000])), int(rng.choice([10, 90, 120]))
    wall, src = path_inputs(cols, iteration + 1, seed=seed)
    blocks = ta.path_blocks(cols, iteration)
    cuts = sorted(set(rng.integers(0, blocks + 1, 3).tolist()) | {0, blocks})
    d_w, d_s = dev(wall), dev(src)
    out = torch.full((cols,), -1, dtype=torch.int32, device="cuda:0")
    for a, b in zip(cuts, cuts[1:]):
        ta.gptb_path(iteration, d_w, d_s, out, start=a, end=b, launch_grid=int(rng.choice([1, 3, 64])),
                     launch_block=int(rng.choice([64, 128, 256])))
    assert np.array_equal(host(out), oracle.path(iteration, wall, src))
    out = torch.full((cols,), -1, dtype=torch.int32, device="cuda:0")
    ta.gptb_path(iteration, d_w, d_s, out, start=1, end=2)
    assert np.array_equal(host(out), oracle.path(iteration, wall, src, out=np.full(cols, -1, np.int32), start=1, end=2))


def test_path_walks_a_grid_pyramid_by_pyramid():
    # Rodinia's host loop: the result of one pyramid is the source of the next
    cols, rows, height = 700, 61, 20
    wall, src = path_inputs(cols, rows, seed=5)
    d_w, a, b = dev(wall), dev(src), torch.zeros(cols, dtype=torch.int32, device="cuda:0")
    cur = src.astype(np.int64)
    for t in range(0, rows - 1, height):
        it = min(height, rows - 1 - t)
        ta.gptb_path(it, d_w, a, b, start_step=t)
        a, b = b, a
    for r in range(rows - 1):
        left, right = np.concatenate(([cur[0]], cur[:-1])), np.concatenate((cur[1:], [cur[-1]]))
        cur = wall[r] + np.minimum(np.minimum(left, cur), right)
    assert np.array_equal(host(a), cur.astype(np.int32))


# ----------------------------------------------------------------------------- lava
def lava_inputs(boxes1d, seed=4):
    rng = np.random.default_rng(seed)
    n = 100 * boxes1d ** 3
    return (rng.integers(1, 11, (n, 4)) / 10.0).astype(np.float32), (rng.integers(1, 11, n) / 10.0).astype(np.float32)


def lava_close(got, want):
    """|d| <= 2e-3 + 2e-5 |ref|: sums of up to 2700 terms of order 0.3 in fp32, the exponential from the
    hardware's 2^x here and from expf there"""
    return bool(np.all(np.abs(got.astype(np.float64) - want.astype(np.float64)) <= 2e-3 + 2e-5 * np.abs(want)))


@pytest.mark.parametrize("boxes1d", [1, 2, 3])
def test_lava_forms_match_the_oracle(boxes1d):
    rv, qv = lava_inputs(boxes1d, seed=boxes1d)
    want = oracle.lava(0.5, boxes1d, rv, qv)
    d_r, d_q = dev(rv), dev(qv)
    out = [torch.zeros((rv.shape[0], 4), device="cuda:0") for _ in range(3)]
    ta.ori_lava(0.5, d_r, d_q, out[0])
    ta.gptb_lava(0.5, d_r, d_q, out[1])
    ta.gptb_lava(0.5, d_r, d_q, out[2], launch_grid=3, launch_block=128)
    assert lava_close(host(out[0]), want)
    # a box is one wavefront's work whatever the launch: the three forms agree bit for bit
    assert np.array_equal(bits(out[1]), bits(out[0])) and np.array_equal(bits(out[2]), bits(out[0]))
    # float64 over the same neighbour lists
    boxes = oracle.lava_boxes(boxes1d)
    r, q = rv.astype(np.float64), qv.astype(np.float64)
    b = boxes[len(boxes) // 2]
    A = r[100 * b["number"]:100 * b["number"] + 100]
    pot = np.zeros(100)
    for other in [b["number"]] + b["nei"][:b["nn"]]["number"].tolist():
        B = r[100 * other:100 * other + 100]
        pot += np.exp(-0.5 * (A[:, None, 0] + B[None, :, 0] - A[:, 1:] @ B[:, 1:].T)) @ q[100 * other:100 * other + 100]
    np.testing.assert_allclose(host(out[0])[100 * b["number"]:100 * b["number"] + 100, 0], pot, rtol=2e-5)
    assert ta.lava_blocks(boxes1d) == oracle.lava_blocks(boxes1d)


def test_lava_box_list_is_the_oracles():
    for boxes1d in (1, 2, 5):
        want = oracle.lava_boxes(boxes1d)
        got = np.zeros(boxes1d ** 3, oracle.LAVA_BOX)
        assert ta.lib().tacker_lava_boxes(boxes1d, got.ctypes.data, got.nbytes) == 0
        assert got.tobytes() == want.tobytes()
    assert ta.lib().tacker_lava_boxes(2, got.ctypes.data, 100) != 0        # buffer too small


@pytest.mark.parametrize("seed", range(4))
def test_lava_any_ascending_tiling_of_the_positions(seed):
    rng = np.random.default_rng(400 + seed)
    boxes1d = int(rng.choice([2, 3]))
    rv, qv = lava_inputs(boxes1d, seed=seed)
    n = ta.lava_blocks(boxes1d)
    d_r, d_q = dev(rv), dev(qv)
    whole = torch.zeros((rv.shape[0], 4), device="cuda:0")
    ta.gptb_lava(0.5, d_r, d_q, whole)
    cuts = sorted(set(rng.integers(0, n + 1, 4).tolist()) | {0, n})
    out = torch.zeros((rv.shape[0], 4), device="cuda:0")
    for a, b in zip(cuts, cuts[1:]):
        ta.gptb_lava(0.5, d_r, d_q, out, a, b, launch_grid=int(rng.choice([1, 5, 64])),
                     launch_block=int(rng.choice([64, 128, 256])))
    assert np.array_equal(bits(out), bits(whole))
    # one position: its box's forces move, on top of what the array held, and nothing else does
    boxes = boxes1d ** 3
    base = np.full((rv.shape[0], 4), 3.0, np.float32)
    out = dev(base)
    ta.gptb_lava(0.5, d_r, d_q, out, boxes + 1, boxes + 2)          # box 1, its first neighbour
    want = oracle.lava(0.5, boxes1d, rv, qv, fv=base, start=boxes + 1, end=boxes + 2)
    got = host(out)
    assert lava_close(got, want) and np.array_equal(np.delete(got, np.s_[100:200], axis=0), np.delete(base, np.s_[100:200], axis=0))


# ----------------------------------------------------------------------------- fused with tzgemm
def _small(name):
    """(ori kernel, block positions, output tensor, oracle's output, dtype view)"""
    if name == "nn":
        loc = nn_inputs(256 * 40 + 9, seed=41)
        out = torch.full((loc.shape[0],), -1.0, device="cuda:0")
        return ta.ori_nn_create(dev(loc), out, 30.0, 90.0), ta.nn_blocks(loc.shape[0]), out, oracle.nn(loc, 30.0, 90.0)
    if name == "hot3d":
        p, t = hot3d_inputs(256, 24, 8, seed=42)
        out = torch.full((8, 24, 256), -1.0, device="cuda:0")
        return ta.ori_hot3d_create(dev(p), dev(t), out), ta.hot3d_blocks(256, 24), out, oracle.hot3d(p, t)
    if name == "lava":
        rv, qv = lava_inputs(2, seed=44)
        out = torch.full((rv.shape[0], 4), -1.0, device="cuda:0")
        return (ta.ori_lava_create(0.5, dev(rv), dev(qv), out), ta.lava_blocks(2), out,
                oracle.lava(0.5, 2, rv, qv, fv=np.full((rv.shape[0], 4), -1.0, np.float32)))
    wall, src = path_inputs(1500, 101, seed=43)
    out = torch.full((1500,), -1, dtype=torch.int32, device="cuda:0")
    return (ta.ori_path_create(100, dev(wall), dev(src), out), ta.path_blocks(1500, 100), out,
            oracle.path(100, wall, src))


def _same(t, want):
    """the oracle's bits; for lava (float32 [n][4] sums) the stated tolerance"""
    if t.dtype == torch.float32 and t.dim() == 2:
        return lava_close(host(t), want)
    return np.array_equal(host(t).view(np.uint32), np.ascontiguousarray(want).view(np.uint32))


@pytest.mark.parametrize("be", ["nn", "hot3d", "path", "lava"])
@pytest.mark.parametrize("variant", [None, "wave_256", "wave_512", "wg_1_1", "wg_1_2"])
def test_mix_with_tzgemm(be, variant):
    M, N, K = 256, 256, 256
    A, B = gemm_inputs(M, N, K, seed=51)
    a, b = dev(A), dev(B)
    solo_c = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(a, b, solo_c)
    ori, n, out, want = _small(be)
    mix_c = torch.zeros((M, N), device="cuda:0")
    g_be = ta.gptb_create(ori, 0, 0, 0, n)
    g_tz = ta.gptb_create(ta.ori_tzgemm_create(a, b, mix_c), 0, 0, 0, 16)
    ta.mix_create(g_be, g_tz, 0, n, 0, 16, variant=variant).execute()
    assert _same(out, want)
    first_bits = bits(out).copy()
    assert np.array_equal(host(mix_c), host(solo_c))
    ok, fro, dmax = gemm_tolerance_ok(host(mix_c), oracle.tzgemm(A, B, f64=True), K)
    assert ok and fro <= 1e-5
    # a slice of the positions rides with a slice of the tiles, the rest follows in a second fused launch
    out.fill_(-1)
    mix_c.zero_()
    cut = max(1, n // 3)
    ta.mix_create(g_be, g_tz, 0, cut, 0, 5, variant=variant).execute()
    ta.mix_create(g_be, g_tz, cut, n, 5, 16, variant=variant).execute()
    assert _same(out, want) and np.array_equal(bits(out), first_bits)      # the same bits however the range is cut
    assert np.array_equal(host(mix_c), host(solo_c))
    assert ta.spin_fail_flag() == 0


RODINIA_PAIRS = [("hot3d", "nn"), ("hot3d", "path"), ("nn", "path"), ("hot3d", "lava"), ("lava", "nn"), ("lava", "path")]


@pytest.mark.parametrize("first,second", RODINIA_PAIRS)
@pytest.mark.parametrize("variant", [None, "wg_1_1", "wg_1_2", "wg_2_1", "ord_1_1", "ord_1_2", "ord_2_1"])
def test_pairs_among_the_three(first, second, variant):
    ori1, n1, out1, want1 = _small(first)
    ori2, n2, out2, want2 = _small(second)
    g1, g2 = ta.gptb_create(ori1, 0, 0, 0, n1), ta.gptb_create(ori2, 0, 0, 0, n2)
    ta.be_pair_create(g1, g2, 0, n1, 0, n2, variant=variant, launch_grid=48).execute()
    assert _same(out1, want1) and _same(out2, want2)
    # partial ranges: what the unfused GPTB launches of the same ranges write
    out1.fill_(-1)
    out2.fill_(-1)
    ta.be_pair_create(g1, g2, 1, n1 - 1, 0, n2 // 2, variant=variant, launch_grid=48).execute()
    got = [host(out1).copy(), host(out2).copy()]
    out1.fill_(-1)
    out2.fill_(-1)
    ta.gptb_create(ori1, 0, 0, 1, n1 - 1).execute()
    ta.gptb_create(ori2, 0, 0, 0, n2 // 2).execute()
    assert np.array_equal(got[0].view(np.uint32), bits(out1)) and np.array_equal(got[1].view(np.uint32), bits(out2))
    assert ta.spin_fail_flag() == 0


def test_create_mix_kernel_knows_the_reference_pairs():
    # src/Creator.cu:554-640
    for name in ("hot3d_nn", "hot3d_path", "nn_path", "hot3d_lava", "lava_nn", "lava_path"):
        assert ta.lib().tacker_get_kernel_info(name.encode(), b"blocksize") == 256
    for name in ("cp_nn", "hot3d_lbm", "path_stencil"):
        assert ta.lib().tacker_get_kernel_info(name.encode(), b"blocksize") == -32767


# ----------------------------------------------------------------------------- the Creator's instances
def _fill_hash(i, seed):
    i = np.asarray(i, np.uint64)
    x = (i & np.uint64(0xFFFFFFFF)).astype(np.uint32) ^ ((i >> np.uint64(32)).astype(np.uint32) * np.uint32(0x9E3779B9)) ^ np.uint32(seed)
    x ^= x >> np.uint32(16)
    x *= np.uint32(0x7FEB352D)
    x ^= x >> np.uint32(15)
    x *= np.uint32(0x846CA68B)
    x ^= x >> np.uint32(16)
    return x


def _fill_uniform(i, seed, lo, hi):
    u = (_fill_hash(i, seed) >> np.uint32(8)).astype(np.float32) * np.float32(1.0 / 16777216.0)
    return np.float32(lo) + (np.float32(hi) - np.float32(lo)) * u


def test_creator_nn_is_the_references_record_count():
    k = ta.create_kernel("nn")
    info = k.info()
    n = 256 * 2560000
    assert (info["ptb_start"], info["ptb_end"], info["ori_grid_x"]) == (0, 2560000, 2560000)
    k.execute()
    torch.cuda.synchronize()
    for first in (0, 256 * 1234567, n - 4096):
        loc = ta.device_to_host(k.param(0) + 8 * first, (4096, 2), np.float32)
        assert np.array_equal(loc.reshape(-1), _fill_uniform(np.arange(2 * first, 2 * first + 8192), 4001, 0.0, 90.0))
        got = ta.device_to_host(k.param(1) + 4 * first, (4096,), np.float32)
        assert np.array_equal(got.view(np.uint32), oracle.nn(loc, 30.0, 90.0).view(np.uint32))
    assert ta.spin_fail_flag() == 0


def test_creator_hot3d_is_the_references_chip():
    k = ta.create_kernel("hot3d")
    info = k.info()
    nx, ny, nz = 16384, 8192, 8
    assert (info["ptb_end"], info["ori_grid_x"], info["ori_grid_y"]) == (256 * 2048, 256, 2048)
    k.execute()
    torch.cuda.synchronize()
    # the chip's first rows, all layers: nine rows of input give eight rows of output
    rows = 9
    plane = nx * ny
    p = np.stack([ta.device_to_host(k.param(0) + 4 * plane * z, (rows, nx), np.float32) for z in range(nz)])
    t = np.stack([ta.device_to_host(k.param(1) + 4 * plane * z, (rows, nx), np.float32) for z in range(nz)])
    idx = (np.arange(nz)[:, None, None] * plane + np.arange(rows)[None, :, None] * nx + np.arange(nx)[None, None, :])
    assert np.array_equal(t, _fill_uniform(idx, 4101, 320.0, 340.0))
    assert np.array_equal(p, _fill_uniform(idx, 4102, 0.0, 0.01))
    got = np.stack([ta.device_to_host(k.param(2) + 4 * plane * z, (rows - 1, nx), np.float32) for z in range(nz)])
    coeff = oracle.hot3d_coefficients(nx, ny, nz)
    want = oracle.hot3d(p, t, coeff=coeff)[:, :rows - 1]     # the slab's last row has another southern neighbour on the chip
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert ta.spin_fail_flag() == 0


def test_creator_path_is_the_references_grid():
    k = ta.create_kernel("path")
    info = k.info()
    assert (info["ptb_start"], info["ptb_end"], info["ori_grid_x"]) == (0, 200, 200)
    k.execute()
    torch.cuda.synchronize()
    grid = oracle.path_source(126, 1200)              # rand() % 10 after srand(9): source row and 125 wall rows
    assert np.array_equal(ta.device_to_host(k.param(2), (1200,), np.int32), grid[0])
    assert np.array_equal(ta.device_to_host(k.param(1), (125, 1200), np.int32), grid[1:])
    got = ta.device_to_host(k.param(3), (1200,), np.int32)
    assert np.array_equal(got, oracle.path(125, grid[1:], grid[0]))
    assert ta.spin_fail_flag() == 0


def test_creator_lava_is_the_references_system():
    k = ta.create_kernel("lava")
    info = k.info()
    boxes = 60 ** 3
    assert (info["ptb_start"], info["ptb_end"], info["ori_grid_x"]) == (0, boxes * 27, boxes)
    # a slice of the launch: the first 2048 boxes against themselves and their first neighbour
    n = 2048
    lib = ta.lib()
    fv_ptr, rv_ptr, qv_ptr = k.param(5), k.param(3), k.param(4)
    assert lib.tkMemset(fv_ptr, 0, 16 * 100 * n) == 0
    k.set_range(0, n)
    k.execute()
    k.set_range(boxes, boxes + n)
    k.execute()
    torch.cuda.synchronize()
    k.set_range(0, boxes * 27)
    rv = ta.device_to_host(rv_ptr, (100 * 60 * 60 * 2, 4), np.float32)          # the first two layers of boxes
    qv = ta.device_to_host(qv_ptr, (100 * 60 * 60 * 2,), np.float32)
    assert np.array_equal(rv.reshape(-1), _fill_uniform(np.arange(rv.size), 4301, 0.1, 1.0))
    assert np.array_equal(qv, _fill_uniform(np.arange(qv.size), 4302, 0.1, 1.0))
    got = ta.device_to_host(fv_ptr, (100 * n, 4), np.float32)
    box_list = np.zeros(boxes, oracle.LAVA_BOX)
    assert lib.tacker_lava_boxes(60, box_list.ctypes.data, box_list.nbytes) == 0
    r, q = rv.astype(np.float64), qv.astype(np.float64)
    for b in (0, 59, 60, 1000, n - 1):
        A = r[100 * b:100 * b + 100]
        pot = np.zeros(100)
        for other in (b, int(box_list[b]["nei"][0]["number"])):
            B = r[100 * other:100 * other + 100]
            pot += np.exp(-0.5 * (A[:, None, 0] + B[None, :, 0] - A[:, 1:] @ B[:, 1:].T)) @ q[100 * other:100 * other + 100]
        np.testing.assert_allclose(got[100 * b:100 * b + 100, 0], pot, rtol=2e-5)
    assert ta.spin_fail_flag() == 0


def test_task_manager_colocates_the_rodinia_kernels():
    # nn and hotspot3D blocks ride with VGG16's layers (tzgemm_nn, tzgemm_hot3d), the nn_path pair
    # (src/mix_kernel/nn_path.cu) runs in the second stage; the query's logits stay the solo query's bits
    task = ta.LcTask("vgg16", 64, 64)
    task.execute()
    torch.cuda.synchronize()
    p, stride, n = task.logits()
    solo_logits = ta.device_to_host(p, (n, stride), np.float32)[:, 0].copy()
    tm = ta.TaskManager(task, "nn", "path")
    tm.configure(qos_budget_ms=50.0, guard_ms=0.5, warmup=1, profile=3, queries=3, verbose=0)
    rep = tm.run("aker", second_stage=True)
    torch.cuda.synchronize()
    assert np.array_equal(ta.device_to_host(p, (n, stride), np.float32)[:, 0], solo_logits)
    assert rep["mixable_times"] == 16 and rep["be1_solo_ms"] > 0 and rep["n_colocated"] == 3
    tm.close()
    tm = ta.TaskManager(task, "hot3d", None)
    tm.configure(qos_budget_ms=50.0, guard_ms=0.5, warmup=1, profile=3, queries=3, verbose=0)
    rep = tm.run("aker", second_stage=False)
    torch.cuda.synchronize()
    assert np.array_equal(ta.device_to_host(p, (n, stride), np.float32)[:, 0], solo_logits)
    assert rep["n_colocated"] == 3 and ta.spin_fail_flag() == 0
    tm.close()
    with pytest.raises(ta.TackerError, match="no fused kernel"):
        ta.TaskManager(task, "nn", "stencil")
    task.close()


def test_bad_arguments_are_refused():
    lib = ta.lib()
    loc, out = dev(nn_inputs(10)), torch.zeros(10, device="cuda:0")
    rv = torch.zeros((100, 4), device="cuda:0")
    assert lib.tacker_ori_lava(0.5, 1, rv.data_ptr(), rv.data_ptr(), rv.data_ptr(), None) == 1       # in place
    assert lib.tacker_ori_lava(0.5, 0, rv.data_ptr(), rv.data_ptr(), out.data_ptr(), None) != 0
    assert lib.tacker_ori_nn(None, out.data_ptr(), 10, 1.0, 1.0, None) == 1
    assert lib.tacker_ori_nn(loc.data_ptr(), out.data_ptr(), 0, 1.0, 1.0, None) == 1
    t = torch.zeros((2, 4, 64), device="cuda:0")
    o = torch.zeros_like(t)
    assert lib.tacker_ori_hot3d(t.data_ptr(), t.data_ptr(), t.data_ptr(), 64, 4, 2, None) == 1      # in place
    assert lib.tacker_ori_hot3d(t.data_ptr(), t.data_ptr(), o.data_ptr(), 60, 4, 2, None) != 0      # nx % 64
    assert lib.tacker_ori_hot3d(t.data_ptr(), t.data_ptr(), o.data_ptr(), 64, 4, 1, None) != 0      # one layer
    w, s = dev(np.zeros((3, 8), np.int32)), dev(np.zeros(8, np.int32))
    r = torch.zeros(8, dtype=torch.int32, device="cuda:0")
    assert lib.tacker_ori_path(0, w.data_ptr(), s.data_ptr(), r.data_ptr(), 8, 4, 0, None) != 0     # no rows
    assert lib.tacker_ori_path(128, w.data_ptr(), s.data_ptr(), r.data_ptr(), 8, 400, 0, None) != 0   # pyramid too high
    assert lib.tacker_ori_path(3, w.data_ptr(), s.data_ptr(), r.data_ptr(), 8, 4, 1, None) != 0     # past the wall
    assert lib.tacker_ori_path(3, w.data_ptr(), s.data_ptr(), s.data_ptr(), 8, 4, 0, None) == 1     # in place
