"""Pins oracle.mriq*, oracle.cp*, oracle.im2col, oracle.gptb_index."""
import ctypes

import numpy as np
import pytest

import oracle


# ------------------------------------------------------------------ mri-q
def mriq_inputs(numK, numX, seed=11):
    rng = np.random.default_rng(seed)
    k = rng.uniform(-0.5, 0.5, (numK, 3)).astype(np.float32)
    phiR = rng.uniform(0, 1, numK).astype(np.float32)
    phiI = rng.uniform(0, 1, numK).astype(np.float32)
    xyz = rng.uniform(-0.5, 0.5, (3, numX)).astype(np.float32)
    return k, phiR, phiI, xyz


def test_phimag_closed_form():
    _, phiR, phiI, _ = mriq_inputs(64, 256)
    got = oracle.mriq_phimag(phiR, phiI)
    np.testing.assert_allclose(got, phiR.astype(np.float64) ** 2 + phiI.astype(np.float64) ** 2, rtol=1e-6)
    assert oracle.mriq_phimag(np.array([3.0], np.float32), np.array([4.0], np.float32))[0] == 25.0


def test_origin_voxel_sums_phimag():
    k, phiR, phiI, xyz = mriq_inputs(128, 256)
    kv = np.concatenate([k, oracle.mriq_phimag(phiR, phiI)[:, None]], 1)
    zero = np.zeros(256, np.float32)
    qr, qi = oracle.mriq(kv, zero, zero, zero, zero, zero)
    np.testing.assert_allclose(qr, kv[:, 3].astype(np.float64).sum(), rtol=1e-5)
    assert np.all(qi == 0)


@pytest.mark.parametrize("f64", [False, True])
def test_matches_numpy_float64_and_accumulates(f64):
    numK, numX = 96, 512
    k, phiR, phiI, xyz = mriq_inputs(numK, numX)
    kv = np.concatenate([k, oracle.mriq_phimag(phiR, phiI)[:, None]], 1).astype(np.float32)
    q0r = np.full(numX, 2.0, np.float32)
    q0i = np.full(numX, -1.0, np.float32)
    qr, qi = oracle.mriq(kv, xyz[0], xyz[1], xyz[2], q0r, q0i, f64=f64)
    arg = 2 * np.pi * (kv[:, :3].astype(np.float64) @ xyz.astype(np.float64))   # [numK][numX]
    want_r = 2.0 + (kv[:, 3:4].astype(np.float64) * np.cos(arg)).sum(0)
    want_i = -1.0 + (kv[:, 3:4].astype(np.float64) * np.sin(arg)).sum(0)
    tol = 1e-6 if f64 else 2e-4
    np.testing.assert_allclose(qr, want_r, rtol=tol, atol=tol)
    np.testing.assert_allclose(qi, want_i, rtol=tol, atol=tol)


def test_single_k_is_one_cos_and_sin():
    kv = np.array([[0.25, 0.0, 0.0, 2.0]], np.float32)
    x = np.full(256, 0.5, np.float32)
    zero = np.zeros(256, np.float32)
    qr, qi = oracle.mriq(kv, x, zero, zero, zero, zero)
    # arg = 2*pi*0.125 = pi/4
    np.testing.assert_allclose(qr, 2.0 * np.sqrt(0.5), rtol=1e-6)
    np.testing.assert_allclose(qi, 2.0 * np.sqrt(0.5), rtol=1e-6)


def test_mriq_block_range():
    numK, numX = 32, 1024
    k, phiR, phiI, xyz = mriq_inputs(numK, numX)
    kv = np.concatenate([k, oracle.mriq_phimag(phiR, phiI)[:, None]], 1).astype(np.float32)
    z = np.zeros(numX, np.float32)
    fr, fi = oracle.mriq(kv, *xyz, z, z)
    pr, pi = oracle.mriq(kv, *xyz, z, z, start=1, end=3)
    assert np.array_equal(pr[256:768], fr[256:768]) and np.all(pr[:256] == 0) and np.all(pr[768:] == 0)
    assert np.array_equal(pi[256:768], fi[256:768])
    # fusion/code/kinfo.json "mriq.ori_blks" = 819 = floor(209715 / 256)
    assert (2097152 // 10) // 256 == 819


def test_mriq_positions_of_the_block_by_chunk_grid():
    # 300 records in chunks of 128 (128, 128, 44) over 4 voxel blocks: 12 positions
    numK, numX = 300, 1024
    k, phiR, phiI, xyz = mriq_inputs(numK, numX)
    kv = np.concatenate([k, oracle.mriq_phimag(phiR, phiI)[:, None]], 1).astype(np.float32)
    q0 = np.linspace(-1, 1, numX).astype(np.float32)
    whole = oracle.mriq(kv, *xyz, q0, q0)
    # all positions = the one k loop, bit for bit (a float carried through memory is unchanged)
    grid = oracle.mriq(kv, *xyz, q0, q0, kchunk=128)
    assert np.array_equal(grid[0], whole[0]) and np.array_equal(grid[1], whole[1])
    # and so is any ascending tiling of the positions
    for tiling in ([(0, 3), (3, 5), (5, 11), (11, 12)], [(0, 4), (4, 8), (8, 12)], [(i, i + 1) for i in range(12)]):
        qr, qi = q0, q0
        for a, b in tiling:
            qr, qi = oracle.mriq(kv, *xyz, qr, qi, start=a, end=b, kchunk=128)
        assert np.array_equal(qr, whole[0]) and np.array_equal(qi, whole[1]), tiling
    # position 6 = chunk 1 onto voxel block 2: records 128..255 only, voxels 512..767 only (numpy, float64)
    qr, qi = oracle.mriq(kv, *xyz, q0, q0, start=6, end=7, kchunk=128, f64=True)
    sel = slice(512, 768)
    phase = 2 * np.pi * (kv[128:256, 0:1].astype(np.float64) * xyz[0][sel] + kv[128:256, 1:2].astype(np.float64) * xyz[1][sel]
                         + kv[128:256, 2:3].astype(np.float64) * xyz[2][sel])
    want_r = q0[sel] + (kv[128:256, 3:4].astype(np.float64) * np.cos(phase)).sum(axis=0)
    want_i = q0[sel] + (kv[128:256, 3:4].astype(np.float64) * np.sin(phase)).sum(axis=0)
    np.testing.assert_allclose(qr[sel], want_r, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(qi[sel], want_i, rtol=1e-6, atol=1e-6)
    rest = np.r_[0:512, 768:1024]
    assert np.array_equal(qr[rest], q0[rest]) and np.array_equal(qi[rest], q0[rest])
    # the last chunk is the short one: position 11 adds records 256..299 to voxel block 3
    qr, _ = oracle.mriq(kv, *xyz, q0, q0, start=11, end=12, kchunk=128, f64=True)
    only_tail, _ = oracle.mriq(kv[256:], *xyz, q0, q0, start=3, end=4, f64=True)
    assert np.array_equal(qr, only_tail)
    # positions past the grid wrap: chunk (p // 4) % 3, block p % 4
    twice = oracle.mriq(kv, *xyz, q0, q0, start=0, end=24, kchunk=128)
    again = oracle.mriq(kv, *xyz, *whole, kchunk=128)
    assert np.array_equal(twice[0], again[0]) and np.array_equal(twice[1], again[1])


# ------------------------------------------------------------------ cp
def test_initatoms_matches_glibc_stream_and_box():
    atoms = oracle.cp_initatoms(count=100)
    libc = ctypes.CDLL("libc.so.6")
    libc.srand(54321)
    r = np.array([libc.rand() for _ in range(400)], np.int64).reshape(100, 4)
    u = (r.astype(np.float32) / np.float32(2147483647.0))
    assert np.array_equal(atoms[:, 0], u[:, 0] * np.float32(409))     # (unsigned)(0.1f*4096) = 409
    assert np.array_equal(atoms[:, 1], u[:, 1] * np.float32(409))
    assert np.all(atoms[:, 2] == 0)                                   # (unsigned)(0.1f*1) = 0
    assert np.array_equal(atoms[:, 3], (u[:, 3].astype(np.float64) * 2.0 - 1.0).astype(np.float32))
    assert atoms[:, :2].min() >= 0 and atoms[:, :2].max() <= 409
    assert atoms[:, 3].min() >= -1 and atoms[:, 3].max() <= 1 and atoms[:, 3].std() > 0.3


def test_atoms_to_const_squares_dz():
    atoms = np.array([[1, 2, 3, 0.5], [4, 5, -1, -0.25]], np.float32)
    got = oracle.cp_atoms_to_const(atoms, zplane=1.0)
    assert np.array_equal(got, np.array([[1, 2, 4, 0.5], [4, 5, 4, -0.25]], np.float32))


def test_cp_single_atom_closed_form_and_accumulate():
    atominfo = np.array([[3.3, 1.7, 0.49, -0.5]], np.float32)
    grid0 = np.full((16, 256), 1.0, np.float32)
    got = oracle.cp(atominfo, grid0, gridspacing=0.1)
    yy, xx = np.meshgrid(np.arange(16), np.arange(256), indexing="ij")
    r = np.sqrt((0.1 * xx - 3.3) ** 2 + (0.1 * yy - 1.7) ** 2 + 0.49)
    np.testing.assert_allclose(got, 1.0 - 0.5 / r, rtol=2e-5)


def test_cp_matches_float64_brute_force_and_ranges():
    atoms = oracle.cp_initatoms(count=70)
    atominfo = oracle.cp_atoms_to_const(atoms[1:65], 0.0)              # atoms+4, 64 atoms: cp_kernel.cu:301-314
    atominfo[:, 2] += np.float32(0.01)                                 # keep r > 0
    H, Wd = 24, 384
    got = oracle.cp(atominfo, np.zeros((H, Wd), np.float32))
    yy, xx = np.meshgrid(np.arange(H), np.arange(Wd), indexing="ij")
    want = np.zeros((H, Wd))
    a = atominfo.astype(np.float64)
    for n in range(64):
        want += a[n, 3] / np.sqrt((0.1 * xx - a[n, 0]) ** 2 + (0.1 * yy - a[n, 1]) ** 2 + a[n, 2])
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5)
    gdx, gdy = Wd // 128, H // 8
    acc = np.zeros((H, Wd), np.float32)
    for s, e in [(0, 4), (4, 5), (5, gdx * gdy)]:
        acc = oracle.cp(atominfo, acc, start=s, end=e)
    assert np.array_equal(acc, got)
    # fusion/code/kinfo.json "cp.ori_blks" = 16384 = (4096/128)*(4096/8)
    assert (4096 // 128) * (4096 // 8) == 16384


def test_cp_positions_of_the_block_by_x_part_grid():
    atoms = oracle.cp_initatoms(count=70)
    atominfo = oracle.cp_atoms_to_const(atoms[1:65], 0.0)
    atominfo[:, 2] += np.float32(0.01)
    H, Wd = 16, 384                                                    # 3 x 2 blocks, 4 parts: 24 positions
    g0 = np.random.default_rng(8).uniform(-1, 1, (H, Wd)).astype(np.float32)
    whole = oracle.cp(atominfo, g0)
    # all positions, and any tiling of them, store the bits of the whole-block form
    assert np.array_equal(oracle.cp(atominfo, g0, parts=4), whole)
    for tiling in ([(0, 5), (5, 7), (7, 19), (19, 24)], [(0, 6), (6, 12), (12, 18), (18, 24)],
                   [(i, i + 1) for i in range(24)], [(13, 24), (0, 13)]):
        acc = g0
        for a, b in tiling:
            acc = oracle.cp(atominfo, acc, start=a, end=b, parts=4)
        assert np.array_equal(acc, whole), tiling
    # position 6 + 2 = part 1 of block 2 (bx 2, by 0): columns 256 + {32..63} of rows 0..7, nothing else
    one = oracle.cp(atominfo, g0, start=8, end=9, parts=4)
    touched = np.zeros((H, Wd), bool)
    touched[0:8, 256 + 32:256 + 64] = True
    assert np.array_equal(one[touched], whole[touched]) and np.array_equal(one[~touched], g0[~touched])
    # points of part 3 against float64 directly (their dx comes out of six chained additions)
    last = oracle.cp(atominfo, np.zeros((H, Wd), np.float32), start=18, end=24, parts=4)
    yy, xx = np.meshgrid(np.arange(H), np.arange(Wd), indexing="ij")
    a = atominfo.astype(np.float64)
    want = sum(a[n, 3] / np.sqrt((0.1 * xx - a[n, 0]) ** 2 + (0.1 * yy - a[n, 1]) ** 2 + a[n, 2]) for n in range(64))
    part3 = (xx % 128) >= 96
    np.testing.assert_allclose(last[part3], want[part3], rtol=1e-4, atol=1e-5)
    assert np.all(last[~part3] == 0)
    # past the grid the positions come round again and add a second time
    twice = oracle.cp(atominfo, g0, start=0, end=48, parts=4)
    assert np.array_equal(twice, oracle.cp(atominfo, whole, parts=4))


# ------------------------------------------------------------------ conv helpers
def test_mnk_known_answers_vgg16():
    # VGG16 batch 1, 224x224: conv1_1 3->64, conv1_2 64->64, conv5 512->512 at 14x14
    assert oracle.mnk_from_conv_args([1, 3, 224, 224, 64, 3, 3, 3, 1, 1, 1, 1, 1, 1]) == [50176, 64, 27]
    assert oracle.mnk_from_conv_args([1, 64, 224, 224, 64, 64, 3, 3, 1, 1, 1, 1, 1, 1]) == [50176, 64, 576]
    assert oracle.mnk_from_conv_args([32, 512, 14, 14, 512, 512, 3, 3, 1, 1, 1, 1, 1, 1]) == [6272, 512, 4608]
    # stride 2, no pad, 7x7 (the comment in src/TaskManager.cu:115-117: 112x112, 7*7*3)
    assert oracle.mnk_from_conv_args([1, 3, 229, 229, 64, 3, 7, 7, 0, 0, 2, 2, 1, 1]) == [112 * 112, 64, 147]


@pytest.mark.parametrize("pad,stride,dil", [((1, 1), (1, 1), (1, 1)), ((0, 1), (2, 1), (1, 1)),
                                             ((2, 2), (1, 2), (2, 1))])
def test_im2col_times_weights_is_direct_convolution(pad, stride, dil):
    rng = np.random.default_rng(12)
    Cin, H, Wd, Cout, kh, kw = 3, 8, 9, 4, 3, 3
    im = rng.uniform(-1, 1, (Cin, H, Wd)).astype(np.float32)
    wt = rng.uniform(-1, 1, (Cout, Cin, kh, kw)).astype(np.float32)
    col = oracle.im2col(im, (kh, kw), pad, stride, dil)
    _, Ho, Wo = col.shape
    got = (wt.reshape(Cout, -1).astype(np.float64) @ col.reshape(Cin * kh * kw, -1)).reshape(Cout, Ho, Wo)
    padded = np.zeros((Cin, H + 2 * pad[0], Wd + 2 * pad[1]))
    padded[:, pad[0]:pad[0] + H, pad[1]:pad[1] + Wd] = im
    want = np.zeros((Cout, Ho, Wo))
    for o in range(Cout):
        for y in range(Ho):
            for x in range(Wo):
                for c in range(Cin):
                    for i in range(kh):
                        for j in range(kw):
                            want[o, y, x] += wt[o, c, i, j] * padded[c, y * stride[0] + i * dil[0],
                                                                     x * stride[1] + j * dil[1]]
    np.testing.assert_allclose(got, want, atol=1e-6)


# ------------------------------------------------------------------ GPTB index
def test_gptb_index_partition_and_wrap():
    gdx, gdy, bdx, bdy = 5, 3, 16, 8
    seen = {}
    for pos in range(gdx * gdy):
        bx, by, _, _ = oracle.gptb_index(pos, 0, gdx, gdy, bdx, bdy)
        seen[(bx, by)] = seen.get((bx, by), 0) + 1
    assert len(seen) == gdx * gdy and set(seen.values()) == {1}
    assert oracle.gptb_index(gdx * gdy + 7, 0, gdx, gdy, bdx, bdy)[:2] == oracle.gptb_index(7, 0, gdx, gdy, bdx, bdy)[:2]
    threads = {oracle.gptb_index(0, t, gdx, gdy, bdx, bdy)[2:] for t in range(bdx * bdy)}
    assert threads == {(x, y) for x in range(bdx) for y in range(bdy)}
    assert oracle.gptb_index(0, 17, gdx, gdy, bdx, bdy)[2:] == (1, 1)
