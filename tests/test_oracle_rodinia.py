"""Pins of the CPU restatements of the Rodinia partners (nn, hotspot3D, pathfinder): closed forms,
invariants, independent numpy formulations and brute force on tiny cases."""
import itertools

import numpy as np
import pytest

import oracle


# ----------------------------------------------------------------------------- nn
def test_nn_known_answers_and_float64():
    loc = np.array([[3.0, 4.0], [0.0, 0.0], [1.0, 0.0], [0.0, -2.5], [30.0, 90.0]], np.float32)
    d = oracle.nn(loc, 0.0, 0.0)
    assert d.tolist() == [5.0, 0.0, 1.0, 2.5, np.float32(np.sqrt(np.float32(900.0 + 8100.0)))]
    rng = np.random.default_rng(1)
    loc = rng.uniform(0, 90, (1000, 2)).astype(np.float32)
    d = oracle.nn(loc, 30.0, 90.0)
    ref = np.hypot(30.0 - loc[:, 0].astype(np.float64), 90.0 - loc[:, 1].astype(np.float64))
    np.testing.assert_allclose(d, ref, rtol=3e-7)
    # the same three float32 roundings, vectorised (numpy's float32 sqrt is correctly rounded)
    dl, dg = np.float32(30.0) - loc[:, 0], np.float32(90.0) - loc[:, 1]
    assert np.array_equal(d, np.sqrt(dl * dl + dg * dg))
    # a swapped component or a dropped square would show here
    assert oracle.nn(np.array([[1.0, 7.0]], np.float32), 1.0, 3.0)[0] == 4.0
    assert oracle.nn(np.array([[7.0, 1.0]], np.float32), 3.0, 1.0)[0] == 4.0


def test_nn_positions_tail_and_wrap():
    rng = np.random.default_rng(2)
    n = 256 * 5 + 77                                    # the last block is partly past the records
    loc = rng.uniform(0, 90, (n, 2)).astype(np.float32)
    whole = oracle.nn(loc, 10.0, 20.0)
    assert oracle.nn_blocks(n) == 6 and oracle.nn_blocks(256) == 1 and oracle.nn_blocks(257) == 2
    # any tiling of the positions gives the one-launch result
    out = np.full(n, -1.0, np.float32)
    for a, b in ((4, 6), (0, 1), (1, 4)):
        out = oracle.nn(loc, 10.0, 20.0, out=out, start=a, end=b)
    assert np.array_equal(out, whole)
    # one position = its 256 records and nothing else
    one = oracle.nn(loc, 10.0, 20.0, out=np.full(n, -1.0, np.float32), start=2, end=3)
    assert np.array_equal(one[512:768], whole[512:768]) and (one[:512] == -1).all() and (one[768:] == -1).all()
    # a grid folded over y: position p is block (p % gx, (p / gx) % gy), record base 256 (gx by + bx)
    folded = oracle.nn(loc, 10.0, 20.0, grid=(2, 3))
    assert np.array_equal(folded, whole)
    # positions past the grid wrap onto it
    again = oracle.nn(loc, 10.0, 20.0, out=np.full(n, -1.0, np.float32), start=6 + 2, end=6 + 3)
    assert np.array_equal(again, one)


# ----------------------------------------------------------------------------- hot3d
def _hot3d_numpy(p, t, k, dtype):
    """Edge-padded formulation: neighbours by slicing a padded array, same term order."""
    t = t.astype(dtype)
    pad = np.pad(t, 1, mode="edge")
    c = {n: dtype(v) for n, v in k.items()}
    out = c["cc"] * t
    out = out + c["cw"] * pad[1:-1, 1:-1, :-2]
    out = out + c["ce"] * pad[1:-1, 1:-1, 2:]
    out = out + c["cs"] * pad[1:-1, 2:, 1:-1]
    out = out + c["cn"] * pad[1:-1, :-2, 1:-1]
    out = out + c["cb"] * pad[:-2, 1:-1, 1:-1]
    out = out + c["ct"] * pad[2:, 1:-1, 1:-1]
    out = out + c["sdc"] * p.astype(dtype)
    out = out + c["ct"] * dtype(80.0)
    return out


def test_hot3d_coefficients_follow_rodinia_formulas():
    nx, ny, nz = 512, 512, 8
    k = oracle.hot3d_coefficients(nx, ny, nz)
    # float64 evaluation of the same physics: dx = height / rows, Cap = 0.5 * 1.75e6 * t * dx * dy, ...
    t_chip, h, w = 0.0005, 0.016, 0.016
    dx, dy, dz = h / ny, w / nx, t_chip / nz
    cap = 0.5 * 1.75e6 * t_chip * dx * dy
    rx, ry, rz = dy / (2 * 100 * t_chip * dx), dx / (2 * 100 * t_chip * dy), dz / (100 * dx * dy)
    dt = 0.001 / (3.0e6 / (0.5 * t_chip * 1.75e6))
    want = {"sdc": dt / cap, "ce": dt / cap / rx, "cn": dt / cap / ry, "ct": dt / cap / rz}
    for name, v in want.items():
        assert k[name] == pytest.approx(v, rel=2e-6), name
    assert k["cw"] == k["ce"] and k["cs"] == k["cn"] and k["cb"] == k["ct"]
    assert k["cc"] == pytest.approx(1 - (2 * want["ce"] + 2 * want["cn"] + 3 * want["ct"]), rel=2e-6)
    # a stable explicit step: all weights positive and they sum to 1 - ct (the top face's exchange)
    assert all(v > 0 for v in k.values())
    assert 2 * k["ce"] + 2 * k["cn"] + 2 * k["ct"] + k["cc"] == pytest.approx(1 - k["ct"], rel=1e-6)


def test_hot3d_closed_forms():
    nx, ny, nz = 64, 8, 5
    k = oracle.hot3d_coefficients(nx, ny, nz)
    zero = np.zeros((nz, ny, nx), np.float32)
    # the ambient temperature without power is a fixed point
    amb = np.full((nz, ny, nx), 80.0, np.float32)
    np.testing.assert_allclose(oracle.hot3d(zero, amb), 80.0, rtol=1e-6)
    # a constant field: every cell T (1 - ct) + ct 80, edges and corners included
    t = np.full((nz, ny, nx), 330.0, np.float32)
    np.testing.assert_allclose(oracle.hot3d(zero, t), 330.0 * (1 - float(k["ct"])) + float(k["ct"]) * 80.0, rtol=1e-6)
    # power alone adds sdc * p
    p = np.random.default_rng(3).uniform(0, 1, (nz, ny, nx)).astype(np.float32)
    np.testing.assert_allclose(oracle.hot3d(p, amb) - 80.0, float(k["sdc"]) * p, rtol=1e-3, atol=1e-4)
    # symmetric weights and insulated faces: the step keeps sum(T) but for the ambient term,
    # sum(out) = sum(T) - ct sum(T) + ct 80 cells
    t = np.random.default_rng(4).uniform(320, 340, (nz, ny, nx)).astype(np.float32)
    out = oracle.hot3d(zero, t).astype(np.float64)
    want = t.astype(np.float64).sum() * (1 - float(k["ct"])) + float(k["ct"]) * 80.0 * t.size
    assert out.sum() == pytest.approx(want, rel=1e-7)


def test_hot3d_against_padded_numpy_and_tilings():
    rng = np.random.default_rng(5)
    nx, ny, nz = 128, 12, 4
    k = {n: np.float32(v) for n, v in zip(("sdc", "ce", "cw", "cn", "cs", "ct", "cb", "cc"),
                                          (0.3, 0.11, 0.07, 0.05, 0.09, 0.13, 0.02, 0.4))}   # all different
    p = rng.uniform(0, 1, (nz, ny, nx)).astype(np.float32)
    t = rng.uniform(320, 340, (nz, ny, nx)).astype(np.float32)
    got = oracle.hot3d(p, t, coeff=k)
    np.testing.assert_allclose(got, _hot3d_numpy(p, t, k, np.float64), rtol=1e-6)
    assert np.array_equal(got, _hot3d_numpy(p, t, k, np.float32))   # same roundings, other indexing
    assert oracle.hot3d_blocks(nx, ny) == 6
    out = np.full_like(t, -1.0)
    for a, b in ((3, 6), (0, 2), (2, 3)):
        out = oracle.hot3d(p, t, coeff=k, out=out, start=a, end=b)
    assert np.array_equal(out, got)
    one = oracle.hot3d(p, t, coeff=k, out=np.full_like(t, -1.0), start=3, end=4)   # block (1, 1): x 64.., y 4..7
    assert np.array_equal(one[:, 4:8, 64:], got[:, 4:8, 64:])
    mask = np.ones_like(t, bool)
    mask[:, 4:8, 64:] = False
    assert (one[mask] == -1).all()
    # two layers: bottom and top only
    assert np.array_equal(oracle.hot3d(p[:2], t[:2], coeff=k), _hot3d_numpy(p[:2], t[:2], k, np.float32))


# ----------------------------------------------------------------------------- path
def _path_rows(wall, src, rows):
    """Textbook pathfinder over the whole grid, a row at a time."""
    cur = src.astype(np.int64)
    for r in range(rows):
        left = np.concatenate(([cur[0]], cur[:-1]))
        right = np.concatenate((cur[1:], [cur[-1]]))
        cur = wall[r] + np.minimum(np.minimum(left, cur), right)
    return cur.astype(np.int32)


@pytest.mark.parametrize("cols,iteration", [(1200, 125), (300, 20), (256, 127), (7, 3), (1, 1), (431, 100)])
def test_path_equals_the_row_by_row_programme(cols, iteration):
    rng = np.random.default_rng(cols + iteration)
    wall = rng.integers(0, 10, (iteration + 2, cols), dtype=np.int32)
    src = rng.integers(0, 10, cols, dtype=np.int32)
    got = oracle.path(iteration, wall, src)
    assert np.array_equal(got, _path_rows(wall, src, iteration))
    # from a later row of the wall
    got1 = oracle.path(iteration, wall, src, start_step=2)
    assert np.array_equal(got1, _path_rows(wall[2:], src, iteration))
    blocks = oracle.path_blocks(cols, iteration)
    assert blocks == -(-cols // (256 - 2 * iteration))
    # any tiling of the positions
    out = np.full(cols, -1, np.int32)
    cuts = sorted({0, blocks // 3, blocks // 2, blocks})
    for a, b in reversed(list(zip(cuts, cuts[1:]))):
        out = oracle.path(iteration, wall, src, out=out, start=a, end=b)
    assert np.array_equal(out, got)


def test_path_one_position_writes_its_columns_only():
    rng = np.random.default_rng(9)
    cols, iteration = 100, 118                       # 20 result columns per position
    wall = rng.integers(0, 10, (iteration, cols), dtype=np.int32)
    src = rng.integers(0, 10, cols, dtype=np.int32)
    whole = oracle.path(iteration, wall, src)
    one = oracle.path(iteration, wall, src, out=np.full(cols, -1, np.int32), start=2, end=3)
    assert np.array_equal(one[40:60], whole[40:60]) and (one[:40] == -1).all() and (one[60:] == -1).all()


def test_path_brute_force_over_all_paths():
    rng = np.random.default_rng(11)
    cols, rows = 5, 4
    wall = rng.integers(0, 10, (rows, cols), dtype=np.int32)
    src = rng.integers(0, 10, cols, dtype=np.int32)
    best = np.full(cols, 1 << 30)
    for start_col in range(cols):
        for moves in itertools.product((-1, 0, 1), repeat=rows):
            x, cost, ok = start_col, int(src[start_col]), True
            for r, m in enumerate(moves):
                x += m
                if x < 0 or x >= cols:
                    ok = False
                    break
                cost += int(wall[r, x])
            if ok:
                best[x] = min(best[x], cost)
    assert np.array_equal(oracle.path(rows, wall, src), best)


def test_path_source_is_rand_mod_ten():
    grid = oracle.path_source(3, 1200)
    assert grid.min() == 0 and grid.max() == 9
    # glibc's rand() after srand(9): the same stream the fft source draws from after its own seed,
    # checked here through its statistics and its reproducibility
    assert np.array_equal(grid, oracle.path_source(3, 1200))
    counts = np.bincount(grid.reshape(-1), minlength=10)
    assert counts.min() > 280 and counts.max() < 440


# ----------------------------------------------------------------------------- lava
def _lava_inputs(boxes1d, seed=21, equal_charges=False):
    rng = np.random.default_rng(seed)
    n = 100 * boxes1d ** 3
    rv = (rng.integers(1, 11, (n, 4)) / 10.0).astype(np.float32)       # 0.1 .. 1.0 as the reference draws them
    qv = np.full(n, 0.5, np.float32) if equal_charges else (rng.integers(1, 11, n) / 10.0).astype(np.float32)
    return rv, qv


def _lava_float64(alpha, boxes1d, rv, qv):
    """The same sums in float64, box pairs found from coordinates (not from the oracle's list)."""
    r, q = rv.astype(np.float64), qv.astype(np.float64)
    a2 = 2.0 * alpha * alpha
    out = np.zeros_like(r)
    coords = [(x, y, z) for z in range(boxes1d) for y in range(boxes1d) for x in range(boxes1d)]
    for a, (ax, ay, az) in enumerate(coords):
        A = r[100 * a:100 * a + 100]
        for b, (bx, by, bz) in enumerate(coords):
            if max(abs(ax - bx), abs(ay - by), abs(az - bz)) > 1:
                continue
            B, qB = r[100 * b:100 * b + 100], q[100 * b:100 * b + 100]
            r2 = A[:, None, 0] + B[None, :, 0] - A[:, 1:] @ B[:, 1:].T
            vij = np.exp(-a2 * r2)
            out[100 * a:100 * a + 100, 0] += vij @ qB
            for c in (1, 2, 3):
                out[100 * a:100 * a + 100, c] += (2 * vij * (A[:, None, c] - B[None, :, c])) @ qB
    return out


def test_lava_box_list():
    boxes = oracle.lava_boxes(4)
    assert len(boxes) == 64
    counts = np.bincount(boxes["nn"], minlength=27)
    assert (counts[7], counts[11], counts[17], counts[26]) == (8, 24, 24, 8) and counts.sum() == 64
    for b in boxes:
        assert b["number"] == b["x"] + 4 * b["y"] + 16 * b["z"] and b["offset"] == 100 * b["number"]
        nei = b["nei"][:b["nn"]]
        assert len(set(nei["number"].tolist())) == b["nn"] and b["number"] not in nei["number"]
        for ne in nei:
            assert max(abs(ne["x"] - b["x"]), abs(ne["y"] - b["y"]), abs(ne["z"] - b["z"])) == 1
            assert ne["number"] == ne["x"] + 4 * ne["y"] + 16 * ne["z"] and ne["offset"] == 100 * ne["number"]
            assert b["number"] in boxes[ne["number"]]["nei"][:boxes[ne["number"]]["nn"]]["number"]     # symmetric
    assert oracle.lava_boxes(1)["nn"].tolist() == [0]


def test_lava_against_float64_and_closed_forms():
    rv, qv = _lava_inputs(2)
    got = oracle.lava(0.5, 2, rv, qv)
    want = _lava_float64(0.5, 2, rv, qv)
    assert np.all(np.abs(got - want) <= 2e-3 + 2e-5 * np.abs(want))          # 800 float32 additions per sum of ~250
    # one box, particle 0 against the box: the potential term by hand
    rv1, qv1 = _lava_inputs(1, seed=5)
    one = oracle.lava(0.5, 1, rv1, qv1)
    r = rv1.astype(np.float64)
    r2 = r[0, 0] + r[:, 0] - r[:, 1:] @ r[0, 1:]
    assert one[0, 0] == pytest.approx(float(np.sum(qv1 * np.exp(-0.5 * r2))), rel=1e-5)
    # alpha enters as a2 = 2 alpha^2
    other = oracle.lava(1.0, 1, rv1, qv1)
    assert other[0, 0] == pytest.approx(float(np.sum(qv1 * np.exp(-2.0 * r2))), rel=1e-5)
    # equal charges: every pair's forces cancel, so all forces sum to zero (the potentials do not)
    rv, qv = _lava_inputs(3, seed=8, equal_charges=True)
    f = oracle.lava(0.5, 3, rv, qv).astype(np.float64)
    assert np.all(np.abs(f[:, 1:].sum(axis=0)) <= 1e-4 * np.abs(f[:, 1:]).sum(axis=0))
    assert f[:, 0].min() > 0


def test_lava_positions():
    rv, qv = _lava_inputs(2, seed=13)
    whole = oracle.lava(0.5, 2, rv, qv)
    n = oracle.lava_blocks(2)
    assert n == 8 * 27
    # any ascending tiling adds the same terms in the same order
    f = np.zeros_like(rv)
    for a, b in ((0, 5), (5, 8), (8, 100), (100, n)):
        f = oracle.lava(0.5, 2, rv, qv, fv=f, start=a, end=b)
    assert np.array_equal(f.view(np.uint32), whole.view(np.uint32))
    # row 0 is every box against itself; a 2^3 system has 7 neighbours a box: rows 8 .. 26 add nothing
    self_only = oracle.lava(0.5, 2, rv, qv, start=0, end=8)
    assert np.all(self_only[:, 0] > 0) and np.all(self_only[:, 0] < whole[:, 0])
    assert np.array_equal(oracle.lava(0.5, 2, rv, qv, start=8 * 8, end=n), np.zeros_like(rv))
    # one position touches its box only, and starts from what the array holds
    base = np.full_like(rv, 3.0)
    one = oracle.lava(0.5, 2, rv, qv, fv=base, start=8 + 3, end=8 + 4)             # box 3, its first neighbour
    assert np.array_equal(np.delete(one, np.s_[300:400], axis=0), np.delete(base, np.s_[300:400], axis=0))
    assert np.all(one[300:400, 0] > 3.0)
    # positions past the grid wrap
    again = oracle.lava(0.5, 2, rv, qv, fv=base, start=n + 8 + 3, end=n + 8 + 4)
    assert np.array_equal(again, one)
