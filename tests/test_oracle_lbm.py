"""Pins oracle.lbm: obstacle permutation, conservation laws, equilibrium fixed
point and an independent gather-form numpy float64 formulation."""
import numpy as np
import pytest

import oracle

NAMES = "C N S E W T B NE NW SE SW NT NB ST SB ET EB WT WB".split()  # lbm_header.h:228-233
VEC = {"C": (0, 0, 0)}
for _n in NAMES[1:]:
    VEC[_n] = (("E" in _n) - ("W" in _n), ("N" in _n) - ("S" in _n), ("T" in _n) - ("B" in _n))
OPP = {n: NAMES[[VEC[m] for m in NAMES].index(tuple(-v for v in VEC[n]))] for n in NAMES}
W = {n: (1 / 3 if sum(map(abs, VEC[n])) == 0 else 1 / 18 if sum(map(abs, VEC[n])) == 1 else 1 / 36)
     for n in NAMES}
OMEGA = 1.95


def make_grid(sx, sy, sz, rng, obstacle_p=0.05, accel_p=0.0):
    cells = sx * sy * sz
    g = np.zeros((20, cells), np.float32)
    for e, n in enumerate(NAMES):
        g[e] = np.float32(W[n]) + rng.uniform(0, 1e-3, cells).astype(np.float32)
    flags = (rng.uniform(0, 1, cells) < obstacle_p).astype(np.uint32)
    flags |= ((rng.uniform(0, 1, cells) < accel_p).astype(np.uint32) << 1)
    g[19] = flags.view(np.float32)
    return g


def numpy_f64(src, sx, sy, sz):
    """Collide in float64, then stream in gather form on the linear cell index."""
    cells = sx * sy * sz
    f = {n: src[e].astype(np.float64) for e, n in enumerate(NAMES)}
    flags = src[19].view(np.uint32)
    rho = sum(f.values())
    u = [sum(VEC[n][d] * f[n] for n in NAMES) / rho for d in range(3)]
    acc = (flags & 2) != 0
    for d, v in enumerate((0.005, 0.002, 0.0)):
        u[d] = np.where(acc, np.float64(np.float32(v)), u[d])
    usq = u[0] ** 2 + u[1] ** 2 + u[2] ** 2
    post = {}
    for n in NAMES:
        cu = sum(VEC[n][d] * u[d] for d in range(3))
        feq = W[n] * rho * (1 + 3 * cu + 4.5 * cu * cu - 1.5 * usq)
        post[n] = (1 - np.float64(np.float32(OMEGA))) * f[n] + np.float64(np.float32(OMEGA)) * feq
    obst = (flags & 1) != 0
    out = {n: np.where(obst, f[OPP[n]], post[n]) for n in NAMES}
    dst = np.full((20, cells), np.nan)
    for e, n in enumerate(NAMES):
        off = VEC[n][0] + VEC[n][1] * sx + VEC[n][2] * sx * sy
        lo, hi = max(0, off), min(cells, cells + off)
        dst[e, lo:hi] = out[n][lo - off:hi - off]
    return dst


@pytest.mark.parametrize("dims", [(4, 4, 4), (12, 5, 6), (7, 3, 9)])
def test_matches_numpy_float64(dims):
    sx, sy, sz = dims
    rng = np.random.default_rng(7)
    src = make_grid(sx, sy, sz, rng, obstacle_p=0.2, accel_p=0.2)
    dst0 = np.full_like(src, -5.0)
    got = oracle.lbm(src.reshape(-1), dst0.reshape(-1), sx, sy, sz).reshape(20, -1)
    want = numpy_f64(src, sx, sy, sz)
    untouched = np.isnan(want)
    assert np.all(got[untouched] == -5.0)          # incl. the whole FLAGS plane
    assert untouched[19].all()
    np.testing.assert_allclose(got[~untouched], want[~untouched], rtol=2e-5, atol=1e-7)


def test_obstacle_cells_are_an_exact_permutation():
    sx, sy, sz = 6, 5, 4
    cells = sx * sy * sz
    rng = np.random.default_rng(8)
    src = np.zeros((20, cells), np.float32)
    src[:19] = rng.uniform(0, 1, (19, cells)).astype(np.float32)
    src[19] = np.ones(cells, np.uint32).view(np.float32)
    got = oracle.lbm(src.reshape(-1), np.full(20 * cells, -5.0, np.float32), sx, sy, sz).reshape(20, -1)
    for e, n in enumerate(NAMES):
        off = VEC[n][0] + VEC[n][1] * sx + VEC[n][2] * sx * sy
        opp = NAMES.index(OPP[n])
        for c in range(cells):
            t = c + off
            if 0 <= t < cells:
                assert got[e, t] == src[opp, c]


def test_fluid_collision_conserves_mass_and_momentum():
    sx, sy, sz = 8, 6, 5
    cells = sx * sy * sz
    rng = np.random.default_rng(9)
    src = make_grid(sx, sy, sz, rng, obstacle_p=0.0)
    src[:19] += rng.uniform(0, 0.05, (19, cells)).astype(np.float32)  # well off equilibrium
    got = oracle.lbm(src.reshape(-1), np.zeros(20 * cells, np.float32), sx, sy, sz).reshape(20, -1)
    # undo the streaming for cells whose 19 targets are all in range
    post = np.zeros((19, cells))
    ok = np.ones(cells, bool)
    for e, n in enumerate(NAMES):
        off = VEC[n][0] + VEC[n][1] * sx + VEC[n][2] * sx * sy
        t = np.arange(cells) + off
        ok &= (t >= 0) & (t < cells)
        post[e] = got[e, np.clip(t, 0, cells - 1)]
    pre = src[:19].astype(np.float64)
    assert ok.sum() > cells // 2
    np.testing.assert_allclose(post.sum(0)[ok], pre.sum(0)[ok], rtol=1e-5)
    for d in range(3):
        cvec = np.array([VEC[n][d] for n in NAMES], np.float64)[:, None]
        np.testing.assert_allclose((cvec * post).sum(0)[ok], (cvec * pre).sum(0)[ok], atol=2e-6)


def test_rest_equilibrium_is_a_fixed_point():
    sx, sy, sz = 5, 5, 5
    cells = sx * sy * sz
    src = np.zeros((20, cells), np.float32)
    for e, n in enumerate(NAMES):
        src[e] = np.float32(W[n]) * np.float32(1.25)
    got = oracle.lbm(src.reshape(-1), np.zeros(20 * cells, np.float32), sx, sy, sz).reshape(20, -1)
    inner = got[:19, sx * sy + sx + 1: cells - sx * sy - sx - 1]
    np.testing.assert_allclose(inner, src[:19, :inner.shape[1]], rtol=3e-6)


def test_block_range_and_launch_shape():
    sx, sy, sz = 8, 4, 3
    rng = np.random.default_rng(10)
    src = make_grid(sx, sy, sz, rng)
    full = oracle.lbm(src.reshape(-1), np.zeros(src.size, np.float32), sx, sy, sz)
    acc = np.zeros(src.size, np.float32)
    for s, e in [(0, 5), (5, 6), (6, 12)]:
        acc = oracle.lbm(src.reshape(-1), acc, sx, sy, sz, s, e)
    assert np.array_equal(acc, full)
    # fusion/code/kinfo.json "lbm.ori_blks" = 16384 = SIZE_Y*SIZE_Z for 128^3
    assert 128 * 128 == 16384
