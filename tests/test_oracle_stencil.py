"""Pins oracle.stencil*: closed forms, an independent sliced numpy formulation,
boundary invariance, and GPTB partition / wrap invariants."""
import numpy as np
import pytest

import oracle

C0 = np.float32(1.0 / 6.0)
C1 = np.float32(1.0 / 6.0 / 6.0)  # src/ori_kernel/stencil_kernel.cu:132-133


def sliced_f64(c0, c1, A0):
    """7-point Jacobi via array slicing in float64 (interior only)."""
    a = A0.astype(np.float64)
    out = a.copy()
    out[1:-1, 1:-1, 1:-1] = (a[2:, 1:-1, 1:-1] + a[:-2, 1:-1, 1:-1] + a[1:-1, 2:, 1:-1] +
                             a[1:-1, :-2, 1:-1] + a[1:-1, 1:-1, 2:] + a[1:-1, 1:-1, :-2]) * float(c1) \
        - a[1:-1, 1:-1, 1:-1] * float(c0)
    return out


@pytest.mark.parametrize("shape", [(8, 8, 8), (6, 10, 70), (5, 7, 130), (4, 9, 33)])
def test_matches_sliced_float64(shape):
    rng = np.random.default_rng(4)
    A0 = rng.uniform(0, 1, shape).astype(np.float32)
    got = oracle.stencil(C0, C1, A0, A0)
    want = sliced_f64(C0, C1, A0)
    np.testing.assert_allclose(got, want, rtol=0, atol=1e-6)
    # a sign or index slip moves results by O(0.1)
    assert np.abs(got - A0)[1:-1, 1:-1, 1:-1].mean() > 0.05


def test_distinct_coefficients_and_asymmetric_field():
    # top/bottom/up/down/left/right each get a distinct slope so that swapping
    # any two neighbours, or c0 with c1, changes the answer.
    nz, ny, nx = 6, 9, 11
    k, j, i = np.meshgrid(np.arange(nz), np.arange(ny), np.arange(nx), indexing="ij")
    A0 = (i * i + 3.0 * j * j * j + 7.0 * k * k * k * k).astype(np.float32)
    c0, c1 = np.float32(0.75), np.float32(0.125)
    got = oracle.stencil(c0, c1, A0, np.zeros_like(A0))
    want = sliced_f64(c0, c1, A0)
    want[0], want[-1] = 0, 0
    want[:, 0], want[:, -1] = 0, 0
    want[:, :, 0], want[:, :, -1] = 0, 0
    np.testing.assert_allclose(got, want, rtol=1e-6)


def test_harmonic_field_maps_to_zero_and_constant_closed_form():
    nz, ny, nx = 7, 12, 66
    k, j, i = np.meshgrid(np.arange(nz), np.arange(ny), np.arange(nx), indexing="ij")
    lin = (2 * i - 3 * j + 5 * k + 1).astype(np.float32)  # integers: exact arithmetic
    # 6*c1 == c0 exactly representable case: c0 = 6/8, c1 = 1/8
    out = oracle.stencil(np.float32(0.75), np.float32(0.125), lin, lin)
    assert np.all(out[1:-1, 1:-1, 1:-1] == 0)
    const = np.full((nz, ny, nx), 3.0, np.float32)
    out = oracle.stencil(np.float32(0.5), np.float32(0.25), const, const)
    assert np.all(out[1:-1, 1:-1, 1:-1] == 3.0 * (6 * 0.25 - 0.5))


def test_boundary_cells_are_never_written():
    rng = np.random.default_rng(5)
    A0 = rng.uniform(0, 1, (5, 9, 70)).astype(np.float32)
    sentinel = np.full_like(A0, -3.0)
    out = oracle.stencil(C0, C1, A0, sentinel)
    inner = np.zeros(A0.shape, bool)
    inner[1:-1, 1:-1, 1:-1] = True
    assert np.all(out[~inner] == -3.0)
    assert np.all(out[inner] != -3.0)


def test_gptb_partition_equals_full_and_wraps():
    rng = np.random.default_rng(6)
    A0 = rng.uniform(0, 1, (5, 12, 130)).astype(np.float32)
    gdx, gdy = oracle.stencil_grid(130, 12)
    assert (gdx, gdy) == (3, 3)
    full = oracle.stencil(C0, C1, A0, A0)
    acc = A0.copy()
    for s, e in [(0, 2), (2, 7), (7, 9)]:
        acc = oracle.stencil_gptb(C0, C1, A0, acc, s, e)
    assert np.array_equal(acc, full)
    # positions beyond gdx*gdy wrap in y and recompute the same cells
    again = oracle.stencil_gptb(C0, C1, A0, full, 9, 18)
    assert np.array_equal(again, full)
    # a strict sub-range leaves the other blocks' cells at their initial value
    part = oracle.stencil_gptb(C0, C1, A0, np.full_like(A0, -3.0), 4, 5)  # block (1,1)
    touched = part != -3.0
    assert touched[:, 4:8, 64:128].any() and not touched[:, :4].any() and not touched[:, 8:].any()
    assert not touched[:, :, :64].any() and not touched[:, :, 128:].any()


def test_z_parts_of_the_position_grid_tile_the_sweep():
    # the position grid (gdx, gdy, gdz) with gdz runs of zrun centre planes: any tiling is one sweep,
    # a position writes only its block's columns and its run's planes, gdz = 1 is the block grid
    rng = np.random.default_rng(8)
    A0 = rng.uniform(0, 1, (21, 12, 130)).astype(np.float32)
    gdx, gdy = oracle.stencil_grid(130, 12)
    blocks = gdx * gdy
    full = oracle.stencil(C0, C1, A0, A0)
    for zrun in (8, 5, 19, 40):
        runs = -(-(21 - 2) // zrun)
        npos = blocks * runs
        assert oracle.stencil_positions(130, 12, 21, zrun) == npos
        acc = A0.copy()
        for s, e in [(5, npos), (0, 2), (2, 5)]:
            acc = oracle.stencil_gptb(C0, C1, A0, acc, s, e, gdz=runs, zrun=zrun)
        assert np.array_equal(acc, full), zrun
        # position p = block p % blocks, run p // blocks: block (1, 1) = 4, its second run if there is one
        r = min(1, runs - 1)
        part = oracle.stencil_gptb(C0, C1, A0, np.full_like(A0, -3.0), r * blocks + 4, r * blocks + 5,
                                   gdz=runs, zrun=zrun)
        touched = part != -3.0
        k_lo, k_hi = 1 + r * zrun, min(20, 1 + (r + 1) * zrun)
        want = np.zeros(A0.shape, bool)
        want[k_lo:k_hi, 4:8, 64:128] = True
        assert np.array_equal(touched, want)
        assert np.array_equal(part[want], full[want])
    # fewer parts than runs: a part is a group of consecutive runs
    acc = A0.copy()
    for s, e in [(0, 7), (7, 2 * blocks)]:
        acc = oracle.stencil_gptb(C0, C1, A0, acc, s, e, gdz=2, zrun=4)   # 5 runs in 2 parts: runs 0-1, 2-4
    assert np.array_equal(acc, full)
    half = oracle.stencil_gptb(C0, C1, A0, np.full_like(A0, -3.0), 0, blocks, gdz=2, zrun=4)
    assert np.all(half[9:] == -3.0) and np.all(half[1:9, 1:-1, 1:-1] != -3.0)


def test_reference_launch_shape_known_answer():
    # fusion/code/kinfo.json "stencil.ori_blks" = 1024 = ceil(512/64)*ceil(512/4)
    gdx, gdy = oracle.stencil_grid(512, 512)
    assert gdx * gdy == 1024
