"""Pins oracle.cutcp / oracle.cutcp_prepare (Parboil's cutoff Coulomb potential,
src/ori_kernel/cutcp_kernel.cu:19-158, src/header/cutcp_header.h:111-300).

The C restatement walks bins through a neighbour list as the reference does.  The checks do not: the
potential of every lattice point is summed in float64 straight over the list of atoms (no bins, no
neighbour list) -- a wrong bin index, a neighbour list that misses a bin within reach, a wrong point
layout inside a region or a wrong sign fails there; a single charge gives the closed form
q (1 - r^2/c^2)^2 / r inside the cutoff and exactly 0 outside; the binning is checked against a
dictionary built in Python, the neighbour list against its defining inequality and the numbers the
reference hard-codes for its own instance (bin grid 32 x 32, src/ori_kernel/cutcp_kernel.cu:224-225)."""
import numpy as np

import oracle

H, CUTOFF = 0.5, 12.0


def atoms_in_box(n, box, seed):
    rng = np.random.default_rng(seed)
    a = np.empty((n, 4), np.float32)
    a[:, :3] = rng.uniform(0, box, (n, 3))
    a[:, 3] = rng.uniform(-1, 1, n)
    a[a[:, 3] == 0, 3] = 0.5
    return a


def brute_force(atoms, regions, h, cutoff2, inv_cutoff2):
    """float64 potential on the (8 rx, 8 ry, 8 rz) lattice, laid out as oracle.cutcp lays it out"""
    rx, ry, rz = regions
    xs, ys, zs = [np.arange(8 * r) * float(h) for r in (rx, ry, rz)]
    pot = np.zeros((8 * rz, 8 * ry, 8 * rx))
    for ax, ay, az, q in atoms.astype(np.float64):
        r2 = (az - zs)[:, None, None] ** 2 + (ay - ys)[None, :, None] ** 2 + (ax - xs)[None, None, :] ** 2
        with np.errstate(divide="ignore", invalid="ignore"):
            term = q / np.sqrt(r2) * (1.0 - r2 * inv_cutoff2) ** 2
        pot += np.where(r2 < cutoff2, term, 0.0)
    return pot.reshape(rz, 8, ry, 8, rx, 8).transpose(0, 2, 4, 1, 3, 5)     # [zr][yr][xr][z][y][x]


def binned_atoms(prep):
    """the atoms that made it into a bin, as a list (the others are the CPU's in the reference)"""
    b = prep["bins"].reshape(-1, 4)
    return b[b[:, 3] != 0]


def test_matches_a_float64_sum_over_the_atom_list():
    n = 24                                       # 3 x 3 x 3 regions
    atoms = atoms_in_box(900, (n - 1) * H, seed=1)
    prep = oracle.cutcp_prepare(atoms, (0, 0, 0), n, n, n, H, CUTOFF)
    assert prep["extra"] + prep["excluded"] + len(binned_atoms(prep)) == len(atoms)
    got = oracle.cutcp(prep, H, CUTOFF ** 2, 1.0 / CUTOFF ** 2, (3, 3, 3))
    want = brute_force(binned_atoms(prep), (3, 3, 3), H, CUTOFF ** 2, 1.0 / CUTOFF ** 2)
    # a lattice point next to an atom sees 1/r of up to ~30; sums of ~900 fp32 terms
    assert np.all(np.abs(got - want) <= 2e-4 + 2e-5 * np.abs(want))
    assert np.abs(want).max() > 1.0


def test_single_charge_closed_form_and_exact_zero_outside_the_cutoff():
    n = 64                                       # 8 x 8 x 8 regions, 31.5 Angstroms: wider than the cutoff
    atom = np.array([[15.3, 16.1, 14.9, 0.75]], np.float32)
    prep = oracle.cutcp_prepare(atom, (0, 0, 0), n, n, n, H, CUTOFF)
    got = oracle.cutcp(prep, H, CUTOFF ** 2, 1.0 / CUTOFF ** 2, (8, 8, 8))
    lat = got.transpose(0, 3, 1, 4, 2, 5).reshape(n, n, n)                  # [z][y][x]
    g = np.arange(n) * H
    r2 = ((atom[0, 2] - g)[:, None, None].astype(np.float64) ** 2 + (atom[0, 1] - g)[None, :, None].astype(np.float64) ** 2 +
          (atom[0, 0] - g)[None, None, :].astype(np.float64) ** 2)
    inside = r2 < CUTOFF ** 2
    want = np.where(inside, 0.75 / np.sqrt(r2) * (1 - r2 / CUTOFF ** 2) ** 2, 0.0)
    assert np.all(np.abs(lat - want) <= 1e-6 + 1e-5 * np.abs(want))
    assert np.all(lat[r2 > (CUTOFF + 1e-3) ** 2] == 0.0) and inside.sum() > 50000 and (~inside).sum() > 100000


def test_binning_against_a_dictionary():
    n = 40
    atoms = atoms_in_box(3000, (n - 1) * H, seed=2)
    atoms[5, 3] = 0.0                                                       # no charge: excluded
    atoms[6, :3] = (-13.0, 1.0, 1.0)                                        # outside the padded bins: excluded
    atoms[7, :3] = (-3.0, 1.0, 1.0)                                         # in a padding bin: kept
    lo = np.array((0.25, -0.5, 0.0), np.float32)
    prep = oracle.cutcp_prepare(atoms, lo, n, n, n, H, CUTOFF)
    c = prep["padding"]
    assert c == 3 and prep["binDim"] == (5 + 6, 5 + 6, 5 + 6)              # ceil(40 * 0.5 / 4) + 2 c
    want = {}
    extra = excluded = 0
    for a in atoms:
        p = a[:3] - lo
        ijk = tuple(int(v) for v in np.floor(p * np.float32(0.25)))
        if a[3] == 0 or not all(-c <= v < 11 - c for v in ijk):
            excluded += 1
        elif len(want.setdefault(ijk, [])) < 8:
            want[ijk].append((p[0], p[1], p[2], a[3]))
        else:
            extra += 1
    assert (prep["extra"], prep["excluded"]) == (extra, excluded) and excluded >= 2
    bins = prep["bins"]
    seen = 0
    for (i, j, k), members in want.items():
        slot = bins[k + c, j + c, i + c]
        assert np.array_equal(slot[:len(members)], np.array(members, np.float32))
        assert np.all(slot[len(members):] == 0)
        seen += len(members)
    assert np.count_nonzero(bins[..., 3]) == seen


def test_neighbour_list_is_its_defining_inequality_and_the_references_instance():
    prep = oracle.cutcp_prepare(np.zeros((0, 4), np.float32), (0, 0, 0), 208, 208, 208, H, CUTOFF)
    # the instance the reference hard-codes: 208^3 points, 26^3 regions, bins 32 x 32 (x 32), zero bin 3 in
    assert prep["binDim"] == (32, 32, 32) and prep["padding"] == 3
    nbr = prep["nbr"]
    # a region is as wide as a bin (8 h = 4): offsets with |v|^2 * 16 < (12 + 4 sqrt 3)^2, k slowest, i fastest
    want = [(i, j, k) for k in range(-3, 4) for j in range(-3, 4) for i in range(-3, 4)
            if (i * i + j * j + k * k) * 16.0 < (12 + np.sqrt(np.float32(3)) * 4) ** 2]
    assert [tuple(v) for v in nbr.tolist()] == want and len(want) == 335
    # h = 0.4: a bin is not a whole number of regions wide, the list is built around a cube of 3 x 3 x 3 bins
    # (all 343 offsets qualify); a cutoff of 24 needs 13 bins across and does not fit the list of 11
    wide = oracle.cutcp_prepare(np.zeros((0, 4), np.float32), (0, 0, 0), 16, 16, 16, 0.4, CUTOFF)
    assert len(wide["nbr"]) == 343
    try:
        oracle.cutcp_prepare(np.zeros((0, 4), np.float32), (0, 0, 0), 16, 16, 16, 0.5, 24.0)
        raise AssertionError("accepted a cutoff beyond the list")
    except ValueError:
        pass


def test_positions_follow_the_gptb_index_and_leave_other_regions_alone():
    n = 24
    atoms = atoms_in_box(400, (n - 1) * H, seed=3)
    prep = oracle.cutcp_prepare(atoms, (0, 0, 0), n, n, 16, H, CUTOFF)
    whole = oracle.cutcp(prep, H, 144.0, 0.006944, (3, 3, 2))
    # position p = region (p / (3 * 2), (p / 2) % 3, p % 2): x slowest (src/gptb_kernel/cutcp_kernel.cu:61-63)
    part = oracle.cutcp(prep, H, 144.0, 0.006944, (3, 3, 2), 7, 9, out=np.full((2, 3, 3, 8, 8, 8), -5.0, np.float32))
    touched = [(1, 0, 1), (1, 1, 0)]                                        # (x, y, z) of positions 7 and 8
    for x in range(3):
        for y in range(3):
            for z in range(2):
                if (x, y, z) in touched:
                    assert np.array_equal(part[z, y, x], whole[z, y, x])
                else:
                    assert np.all(part[z, y, x] == -5.0)
    tiled = np.zeros_like(whole)
    for a, b in ((0, 5), (5, 6), (6, 18)):
        tiled = oracle.cutcp(prep, H, 144.0, 0.006944, (3, 3, 2), a, b, out=tiled)
    assert np.array_equal(tiled, whole)


def test_any_ascending_tiling_of_the_region_by_part_grid_is_the_one_walk():
    # 335 neighbour bins dealt round-robin into 11 parts: position p adds part p // regions (entries part,
    # part + 11, ...) to region p % regions, the energies resting in the output between parts
    n = 24
    atoms = atoms_in_box(600, (n - 1) * H, seed=5)
    prep = oracle.cutcp_prepare(atoms, (0, 0, 0), n, n, 16, H, CUTOFF)
    regions = (3, 3, 2)
    whole = oracle.cutcp(prep, H, 144.0, 0.006944, regions)
    total = oracle.cutcp_positions(regions, len(prep["nbr"]))
    assert total == 18 * 11
    rng = np.random.default_rng(6)
    for _ in range(3):
        cuts = sorted(set(rng.integers(0, total + 1, 5).tolist()) | {0, total})
        out = np.full((2, 3, 3, 8, 8, 8), 7.0, np.float32)              # part 0 does not read what is there
        for a, b in zip(cuts, cuts[1:]):
            out = oracle.cutcp(prep, H, 144.0, 0.006944, regions, a, b, out=out, parts="chunks")
        if _ == 0:
            first = out
        assert np.array_equal(out.view(np.uint32), first.view(np.uint32))     # whatever the tiling: the same bits
        # ... and the one ascending walk of the reference up to the order of the additions
        assert np.all(np.abs(out - whole) <= 1e-5 + 2e-6 * np.abs(whole))
    # one position = one part of one region: float64 over the atoms of exactly those 32 bins
    pos = 18 * 4 + 7                                                    # part 4 of region 7 = (x 1, y 0, z 1)
    got = oracle.cutcp(prep, H, 144.0, 0.006944, regions, pos, pos + 1, parts="chunks")
    # part 4 starts from the energies in memory (zero here) and adds its bins only: entries 4, 15, 26, ...
    bins, c = prep["bins"], prep["padding"]
    centre = [int(np.floor((8 * r + 4) * H * 0.25)) for r in (1, 0, 1)]
    members = []
    for i, j, k in prep["nbr"][4::11]:
        slot = bins[centre[2] + k + c, centre[1] + j + c, centre[0] + i + c]
        for a in slot:
            if a[3] == 0:
                break
            members.append(a)
    want = brute_force(np.array(members, np.float32).reshape(-1, 4), regions, H, 144.0, 0.006944)
    assert len(members) > 10 and np.all(np.abs(got[1, 0, 1] - want[1, 0, 1]) <= 1e-4 + 2e-5 * np.abs(want[1, 0, 1]))
    other = np.ones_like(got, bool)
    other[1, 0, 1] = False
    assert np.all(got[other] == 0.0)
