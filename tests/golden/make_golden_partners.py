#!/usr/bin/env python3
"""Writes tests/golden/kernels_partners.npz: small seeded inputs of the later best-effort partners
(sgemm, fft, cutcp, nn, hotspot3D, pathfinder, lavaMD) and the outputs of the CPU oracle on them.

As for kernels_small.npz the reference holds no outputs for these kernels; the vectors come from
the oracle, which tests/test_oracle_{sgemm,fft,cutcp,rodinia}.py pin.  The GPU parity tests
compare the HIP path with this file.

    python tests/golden/make_golden_partners.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402


def main():
    rng = np.random.default_rng(20241125)
    out = {}
    # sgemm 128 x 32 x 100: C = 2 C + 2 A B
    sA, sB = rng.uniform(0, 1, (100, 128)).astype(np.float32), rng.uniform(0, 1, (100, 32)).astype(np.float32)
    sC = rng.uniform(-1, 1, (32, 128)).astype(np.float32)
    out.update(sgemm_A=sA, sgemm_B=sB, sgemm_C0=sC, sgemm_C=oracle.sgemm(sA, sB, sC))
    # fft: 6 transforms of 256 points
    data = rng.uniform(-1, 1, (6, 256, 2)).astype(np.float32)
    out.update(fft_in=data, fft_out=oracle.fft(data))
    # cutcp: 120 atoms in a 16 x 16 x 8 lattice of spacing 0.5, cutoff 12
    atoms = np.empty((120, 4), np.float32)
    atoms[:, :3] = rng.uniform(0, 3.5, (120, 3))
    atoms[:, 3] = rng.uniform(0.1, 1, 120) * rng.choice([-1, 1], 120)
    prep = oracle.cutcp_prepare(atoms, (0, 0, 0), 16, 16, 8, 0.5, 12.0)
    out.update(cutcp_atoms=atoms, cutcp_energies=oracle.cutcp(prep, 0.5, 144.0, 0.006944, (2, 2, 1)))
    # nn: 700 records against (30, 90)
    loc = rng.uniform(0, 90, (700, 2)).astype(np.float32)
    out.update(nn_locations=loc, nn_distances=oracle.nn(loc, 30.0, 90.0))
    # hotspot3D 64 x 8 x 4, two steps
    p = rng.uniform(0, 0.01, (4, 8, 64)).astype(np.float32)
    t = rng.uniform(320, 340, (4, 8, 64)).astype(np.float32)
    t1 = oracle.hot3d(p, t)
    out.update(hot3d_power=p, hot3d_t0=t, hot3d_t1=t1, hot3d_t2=oracle.hot3d(p, t1))
    # pathfinder 300 columns, pyramid of 40 rows
    wall = rng.integers(0, 10, (41, 300), dtype=np.int32)
    src = rng.integers(0, 10, 300, dtype=np.int32)
    out.update(path_wall=wall, path_src=src, path_result=oracle.path(40, wall, src))
    # lavaMD 2^3 boxes
    rv = (rng.integers(1, 11, (800, 4)) / 10.0).astype(np.float32)
    qv = (rng.integers(1, 11, 800) / 10.0).astype(np.float32)
    out.update(lava_rv=rv, lava_qv=qv, lava_fv=oracle.lava(0.5, 2, rv, qv))
    path = os.path.join(HERE, "kernels_partners.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
