#!/usr/bin/env python3
"""Writes tests/golden/kernels_small.npz: small seeded inputs of every kernel of the
path and the outputs of the CPU oracle on them.

The reference holds no golden outputs for these kernels (its only checks compare
two GPU runs with each other), so the vectors come from the oracle, which is
pinned by closed forms and independent formulations in tests/test_oracle_*.py.
The GPU parity tests compare the HIP path with these files, so a GPU box needs
neither the reference nor a rebuilt oracle to check them.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402


def main():
    rng = np.random.default_rng(20240607)
    out = {}
    # tzgemm 128x256x128: fp64-accumulated truth and the fp32 ordered witness
    A = rng.uniform(-1, 1, (128, 128)).astype(np.float16)
    B = rng.uniform(-1, 1, (256, 128)).astype(np.float16)
    out.update(gemm_A=A, gemm_B=B, gemm_C64=oracle.tzgemm(A, B, f64=True), gemm_C32=oracle.tzgemm(A, B))
    # stencil 5 x 10 x 70, three sweeps with pointer swap
    a0 = rng.uniform(0, 1, (5, 10, 70)).astype(np.float32)
    c0, c1 = np.float32(1 / 6), np.float32(1 / 36)
    a, b = a0.copy(), a0.copy()
    for _ in range(3):
        b = oracle.stencil(c0, c1, a, b)
        a, b = b, a
    out.update(stencil_A0=a0, stencil_after3=a)
    # lbm 12 x 5 x 6 with obstacles and accelerated cells, two steps
    sx, sy, sz = 12, 5, 6
    cells = sx * sy * sz
    w = np.array([1 / 3] + [1 / 18] * 6 + [1 / 36] * 12, np.float32)
    g = np.zeros((20, cells), np.float32)
    g[:19] = w[:, None] + rng.uniform(0, 1e-3, (19, cells)).astype(np.float32)
    flags = (rng.uniform(0, 1, cells) < 0.2).astype(np.uint32) | ((rng.uniform(0, 1, cells) < 0.1).astype(np.uint32) << 1)
    g[19] = flags.view(np.float32)
    src = g.reshape(-1)
    d1 = oracle.lbm(src, src.copy(), sx, sy, sz)
    d2 = oracle.lbm(d1, src.copy(), sx, sy, sz)
    out.update(lbm_dims=np.array([sx, sy, sz]), lbm_src=src, lbm_step1=d1, lbm_step2=d2)
    # mri-q 96 samples x 512 voxels
    k = rng.uniform(-0.5, 0.5, (96, 3)).astype(np.float32)
    phiR, phiI = rng.uniform(0, 1, 96).astype(np.float32), rng.uniform(0, 1, 96).astype(np.float32)
    xyz = rng.uniform(-0.5, 0.5, (3, 512)).astype(np.float32)
    kv = np.concatenate([k, oracle.mriq_phimag(phiR, phiI)[:, None]], 1).astype(np.float32)
    z = np.zeros(512, np.float32)
    qr, qi = oracle.mriq(kv, *xyz, z, z, f64=True)
    out.update(mriq_phiR=phiR, mriq_phiI=phiI, mriq_kvals=kv, mriq_xyz=xyz, mriq_Qr=qr, mriq_Qi=qi)
    # cp 16 x 256 with the first 64 atoms after atom 0 of the glibc stream
    atoms = oracle.cp_initatoms(70)[1:65]
    grid = oracle.cp(oracle.cp_atoms_to_const(atoms, 0.0), np.zeros((16, 256), np.float32))
    out.update(cp_atoms=atoms, cp_grid=grid)
    # im2col 3 x 6 x 7, 3x3, pad 1
    im = rng.uniform(-1, 1, (3, 6, 7)).astype(np.float32)
    out.update(im2col_im=im, im2col_col=oracle.im2col(im, (3, 3), (1, 1), (1, 1)))
    # mri-fhd 96 samples x 512 voxels (drawn last: the entries above keep their values)
    fk = rng.uniform(-0.5, 0.5, (96, 3)).astype(np.float32)
    fphi, fd = rng.uniform(0, 1, (2, 96)).astype(np.float32), rng.uniform(0, 1, (2, 96)).astype(np.float32)
    fxyz = rng.uniform(-0.5, 0.5, (3, 512)).astype(np.float32)
    re, im_ = oracle.mrif_rhophi(fphi[0], fphi[1], fd[0], fd[1])
    fkv = np.concatenate([fk, re[:, None], im_[:, None]], 1).astype(np.float32)
    fr, fi = oracle.mrif(fkv, *fxyz, z, z, f64=True)
    out.update(mrif_phi=fphi, mrif_d=fd, mrif_kvals=fkv, mrif_xyz=fxyz, mrif_outR=fr, mrif_outI=fi)
    path = os.path.join(HERE, "kernels_small.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
