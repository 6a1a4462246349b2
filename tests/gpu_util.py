"""Shared helpers of the GPU parity tests: seeded inputs and device staging."""
import numpy as np
import torch

import oracle
import tacker_amd as ta

DEV = "cuda:0"
_ready = False


def setup():
    global _ready
    if not _ready:
        ta.init(0)
        _ready = True


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def gemm_inputs(M, N, K, seed=1337):
    rng = np.random.default_rng(seed)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float16)
    B = rng.uniform(-1, 1, (N, K)).astype(np.float16)
    return A, B


def gemm_tolerance_ok(got, truth, K):
    """|d| <= 5e-3 + 1e-5*|ref| elementwise and rel-Frobenius <= 1e-5 (fp32
    accumulation of K <= 4096 products of U[-1,1] halves against an fp64 sum)."""
    d = np.abs(got.astype(np.float64) - truth.astype(np.float64))
    elem = np.all(d <= 5e-3 + 1e-5 * np.abs(truth))
    fro = np.linalg.norm(d) / np.linalg.norm(truth)
    return bool(elem), float(fro), float(d.max())


def stencil_inputs(nz, ny, nx, seed=1337):
    rng = np.random.default_rng(seed)
    return rng.uniform(0, 1, (nz, ny, nx)).astype(np.float32)


LBM_W = np.array([1 / 3] + [1 / 18] * 6 + [1 / 36] * 12, np.float32)


def lbm_inputs(sx, sy, sz, seed=1337, obstacle_p=0.05, accel_p=0.0):
    rng = np.random.default_rng(seed)
    cells = sx * sy * sz
    g = np.zeros((20, cells), np.float32)
    g[:19] = LBM_W[:, None] + rng.uniform(0, 1e-3, (19, cells)).astype(np.float32)
    flags = (rng.uniform(0, 1, cells) < obstacle_p).astype(np.uint32)
    flags |= (rng.uniform(0, 1, cells) < accel_p).astype(np.uint32) << 1
    g[19] = flags.view(np.float32)
    return g.reshape(-1)


def mriq_inputs(numK, numX, seed=1337):
    rng = np.random.default_rng(seed)
    k = rng.uniform(-0.5, 0.5, (numK, 3)).astype(np.float32)
    phiR = rng.uniform(0, 1, numK).astype(np.float32)
    phiI = rng.uniform(0, 1, numK).astype(np.float32)
    xyz = rng.uniform(-0.5, 0.5, (3, numX)).astype(np.float32)
    return k, phiR, phiI, xyz


C0 = float(np.float32(1.0 / 6.0))
C1 = float(np.float32(1.0 / 6.0 / 6.0))


# ---- launching a kernel of the registry by key (the device layer of include/tacker_amd.h) ----
import ctypes as _C

_registry = {}


class _Dim3(_C.Structure):
    _fields_ = [("x", _C.c_uint), ("y", _C.c_uint), ("z", _C.c_uint)]


def registry():
    """key -> device function handle, as tk_register_kernels hands them out."""
    if not _registry:
        lib = ta.lib()
        cb_t = _C.CFUNCTYPE(None, _C.c_char_p, _C.c_void_p, _C.c_void_p)
        cb = cb_t(lambda key, func, ctx: _registry.__setitem__(key.decode(), func))
        lib.tk_register_kernels.argtypes = [cb_t, _C.c_void_p]
        assert lib.tk_register_kernels(cb, None) == 0
        lib.tkLaunchKernel.argtypes = [_C.c_void_p, _Dim3, _Dim3, _C.POINTER(_C.c_void_p), _C.c_size_t, _C.c_void_p]
    return _registry


def launch(key, grid, block, args):
    """args: ctypes values (c_int, c_float, c_void_p ...), in the kernel's parameter order."""
    func = registry()[key]
    holders = list(args)
    ptrs = (_C.c_void_p * len(holders))(*[_C.cast(_C.pointer(a), _C.c_void_p) for a in holders])
    rc = ta.lib().tkLaunchKernel(func, _Dim3(grid, 1, 1), _Dim3(block, 1, 1), ptrs, 0,
                                 torch.cuda.current_stream().cuda_stream)
    assert rc == 0, rc


def mrif_inputs(numK, numX, seed=1337):
    """k samples, phi (2, numK), d (2, numK), voxel coordinates (3, numX)"""
    rng = np.random.default_rng(seed)
    k = rng.uniform(-0.5, 0.5, (numK, 3)).astype(np.float32)
    phi = rng.uniform(0, 1, (2, numK)).astype(np.float32)
    d = rng.uniform(0, 1, (2, numK)).astype(np.float32)
    xyz = rng.uniform(-0.5, 0.5, (3, numX)).astype(np.float32)
    return k, phi, d, xyz


def mrif_table(k, phi, d):
    """AoS table {Kx,Ky,Kz,RhoPhiR,RhoPhiI} with RhoPhi from the oracle"""
    import oracle
    re, im = oracle.mrif_rhophi(phi[0], phi[1], d[0], d[1])
    return np.concatenate([k, re[:, None], im[:, None]], 1).astype(np.float32)
