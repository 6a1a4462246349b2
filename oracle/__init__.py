"""ctypes front end of the CPU oracle (``oracle/tacker_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke``
and by the ``cpu_baseline`` leg of ``bench.py``; the product package never
imports it.  All functions take and return numpy arrays.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libtacker_oracle.so")
_lib = None


def build(force=False):
    """Compile the oracle with gcc (see ``oracle/Makefile``)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-B", "libtacker_oracle.so"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _declare(_lib)
    return _lib


_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_u16p = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")


def _declare(l):
    l.orc_num_threads.restype = C.c_int
    l.orc_tzgemm_dims.argtypes = [C.c_int, C.c_int, C.c_int, _i32p]
    l.orc_tzgemm_tile_origin.argtypes = [C.c_uint, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int)]
    l.orc_tzgemm.argtypes = [_u16p, _u16p, _f32p, C.c_int, C.c_int, C.c_int, C.c_float, C.c_int,
                             C.c_int, C.c_int]
    l.orc_gptb_index.argtypes = [C.c_uint, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _i32p]
    l.orc_stencil_gptb.argtypes = [C.c_float, C.c_float, _f32p, _f32p, C.c_int, C.c_int, C.c_int,
                                   C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
    l.orc_stencil.argtypes = [C.c_float, C.c_float, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
    l.orc_sgemm_gptb.argtypes = [_f32p, _f32p, _f32p, _f32p] + [C.c_int] * 9
    l.orc_cutcp_gptb.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_float, C.c_float, C.c_float, C.c_void_p, _i32p] + [C.c_int] * 7
    l.orc_cutcp_prepare.argtypes = [_f32p, C.c_int, _f32p, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float, _i32p, _i32p,
                                    C.c_void_p, C.c_void_p, _i32p]
    l.orc_fft_gptb.argtypes = [_f32p, C.c_int, C.c_int, C.c_int]
    l.orc_fft_source.argtypes = [_f32p, C.c_int]
    l.orc_nn_gptb.argtypes = [_f32p, _f32p, C.c_int, C.c_float, C.c_float] + [C.c_int] * 5
    l.orc_hot3d_gptb.argtypes = ([_f32p, _f32p, _f32p, C.c_float, C.c_int, C.c_int, C.c_int] + [C.c_float] * 7 +
                                 [C.c_int] * 6)
    l.orc_hot3d_coefficients.argtypes = [C.c_int, C.c_int, C.c_int, _f32p]
    l.orc_path_gptb.argtypes = [C.c_int, _i32p, _i32p, _i32p] + [C.c_int] * 5
    l.orc_path_source.argtypes = [_i32p, C.c_longlong]
    l.orc_lava_boxes.argtypes = [C.c_int, C.c_void_p]
    l.orc_lava_gptb.argtypes = [C.c_float, C.c_void_p, _f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
    l.orc_lbm_gptb.argtypes = [_f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
    l.orc_lbm.argtypes = [_f32p, _f32p, C.c_int, C.c_int, C.c_int]
    l.orc_mriq_phimag.argtypes = [_f32p, _f32p, _f32p, C.c_int]
    l.orc_mrif_rhophi.argtypes = [C.c_int, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p]
    l.orc_mrif_gptb.argtypes = [C.c_int, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, C.c_int,
                                C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
    l.orc_mriq_gptb.argtypes = [C.c_int, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, C.c_int,
                                C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
    l.orc_cp_initatoms.argtypes = [_f32p, C.c_int, C.c_uint, C.c_uint, C.c_uint, C.c_float]
    l.orc_cp_atoms_to_const.argtypes = [_f32p, C.c_int, C.c_float, _f32p]
    l.orc_cp_gptb.argtypes = [C.c_int, C.c_float, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
    l.orc_mnk_from_conv_args.argtypes = [_i32p, _i32p]
    l.orc_im2col.argtypes = [C.c_int, _f32p] + [C.c_int] * 12 + [_f32p]


def num_threads():
    return int(lib().orc_num_threads())


# --------------------------------------------------------------------------- tzgemm
ALPHA = np.float32(1.1)  # alpha_g, src/header/tzgemm_header.h:64


def tzgemm_dims(m, n, k):
    out = np.zeros(4, np.int32)
    lib().orc_tzgemm_dims(m, n, k, out)
    return [int(v) for v in out]


def tzgemm_tile_origin(pos, N):
    r, c = C.c_int(), C.c_int()
    lib().orc_tzgemm_tile_origin(pos, N, C.byref(r), C.byref(c))
    return r.value, c.value


def tzgemm(A, B, C_init=None, alpha=ALPHA, start=0, end=None, f64=False):
    """A [M][K] float16, B [N][K] float16 -> C [M][N] float32 (tiles [start,end))."""
    A = np.ascontiguousarray(A, np.float16)
    B = np.ascontiguousarray(B, np.float16)
    M, K = A.shape
    N = B.shape[0]
    assert B.shape[1] == K
    if end is None:
        end = (M // 64) * (N // 64)
    out = np.zeros((M, N), np.float32) if C_init is None else np.array(C_init, np.float32, order="C")
    lib().orc_tzgemm(A.view(np.uint16), B.view(np.uint16), out, M, N, K, float(alpha), start, end,
                     1 if f64 else 0)
    return out


def gptb_index(block_pos, t, gdx, gdy, bdx, bdy):
    out = np.zeros(4, np.int32)
    lib().orc_gptb_index(block_pos, t, gdx, gdy, bdx, bdy, out)
    return tuple(int(v) for v in out)


# --------------------------------------------------------------------------- stencil
def stencil_grid(nx, ny):
    """Natural launch grid of ori_stencil (src/ori_kernel/stencil_kernel.cu:166-173)."""
    return (nx + 63) // 64, (ny + 3) // 4


def stencil(c0, c1, A0, Anext):
    """One sweep; arrays are [nz][ny][nx] float32. Returns the new Anext."""
    nz, ny, nx = A0.shape
    out = np.array(Anext, np.float32, order="C")
    lib().orc_stencil(c0, c1, np.ascontiguousarray(A0, np.float32), out, nx, ny, nz)
    return out


STENCIL_Z_RUN = 8


def stencil_positions(nx, ny, nz, zrun=STENCIL_Z_RUN):
    """Block positions of the device objects' grid: blocks x runs of zrun centre planes."""
    gdx, gdy = stencil_grid(nx, ny)
    return gdx * gdy * max(1, -(-(nz - 2) // zrun))


def stencil_gptb(c0, c1, A0, Anext, start, end, gdx=None, gdy=None, bdx=32, bdy=4, gdz=1, zrun=STENCIL_Z_RUN):
    """Positions [start, end) of the (gdx, gdy, gdz) grid; gdz = 1 (default): whole block columns, the
    reference's kernel; gdz = 'runs': one run of zrun centre planes per position."""
    nz, ny, nx = A0.shape
    if gdx is None:
        gdx, gdy = stencil_grid(nx, ny)
    if gdz == "runs":
        gdz = max(1, -(-(nz - 2) // zrun))
    out = np.array(Anext, np.float32, order="C")
    lib().orc_stencil_gptb(c0, c1, np.ascontiguousarray(A0, np.float32), out, nx, ny, nz, gdx, gdy, gdz,
                           bdx, bdy, zrun, start, end)
    return out


# --------------------------------------------------------------------------- lbm
LBM_ENTRIES = 20


def lbm(src, dst, sx, sy, sz, start=0, end=None):
    """src/dst are flat float32 arrays of 20*cells (entry-major SoA). Returns new dst."""
    if end is None:
        end = sy * sz
    src = np.ascontiguousarray(src, np.float32)
    out = np.array(dst, np.float32, order="C")
    assert src.size == 20 * sx * sy * sz and out.size == src.size
    lib().orc_lbm_gptb(src, out, sx, sy, sz, start, end)
    return out


# --------------------------------------------------------------------------- mri-q
def mriq_phimag(phiR, phiI):
    out = np.zeros_like(phiR, dtype=np.float32)
    lib().orc_mriq_phimag(np.ascontiguousarray(phiR, np.float32),
                          np.ascontiguousarray(phiI, np.float32), out, phiR.size)
    return out


def mriq(kvals, x, y, z, Qr, Qi, start=0, end=None, gdx=None, f64=False, kchunk=None):
    """kvals is [numK][4] float32 {Kx,Ky,Kz,PhiMag}. Returns (Qr, Qi).

    Block positions [start, end).  kchunk=None: one position per block of 256 voxels, each adding
    the whole table.  kchunk=n: positions form a grid of gdx voxel blocks by ceil(numK / n) chunks of
    the table; position p adds chunk (p // gdx) % chunks to voxel block p % gdx."""
    kvals = np.ascontiguousarray(kvals, np.float32)
    numK = kvals.shape[0]
    numX = x.size
    if gdx is None:
        gdx = numX // 256
    if kchunk is None:
        gdy, kchunk = 1, max(numK, 1)
    else:
        gdy = max(1, -(-numK // kchunk))
    if end is None:
        end = gdx * gdy
    qr = np.array(Qr, np.float32, order="C")
    qi = np.array(Qi, np.float32, order="C")
    lib().orc_mriq_gptb(numK, kvals.reshape(-1), np.ascontiguousarray(x, np.float32),
                        np.ascontiguousarray(y, np.float32), np.ascontiguousarray(z, np.float32),
                        qr, qi, gdx, gdy, kchunk, start, end, 1 if f64 else 0)
    return qr, qi


# --------------------------------------------------------------------------- mri-fhd
def mrif_rhophi(phiR, phiI, dR, dI):
    f = lambda a: np.ascontiguousarray(a, np.float32)
    re, im = np.zeros(phiR.size, np.float32), np.zeros(phiR.size, np.float32)
    lib().orc_mrif_rhophi(phiR.size, f(phiR), f(phiI), f(dR), f(dI), re, im)
    return re, im


def mrif(kvals, x, y, z, outR, outI, start=0, end=None, gdx=None, f64=False, kchunk=None):
    """kvals is [numK][5] float32 {Kx,Ky,Kz,RhoPhiR,RhoPhiI}. Returns (outR, outI).
    Block positions as in mriq()."""
    kvals = np.ascontiguousarray(kvals, np.float32)
    numK = kvals.shape[0]
    numX = x.size
    if gdx is None:
        gdx = numX // 256
    if kchunk is None:
        gdy, kchunk = 1, max(numK, 1)
    else:
        gdy = max(1, -(-numK // kchunk))
    if end is None:
        end = gdx * gdy
    r = np.array(outR, np.float32, order="C")
    i = np.array(outI, np.float32, order="C")
    lib().orc_mrif_gptb(numK, kvals.reshape(-1), np.ascontiguousarray(x, np.float32),
                        np.ascontiguousarray(y, np.float32), np.ascontiguousarray(z, np.float32),
                        r, i, gdx, gdy, kchunk, start, end, 1 if f64 else 0)
    return r, i


# --------------------------------------------------------------------------- cp
def cp_initatoms(count=4000, volx=4096, voly=4096, volz=1, gridspacing=0.1):
    atoms = np.zeros(count * 4, np.float32)
    lib().orc_cp_initatoms(atoms, count, volx, voly, volz, gridspacing)
    return atoms.reshape(count, 4)


def cp_atoms_to_const(atoms, zplane=0.0):
    atoms = np.ascontiguousarray(atoms, np.float32).reshape(-1)
    out = np.zeros_like(atoms)
    lib().orc_cp_atoms_to_const(atoms, atoms.size // 4, zplane, out)
    return out.reshape(-1, 4)


def cp(atominfo, energygrid, gridspacing=0.1, start=0, end=None, parts=1):
    """energygrid is [voly][volx] float32 (volx multiple of 128, voly multiple of 8).

    Block positions [start, end) of the (volx/128, voly/8, parts) grid: parts=1, a position is a block of
    128 x 8 points; parts=4, position p is part p // blocks (2 of the 8 x-points of each thread) of block
    p % blocks."""
    voly, volx = energygrid.shape
    gdx, gdy = volx // 128, voly // 8
    if end is None:
        end = gdx * gdy * parts
    atominfo = np.ascontiguousarray(atominfo, np.float32).reshape(-1)
    out = np.array(energygrid, np.float32, order="C")
    lib().orc_cp_gptb(atominfo.size // 4, gridspacing, out.reshape(-1), atominfo, gdx, gdy, parts, start, end)
    return out


# --------------------------------------------------------------------------- sgemm
SGEMM_K_CHUNK = 64


def sgemm_positions(M, N, K, chunk=SGEMM_K_CHUNK):
    return (M // 128) * (N // 16) * -(-K // chunk)


def sgemm(A, B, Cm, start=0, end=None, parts=1, W=None, chunk=SGEMM_K_CHUNK):
    """C = 2 C + 2 A B with A [K][M], B [K][N], C [N][M] float32 (M multiple of 128, N of 16).

    Block positions [start, end) of the (M/128, N/16, parts) grid: parts=1, a position is a block's whole
    k loop (the reference's kernel); parts='chunks', position p adds k part p // blocks (chunk k steps) to
    block p % blocks, partial results resting in W ([N][M], updated in place when given) between parts.
    Returns the new C."""
    A = np.ascontiguousarray(A, np.float32)
    B = np.ascontiguousarray(B, np.float32)
    K, M = A.shape
    N = B.shape[1]
    assert B.shape[0] == K and Cm.shape == (N, M) and M % 128 == 0 and N % 16 == 0
    gdx, gdy = M // 128, N // 16
    if parts == "chunks":
        parts = -(-K // chunk)
    if end is None:
        end = gdx * gdy * parts
    out = np.array(Cm, np.float32, order="C")
    if W is None:
        W = np.zeros((N, M), np.float32)
    assert W.dtype == np.float32 and W.flags["C_CONTIGUOUS"] and W.shape == (N, M)
    lib().orc_sgemm_gptb(A.reshape(-1), B.reshape(-1), out.reshape(-1), W.reshape(-1), M, N, K, gdx, gdy, parts,
                         chunk, start, end)
    return out


# --------------------------------------------------------------------------- cutcp
def cutcp_prepare(atoms, lo, nx, ny, nz, h, cutoff):
    """prepare_input of the reference: dict with binDim (x, y, z), padding, bins [z][y][x][8][4] float32
    (padding bins included), nbr [n][3] int32, extra, excluded."""
    atoms = np.ascontiguousarray(atoms, np.float32).reshape(-1, 4)
    lo = np.ascontiguousarray(lo, np.float32)
    dims, pad, counts = np.zeros(3, np.int32), np.zeros(1, np.int32), np.zeros(2, np.int32)
    nbr = np.zeros((1331, 3), np.int32)
    n = lib().orc_cutcp_prepare(atoms.reshape(-1), len(atoms), lo, nx, ny, nz, h, cutoff, dims, pad, None,
                                nbr.ctypes.data, counts)
    if n < 0:
        raise ValueError("cutcp: spacing or cutoff outside what the neighbour list covers")
    bins = np.zeros((int(dims[2]), int(dims[1]), int(dims[0]), 8, 4), np.float32)
    lib().orc_cutcp_prepare(atoms.reshape(-1), len(atoms), lo, nx, ny, nz, h, cutoff, dims, pad, bins.ctypes.data,
                            nbr.ctypes.data, counts)
    return {"binDim": tuple(int(d) for d in dims), "padding": int(pad[0]), "bins": bins, "nbr": nbr[:n].copy(),
            "extra": int(counts[0]), "excluded": int(counts[1])}


CUTCP_NBR_CHUNK = 32


def cutcp_positions(regions, nbr_len, chunk=CUTCP_NBR_CHUNK):
    return regions[0] * regions[1] * regions[2] * max(1, -(-nbr_len // chunk))


def cutcp(prep, h, cutoff2, inv_cutoff2, regions, start=0, end=None, out=None, parts=1, chunk=CUTCP_NBR_CHUNK):
    """Energies [regions z][y][x][8][8][8] float32 (point (x, y, z) of a region at [z][y][x]) after the block
    positions [start, end) of the (regions) x (parts) grid: parts=1, a position is a region's whole neighbour
    list in ascending order (the reference's kernel); parts='chunks', the list is dealt round-robin into
    ceil(len / chunk) parts and position p adds part p // regions (entries part, part + parts, ...) to region
    p % regions, going on from the energies in ``out``.  Other regions keep what ``out`` holds (zeros)."""
    rx, ry, rz = regions
    bins = prep["bins"]
    c = prep["padding"]
    bdx, bdy = prep["binDim"][0], prep["binDim"][1]
    zero = bins.ctypes.data + (((c * bdy + c) * bdx + c) * 32) * 4
    res = np.zeros((rz, ry, rx, 8, 8, 8), np.float32) if out is None else np.array(out, np.float32, order="C")
    nbr = np.ascontiguousarray(prep["nbr"], np.int32)
    if parts == "chunks":
        parts = max(1, -(-len(nbr) // chunk))
    if end is None:
        end = rx * ry * rz * parts
    lib().orc_cutcp_gptb(bdx, bdy, zero, h, cutoff2, inv_cutoff2, res.ctypes.data, nbr.reshape(-1), len(nbr), rx, ry, rz,
                         parts, start, end)
    return res


# --------------------------------------------------------------------------- fft
FFT_N = 256


def fft(data, start=0, end=None):
    """Batched 256-point forward transforms, in place in the reference and returned here: data is
    [batches][256][2] float32 (re, im); block positions [start, end), position p = batch entry p % batches."""
    out = np.array(data, np.float32, order="C")
    assert out.ndim == 3 and out.shape[1:] == (FFT_N, 2)
    if end is None:
        end = out.shape[0]
    lib().orc_fft_gptb(out.reshape(-1), out.shape[0], start, end)
    return out


def fft_source(batches):
    """The reference's input: rand() after srand(54321), scaled to [-1, 1]."""
    out = np.zeros((batches, FFT_N, 2), np.float32)
    lib().orc_fft_source(out.reshape(-1), out.size)
    return out


# --------------------------------------------------------------------------- Rodinia partners
NN_BLOCK = 256
HOT3D_TILE = (64, 4)
PATH_BLOCK = 256


def nn_blocks(num_records):
    return (num_records - 1) // NN_BLOCK + 1 if num_records > 0 else 0


def nn(locations, lat, lng, out=None, start=0, end=None, grid=None, block=NN_BLOCK):
    """Distances of [n][2] float32 {lat, lng} records to (lat, lng); block positions [start, end) of
    `block` records over a grid (gx, gy) (default: all blocks in x).  Records no position covers
    keep `out`'s value (zeros if not given)."""
    loc = np.ascontiguousarray(locations, np.float32)
    n = loc.shape[0]
    res = np.zeros(n, np.float32) if out is None else np.array(out, np.float32)
    gx, gy = grid if grid is not None else ((n - 1) // block + 1, 1)
    if end is None:
        end = gx * gy
    lib().orc_nn_gptb(loc.reshape(-1), res, n, np.float32(lat), np.float32(lng), gx, gy, block, start, end)
    return res


def hot3d_coefficients(nx, ny, nz):
    out = np.zeros(8, np.float32)
    lib().orc_hot3d_coefficients(nx, ny, nz, out)
    return dict(zip(("sdc", "ce", "cw", "cn", "cs", "ct", "cb", "cc"), out))


def hot3d_blocks(nx, ny):
    return (nx // HOT3D_TILE[0]) * (ny // HOT3D_TILE[1])


def hot3d(p, t_in, coeff=None, out=None, start=0, end=None):
    """One hotspot3D step on [nz][ny][nx] float32 arrays; block positions [start, end) of 64 x 4
    columns.  Cells no position covers keep `out`'s value (zeros if not given)."""
    p = np.ascontiguousarray(p, np.float32)
    t = np.ascontiguousarray(t_in, np.float32)
    nz, ny, nx = t.shape
    k = coeff or hot3d_coefficients(nx, ny, nz)
    res = np.zeros_like(t) if out is None else np.array(out, np.float32)
    gx, gy = -(-nx // HOT3D_TILE[0]), -(-ny // HOT3D_TILE[1])
    if end is None:
        end = gx * gy
    f = np.float32
    lib().orc_hot3d_gptb(p.reshape(-1), t.reshape(-1), res.reshape(-1), f(k["sdc"]), nx, ny, nz, f(k["ce"]), f(k["cw"]),
                         f(k["cn"]), f(k["cs"]), f(k["ct"]), f(k["cb"]), f(k["cc"]), gx, gy, HOT3D_TILE[0],
                         HOT3D_TILE[1], start, end)
    return res


def path_blocks(cols, iteration):
    small = PATH_BLOCK - 2 * iteration
    return -(-cols // small) if small > 0 and cols > 0 else 0


def path(iteration, wall, src, out=None, start_step=0, start=0, end=None):
    """`iteration` rows of pathfinder from row start_step of wall ([rows - 1][cols] int32, the grid
    without its first row), src = [cols] int32; block positions [start, end).  Columns no position
    covers keep `out`'s value (zeros if not given)."""
    w = np.ascontiguousarray(wall, np.int32)
    s = np.ascontiguousarray(src, np.int32)
    cols = s.shape[0]
    res = np.zeros(cols, np.int32) if out is None else np.array(out, np.int32)
    if end is None:
        end = path_blocks(cols, iteration)
    lib().orc_path_gptb(iteration, w.reshape(-1), s, res, cols, start_step, iteration, start, end)
    return res


def path_source(rows, cols):
    out = np.zeros((rows, cols), np.int32)
    lib().orc_path_source(out.reshape(-1), out.size)
    return out


LAVA_PARTS = 27
LAVA_BOX = np.dtype([("x", "<i4"), ("y", "<i4"), ("z", "<i4"), ("number", "<i4"), ("offset", "<i8"), ("nn", "<i4"),
                     ("pad", "<i4"), ("nei", [("x", "<i4"), ("y", "<i4"), ("z", "<i4"), ("number", "<i4"),
                                              ("offset", "<i8")], 26)])


def lava_boxes(boxes1d):
    """The box list of a boxes1d^3 system as a structured array (the reference's box_str layout)."""
    assert lib().orc_lava_box_bytes() == LAVA_BOX.itemsize == 656
    out = np.zeros(boxes1d ** 3, LAVA_BOX)
    lib().orc_lava_boxes(boxes1d, out.ctypes.data)
    return out


def lava_blocks(boxes1d):
    return boxes1d ** 3 * LAVA_PARTS


def lava(alpha, boxes1d, rv, qv, fv=None, start=0, end=None):
    """lavaMD: rv [n][4] float32 {v, x, y, z}, qv [n] float32, n = 100 boxes1d^3; block positions
    [start, end) of the boxes x 27 parts grid added onto fv (zeros if not given)."""
    boxes = lava_boxes(boxes1d)
    r = np.ascontiguousarray(rv, np.float32)
    q = np.ascontiguousarray(qv, np.float32)
    f = np.zeros_like(r) if fv is None else np.array(fv, np.float32)
    if end is None:
        end = lava_blocks(boxes1d)
    lib().orc_lava_gptb(np.float32(alpha), boxes.ctypes.data, r.reshape(-1), q, f.reshape(-1), boxes1d ** 3, start, end)
    return f


# --------------------------------------------------------------------------- conv helpers
def mnk_from_conv_args(args14):
    a = np.asarray(args14, np.int32)
    out = np.zeros(3, np.int32)
    lib().orc_mnk_from_conv_args(a, out)
    return [int(v) for v in out]


def im2col(data_im, kernel, pad, stride, dilation=(1, 1)):
    """data_im [C][H][W] -> col [C*kh*kw][Ho][Wo] (Caffe layout)."""
    data_im = np.ascontiguousarray(data_im, np.float32)
    Cc, H, W = data_im.shape
    kh, kw = kernel
    ph, pw = pad
    sh, sw = stride
    dh, dw = dilation
    Ho = (H + 2 * ph - (dh * (kh - 1) + 1)) // sh + 1
    Wo = (W + 2 * pw - (dw * (kw - 1) + 1)) // sw + 1
    col = np.zeros((Cc * kh * kw, Ho, Wo), np.float32)
    lib().orc_im2col(Cc * Ho * Wo, data_im.reshape(-1), H, W, kh, kw, ph, pw, sh, sw, dh, dw, Ho, Wo,
                     col.reshape(-1))
    return col
