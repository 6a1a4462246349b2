/*
 * tacker_oracle.c -- CPU restatement of the reference's hot-path kernels.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the parity checker for the HIP path
 * and the "port" CPU baseline of the benchmark.  Nothing in the product
 * (tacker_amd/) may include, link, load or call it.
 *
 * Every function restates one reference function in plain C with the
 * reference's own operation order (compile with -ffp-contract=off so that no
 * multiply-add is fused behind our back).  Citations are relative to the
 * reference tree (sjtu-epcc/Tacker).
 *
 * Pinning status (what fixes each function besides "we typed it"):
 *   orc_tzgemm_dims       known answers held by the reference: the K keys
 *                         128/512/1152/2304/4608 of src/config/kinfo-vgg16.json:8-12
 *                         and (12800,512,4096) of src/Creator.cu:255-261.
 *   orc_tzgemm_*          closed forms (A=I, all-ones), bijection of the tile
 *                         map, numpy float64 matmul.
 *   orc_stencil*          harmonic fields -> 0, constant field, numpy roll
 *                         formulation in float64, boundary invariance.
 *   orc_lbm*              obstacle = exact permutation, mass / momentum
 *                         conservation, rest-equilibrium fixed point,
 *                         independent numpy formulation.
 *   orc_mriq*             x=0 closed form, single-k closed form, numpy
 *                         float64 brute force; block-by-chunk positions: any
 *                         ascending tiling = the one k loop bit for bit, one
 *                         position = numpy float64 over its record range.
 *   orc_mrif*             x=0 closed form, single-k closed form, numpy complex128
 *                         sum conj(phi) d e^{i 2 pi k.x}; block-by-chunk
 *                         positions as orc_mriq.
 *   orc_cp*               single atom closed form, numpy float64 brute force,
 *                         ori_blks = 16384 held by fusion/code/kinfo.json.
 *   orc_sgemm_gptb        float64 matrix product, integer operands (exact), one-hot A, the
 *                         fused multiply-add per step against exact rationals, any
 *                         ascending tiling of the position grid (tests/test_oracle_sgemm.py).
 *   orc_cutcp*            float64 sum over the atom list without bins, single-charge closed form and
 *                         exact zero outside the cutoff, binning against a Python dictionary,
 *                         neighbour list by its inequality, the 32 x 32 bin grid the reference
 *                         hard-codes, any ascending tiling of the region-by-part grid
 *                         (tests/test_oracle_cutcp.py).
 *   orc_fft*              the float64 transform (numpy's FFT and the defining sum), unit
 *                         impulses = rows of the DFT matrix, pure tones, linearity,
 *                         Parseval, position wrap; the input stream against the cp atoms'
 *                         draw of the same seeded rand().
 *   orc_nn_gptb           3-4-5 and axis-aligned known answers, numpy float64 hypot, the float32
 *                         vectorised evaluation, block wrap and the record-count tail, any tiling
 *                         of the block positions (tests/test_oracle_rodinia.py).
 *   orc_hot3d_gptb        the ambient temperature as a fixed point, a constant field's closed
 *                         form T (1 - ct) + ct 80, heat content conserved inside an insulated
 *                         chip but for the top face's term, an edge-padded numpy formulation
 *                         in float64 and in float32, the coefficients against Rodinia's formulas
 *                         in float64, any tiling of the positions.
 *   orc_path_gptb         the textbook row-by-row dynamic programme over the whole grid (numpy),
 *                         brute force over all paths on a tiny wall, window edges at both ends of
 *                         the grid, column counts that are not a multiple of the window's yield,
 *                         any tiling of the positions; the input stream against rand() % 10.
 *   orc_lava*             the neighbour lists by count (corner 7, edge 11, face 17, inside 26) and
 *                         by symmetry, a float64 numpy evaluation of the same sums over the same
 *                         lists, a single pair's closed form, equal charges => the forces of all
 *                         particles sum to zero, any ascending tiling of the box-by-part grid
 *                         (tests/test_oracle_rodinia.py).
 *   orc_im2col            direct convolution brute force.
 *   orc_gptb_index        partition invariance (any launch grid covers every
 *                         block once).
 * Unpinned at the bit level (tolerance applies): the reference's WMMA
 * accumulation order and the CUDA libdevice sin/cos last-ulp behaviour; no
 * reference file holds golden outputs for them.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------ */
/* fp16 helpers                                                             */
/* ------------------------------------------------------------------------ */

static float half_bits_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: renormalise */
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while (!(man & 0x400u));
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

ORC_API int orc_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------------ */
/* tzgemm                                                                   */
/* ------------------------------------------------------------------------ */

/* src/tzgemm_kernel.h:30-48 getTZGEMMGridDim: floor to multiples of 128 (min
 * 128); tiles = (M/16 * N/16) / (4*4) 64x64 CTA tiles. */
ORC_API void orc_tzgemm_dims(int m, int n, int k, int out[4])
{
    int M = (m < 128) ? 128 : (m / 128) * 128;
    int N = (n < 128) ? 128 : (n / 128) * 128;
    int K = (k < 128) ? 128 : (k / 128) * 128;
    int m_tiles = M / 16, n_tiles = N / 16;
    out[0] = M;
    out[1] = N;
    out[2] = K;
    out[3] = (m_tiles * n_tiles) / (4 * 4);
}

/* src/mix_kernel/tzgemm_stencil.cu:54-56: origin (in elements) of CTA tile
 * block_pos.  tile_i = ((pos*4)/N_TILES)*4, tile_j = (pos*4)%N_TILES in units
 * of 16. */
ORC_API void orc_tzgemm_tile_origin(unsigned pos, int N, int *row0, int *col0)
{
    unsigned n_tiles = (unsigned)N / 16u;
    unsigned ti = ((pos * 4u) / n_tiles) * 4u;
    unsigned tj = (pos * 4u) % n_tiles;
    *row0 = (int)(ti * 16u);
    *col0 = (int)(tj * 16u);
}

/* src/mix_kernel/tzgemm_stencil.cu:5-172 (fp16 branch, int2 store):
 * C[i][j] = alpha * sum_k float(A[i][k]) * float(B[j][k]) for the 64x64 tiles
 * block_pos in [start,end); other elements of C are left untouched.  A is
 * [M][K], B is [N][K], C is [M][N], all row-major.  accumulate_f64 = 0: fp32
 * sequential accumulation (tolerance witness); 1: fp64 accumulation (truth).
 * alpha is applied once after the K reduction (:152), in fp32. */
ORC_API void orc_tzgemm(const uint16_t *A, const uint16_t *B, float *C, int M, int N, int K,
                        float alpha, int start, int end, int accumulate_f64)
{
    (void)M;
    float *Af = (float *)malloc(sizeof(float) * (size_t)M * K);
    float *Bf = (float *)malloc(sizeof(float) * (size_t)N * K);
    for (size_t i = 0; i < (size_t)M * K; i++) Af[i] = half_bits_to_float(A[i]);
    for (size_t i = 0; i < (size_t)N * K; i++) Bf[i] = half_bits_to_float(B[i]);
#pragma omp parallel for schedule(dynamic, 1)
    for (int pos = start; pos < end; pos++) {
        int r0, c0;
        orc_tzgemm_tile_origin((unsigned)pos, N, &r0, &c0);
        for (int i = r0; i < r0 + 64; i++) {
            const float *a = Af + (size_t)i * K;
            for (int j = c0; j < c0 + 64; j++) {
                const float *b = Bf + (size_t)j * K;
                if (accumulate_f64) {
                    double acc = 0.0;
                    for (int k = 0; k < K; k++) acc += (double)a[k] * (double)b[k];
                    C[(size_t)i * N + j] = (float)((double)alpha * acc);
                } else {
                    float acc = 0.0f;
                    for (int k = 0; k < K; k++) acc = acc + a[k] * b[k];
                    C[(size_t)i * N + j] = acc * alpha;
                }
            }
        }
    }
    free(Af);
    free(Bf);
}

/* ------------------------------------------------------------------------ */
/* GPTB index reconstruction                                                */
/* ------------------------------------------------------------------------ */

/* src/gptb_kernel/stencil_kernel.cu:6-24, cp_kernel.cu:13-41: a linear
 * block_pos and a role-local thread index t = threadIdx.x - thread_base are
 * unfolded into (block_id_x, block_id_y) and (thread_id_x, thread_id_y).
 * block_id_y wraps modulo grid_dimension_y. out = {bx, by, tx, ty}. */
ORC_API void orc_gptb_index(unsigned block_pos, int t, int grid_dimension_x, int grid_dimension_y,
                            int block_dimension_x, int block_dimension_y, int out[4])
{
    out[0] = (int)(block_pos % (unsigned)grid_dimension_x);
    out[1] = (int)((block_pos / (unsigned)grid_dimension_x) % (unsigned)grid_dimension_y);
    out[2] = t % block_dimension_x;
    out[3] = (t / block_dimension_x) % block_dimension_y;
}

/* ------------------------------------------------------------------------ */
/* stencil                                                                  */
/* ------------------------------------------------------------------------ */

#define IDX3(nx, ny, i, j, k) ((size_t)(i) + (size_t)(nx) * ((size_t)(j) + (size_t)(ny) * (size_t)(k)))

/* One block of src/ori_kernel/stencil_kernel.cu:9-94 (= general_ptb_stencil
 * body, src/gptb_kernel/stencil_kernel.cu:26-102): block (bx,by) of
 * block_dimension (bdx,bdy) covers x in [2*bdx*bx, 2*bdx*bx + 2*bdx),
 * y in [bdy*by, bdy*by + bdy), marches k = k_lo .. k_hi-1 (the reference: 1 .. nz-2). */
static void stencil_block(float c0, float c1, const float *A0, float *Anext, int nx, int ny, int nz,
                          int bx, int by, int bdx, int bdy, int k_lo, int k_hi)
{
    (void)nz;
    for (int ty = 0; ty < bdy; ty++) {
        int j = by * bdy + ty;
        for (int half = 0; half < 2; half++) {
            for (int tx = 0; tx < bdx; tx++) {
                int i = bx * bdx * 2 + tx + half * bdx;
                /* :26-27 write regions */
                int w = (half == 0) ? (i > 0 && j > 0 && i < nx - 1 && j < ny - 1)
                                    : (j > 0 && i < nx - 1 && j < ny - 1);
                if (!w) continue;
                for (int k = k_lo; k < k_hi; k++) {
                    float top = A0[IDX3(nx, ny, i, j, k + 1)];
                    float bottom = A0[IDX3(nx, ny, i, j, k - 1)];
                    float up = A0[IDX3(nx, ny, i, j + 1, k)];
                    float down = A0[IDX3(nx, ny, i, j - 1, k)];
                    float right = A0[IDX3(nx, ny, i + 1, j, k)];
                    float left = A0[IDX3(nx, ny, i - 1, j, k)];
                    float centre = A0[IDX3(nx, ny, i, j, k)];
                    /* :68-69 and :82-83: same association order for both halves */
                    float s = top + bottom;
                    s = s + up;
                    s = s + down;
                    s = s + right;
                    s = s + left;
                    float p = s * c1;
                    float q = centre * c0;
                    Anext[IDX3(nx, ny, i, j, k)] = p - q;
                }
            }
        }
    }
}

/* GPTB form: block positions [start,end) of a (gdx,gdy,gdz) grid of (bdx,bdy) blocks, index
 * reconstruction as in the reference's kernels (block_id_x = pos % gdx, block_id_y =
 * pos / gdx % gdy, src/gptb_kernel/stencil_kernel.cu:22-24; block_id_z = pos / (gdx*gdy) % gdz
 * as in its 3-D kernels).  The z index cuts the march of a block column: with
 * runs = ceil((nz-2) / zrun) runs of zrun centre planes, position p computes the runs
 * [part*runs/gdz, (part+1)*runs/gdz) of block p % (gdx*gdy), part = p / (gdx*gdy) % gdz.
 * gdz = 1: a position is a whole block column, the reference's kernel. */
ORC_API void orc_stencil_gptb(float c0, float c1, const float *A0, float *Anext, int nx, int ny,
                              int nz, int gdx, int gdy, int gdz, int bdx, int bdy, int zrun, int start, int end)
{
    if (nz < 3 || gdz < 1 || zrun < 1) return;
    const int runs = (nz - 2 + zrun - 1) / zrun;
#pragma omp parallel for schedule(static)
    for (int pos = start; pos < end; pos++) {
        int bx = pos % gdx;
        int by = (pos / gdx) % gdy;
        int part = (pos / (gdx * gdy)) % gdz;
        int k_lo = 1 + (part * runs / gdz) * zrun;
        int k_hi = 1 + ((part + 1) * runs / gdz) * zrun;
        if (k_hi > nz - 1) k_hi = nz - 1;
        stencil_block(c0, c1, A0, Anext, nx, ny, nz, bx, by, bdx, bdy, k_lo, k_hi);
    }
}

/* Ori form: the natural grid (ceil(nx/64), ceil(ny/4)) of (32,4) blocks,
 * src/ori_kernel/stencil_kernel.cu:166-173. */
ORC_API void orc_stencil(float c0, float c1, const float *A0, float *Anext, int nx, int ny, int nz)
{
    int gdx = (nx + 32 * 2 - 1) / (32 * 2);
    int gdy = (ny + 4 - 1) / 4;
    orc_stencil_gptb(c0, c1, A0, Anext, nx, ny, nz, gdx, gdy, 1, 32, 4, nz, 0, gdx * gdy);
}

/* ------------------------------------------------------------------------ */
/* lbm                                                                      */
/* ------------------------------------------------------------------------ */

/* Entry order, src/header/lbm_header.h:228-233. */
enum { LC = 0, LN, LS, LE, LW, LT, LB, LNE, LNW, LSE, LSW, LNT, LNB, LST, LSB, LET, LEB, LWT, LWB,
       LFLAGS, L_ENTRIES };

/* Direction of each entry, src/header/lbm_header.h:102-121. */
static const int lbm_dx[19] = {0, 0, 0, +1, -1, 0, 0, +1, -1, +1, -1, 0, 0, 0, 0, +1, +1, -1, -1};
static const int lbm_dy[19] = {0, +1, -1, 0, 0, 0, 0, +1, +1, -1, -1, +1, +1, -1, -1, 0, 0, 0, 0};
static const int lbm_dz[19] = {0, 0, 0, 0, 0, +1, -1, 0, 0, 0, 0, +1, -1, +1, -1, +1, -1, +1, -1};

/* One cell of src/ori_kernel/lbm_kernel.cu:9-154.  src/dst point at entry
 * plane 0 of cell (0,0,0) (i.e. base + REAL_MARGIN).  SoA layout
 * CALC_INDEX(x,y,z,e) = cells*e + x + y*sx + z*sx*sy (lbm_header.h:43-44),
 * SCATTER mode (:47-51), no boundary clamping: the neighbour is reached by
 * linear index arithmetic.
 *
 * A scatter whose linear target cell index falls outside [0, cells) would land
 * in the adjacent entry plane, where the reference has a write-write race with
 * that plane's in-range writer (two threads, two values, one address).  This
 * restatement resolves the race the same way on every run: the in-range
 * writer wins, i.e. the out-of-range store is dropped. */
static void lbm_cell(const float *src, float *dst, long cells, long c, const long off[19])
{
    float f[19];
    for (int e = 0; e < 19; e++) f[e] = src[cells * e + c];
    uint32_t flags;
    memcpy(&flags, &src[cells * LFLAGS + c], 4);

    if (flags & 1u) { /* OBSTACLE: :49-57 */
        float t;
        t = f[LN]; f[LN] = f[LS]; f[LS] = t;
        t = f[LE]; f[LE] = f[LW]; f[LW] = t;
        t = f[LT]; f[LT] = f[LB]; f[LB] = t;
        t = f[LNE]; f[LNE] = f[LSW]; f[LSW] = t;
        t = f[LNW]; f[LNW] = f[LSE]; f[LSE] = t;
        t = f[LNT]; f[LNT] = f[LSB]; f[LSB] = t;
        t = f[LNB]; f[LNB] = f[LST]; f[LST] = t;
        t = f[LET]; f[LET] = f[LWB]; f[LWB] = t;
        t = f[LEB]; f[LEB] = f[LWT]; f[LWT] = t;
    } else {
        float ux, uy, uz, rho, u2, temp1, temp2, temp_base;
        /* :63-72 */
        rho = f[LC] + f[LN];
        rho = rho + f[LS]; rho = rho + f[LE]; rho = rho + f[LW]; rho = rho + f[LT];
        rho = rho + f[LB]; rho = rho + f[LNE]; rho = rho + f[LNW]; rho = rho + f[LSE];
        rho = rho + f[LSW]; rho = rho + f[LNT]; rho = rho + f[LNB]; rho = rho + f[LST];
        rho = rho + f[LSB]; rho = rho + f[LET]; rho = rho + f[LEB]; rho = rho + f[LWT];
        rho = rho + f[LWB];
        /* :74-88 (unary plus, then left to right) */
        ux = f[LE] - f[LW];
        ux = ux + f[LNE]; ux = ux - f[LNW]; ux = ux + f[LSE]; ux = ux - f[LSW];
        ux = ux + f[LET]; ux = ux + f[LEB]; ux = ux - f[LWT]; ux = ux - f[LWB];
        uy = f[LN] - f[LS];
        uy = uy + f[LNE]; uy = uy + f[LNW]; uy = uy - f[LSE]; uy = uy - f[LSW];
        uy = uy + f[LNT]; uy = uy + f[LNB]; uy = uy - f[LST]; uy = uy - f[LSB];
        uz = f[LT] - f[LB];
        uz = uz + f[LNT]; uz = uz - f[LNB]; uz = uz + f[LST]; uz = uz - f[LSB];
        uz = uz + f[LET]; uz = uz - f[LEB]; uz = uz + f[LWT]; uz = uz - f[LWB];
        ux = ux / rho; /* :90-92 */
        uy = uy / rho;
        uz = uz / rho;
        if (flags & 2u) { /* ACCEL :93-97 */
            ux = 0.005f;
            uy = 0.002f;
            uz = 0.000f;
        }
        {
            float a = ux * ux, b = uy * uy, cc = uz * uz;
            float s = a + b;
            s = s + cc;
            u2 = 1.5f * s;
            u2 = u2 - 1.0f; /* :98 */
        }
        const float OMEGA = 1.95f;
        const float DFL1 = 1.0f / 3.0f, DFL2 = 1.0f / 18.0f, DFL3 = 1.0f / 36.0f;
        temp_base = OMEGA * rho;
        temp1 = DFL1 * temp_base;
        temp2 = 1.0f - OMEGA;
#define LBM_RELAX(entry, expr)                 \
    do {                                       \
        float lhs_ = temp2 * f[entry];         \
        float e_ = (expr);                     \
        float rhs_ = temp1 * e_;               \
        f[entry] = lhs_ + rhs_;                \
    } while (0)
#define LBM_Q(v, sgn) ((v) * (4.5f * (v) + (sgn)) - u2)
        LBM_RELAX(LC, -u2); /* :105 */
        temp1 = DFL2 * temp_base;
        LBM_RELAX(LN, LBM_Q(uy, 3.0f));
        LBM_RELAX(LS, uy * (4.5f * uy - 3.0f) - u2);
        LBM_RELAX(LT, LBM_Q(uz, 3.0f));
        LBM_RELAX(LB, uz * (4.5f * uz - 3.0f) - u2);
        LBM_RELAX(LE, LBM_Q(ux, 3.0f));
        LBM_RELAX(LW, ux * (4.5f * ux - 3.0f) - u2);
        temp1 = DFL3 * temp_base;
        {
            float v;
            v = (+uy + uz); LBM_RELAX(LNT, LBM_Q(v, 3.0f));
            v = (+uy - uz); LBM_RELAX(LNB, LBM_Q(v, 3.0f));
            v = (-uy + uz); LBM_RELAX(LST, LBM_Q(v, 3.0f));
            v = (-uy - uz); LBM_RELAX(LSB, LBM_Q(v, 3.0f));
            v = (+ux + uy); LBM_RELAX(LNE, LBM_Q(v, 3.0f));
            v = (+ux - uy); LBM_RELAX(LSE, LBM_Q(v, 3.0f));
            v = (+ux + uz); LBM_RELAX(LET, LBM_Q(v, 3.0f));
            v = (+ux - uz); LBM_RELAX(LEB, LBM_Q(v, 3.0f));
            v = (-ux + uy); LBM_RELAX(LNW, LBM_Q(v, 3.0f));
            v = (-ux - uy); LBM_RELAX(LSW, LBM_Q(v, 3.0f));
            v = (-ux + uz); LBM_RELAX(LWT, LBM_Q(v, 3.0f));
            v = (-ux - uz); LBM_RELAX(LWB, LBM_Q(v, 3.0f));
        }
#undef LBM_RELAX
#undef LBM_Q
    }
    for (int e = 0; e < 19; e++) { /* :133-153 scatter */
        long t = c + off[e];
        if (t >= 0 && t < cells) dst[cells * e + t] = f[e];
    }
}

/* GPTB form (src/gptb_kernel/lbm_kernel.cu:3-178): block_pos -> (y,z) with
 * y = pos % sy, z = (pos / sy) % sz; thread_id_x = x in [0,sx).  The grid is
 * (sy,sz) blocks of sx threads (src/ori_kernel/lbm_kernel.cu:218-222). */
ORC_API void orc_lbm_gptb(const float *src, float *dst, int sx, int sy, int sz, int start, int end)
{
    long cells = (long)sx * sy * sz;
    long off[19];
    for (int e = 0; e < 19; e++) off[e] = lbm_dx[e] + (long)lbm_dy[e] * sx + (long)lbm_dz[e] * sx * sy;
#pragma omp parallel for schedule(static)
    for (int pos = start; pos < end; pos++) {
        int y = pos % sy;
        int z = (pos / sy) % sz;
        for (int x = 0; x < sx; x++) {
            long c = x + (long)y * sx + (long)z * sx * sy;
            lbm_cell(src, dst, cells, c, off);
        }
    }
}

ORC_API void orc_lbm(const float *src, float *dst, int sx, int sy, int sz)
{
    orc_lbm_gptb(src, dst, sx, sy, sz, 0, sy * sz);
}

/* ------------------------------------------------------------------------ */
/* mri-q                                                                    */
/* ------------------------------------------------------------------------ */

/* src/ori_kernel/mriq_kernel.cu:47-54 */
ORC_API void orc_mriq_phimag(const float *phiR, const float *phiI, float *phiMag, int numK)
{
    for (int k = 0; k < numK; k++) {
        float real = phiR[k];
        float imag = phiI[k];
        float a = real * real, b = imag * imag;
        phiMag[k] = a + b;
    }
}

/* src/ori_kernel/mriq_kernel.cu:56-105 with the k loop running over all numK
 * samples (the reference's "QGrid < 1" loop stops after the first 1024-sample
 * chunk, :58-59; the intended Parboil semantics is every chunk in order, which
 * for one voxel is simply k = 0..numK-1 in sequence).  kvals is the AoS table
 * {Kx,Ky,Kz,PhiMag} (src/header/mriq_header.h:12-17).
 *
 * GPTB form (src/gptb_kernel/mriq_kernel.cu:17-33 index reconstruction, with the
 * host's loop over k chunks, src/ori_kernel/mriq_kernel.cu:258-283, as the y index
 * of the grid): block positions [start,end) of a gdx x gdy grid; position p adds
 * the records [c*kchunk, min(numK,(c+1)*kchunk)) of chunk c = (p / gdx) % gdy to
 * the 256 voxels (KERNEL_Q_THREADS_PER_BLOCK) of block p % gdx, positions in
 * ascending order.  gdy = 1 and kchunk >= numK is the plain form: every position
 * adds the whole table.  Read-modify-write on Qr/Qi.  f64 = 1: double arithmetic
 * throughout (truth), written back as float once per position. */
static void orc_mriq_voxel(int k0, int k1, const float *kvals, const float *x, const float *y,
                           const float *z, float *Qr, float *Qi, int xi, int f64)
{
    const float PIx2 = 6.2831853071795864769252867665590058f;
    if (f64) {
        double sx = x[xi], sy = y[xi], sz = z[xi];
        double qr = Qr[xi], qi = Qi[xi];
        for (int k = k0; k < k1; k++) {
            const float *kv = kvals + 4 * (size_t)k;
            double arg = 6.2831853071795864769252867665590058 *
                         ((double)kv[0] * sx + (double)kv[1] * sy + (double)kv[2] * sz);
            qr += (double)kv[3] * cos(arg);
            qi += (double)kv[3] * sin(arg);
        }
        Qr[xi] = (float)qr;
        Qi[xi] = (float)qi;
    } else {
        float sx = x[xi], sy = y[xi], sz = z[xi];
        float qr = Qr[xi], qi = Qi[xi];
        for (int k = k0; k < k1; k++) {
            const float *kv = kvals + 4 * (size_t)k;
            float a = kv[0] * sx, b = kv[1] * sy, c = kv[2] * sz;
            float d = a + b;
            d = d + c;
            float arg = PIx2 * d;
            float pc = kv[3] * cosf(arg);
            float ps = kv[3] * sinf(arg);
            qr = qr + pc;
            qi = qi + ps;
        }
        Qr[xi] = qr;
        Qi[xi] = qi;
    }
}

ORC_API void orc_mriq_gptb(int numK, const float *kvals, const float *x, const float *y,
                           const float *z, float *Qr, float *Qi, int gdx, int gdy, int kchunk,
                           int start, int end, int f64)
{
    /* one thread per voxel block; its positions are start-aligned p, p+gdx, ... in order */
#pragma omp parallel for schedule(static)
    for (int bx = 0; bx < gdx; bx++) {
        int first = start + ((bx - start % gdx) + gdx) % gdx;
        for (int pos = first; pos < end; pos += gdx) {
            int chunk = (pos / gdx) % gdy;
            long k0 = (long)chunk * kchunk, k1 = k0 + kchunk;
            if (k0 > numK) k0 = numK;
            if (k1 > numK) k1 = numK;
            for (int t = 0; t < 256; t++)
                orc_mriq_voxel((int)k0, (int)k1, kvals, x, y, z, Qr, Qi, bx * 256 + t, f64);
        }
    }
}

/* ------------------------------------------------------------------------ */
/* mri-fhd                                                                  */
/* ------------------------------------------------------------------------ */

/* src/ori_kernel/mrif_kernel.cu:62-75: RhoPhi = conj(phi) * d */
ORC_API void orc_mrif_rhophi(int numK, const float *phiR, const float *phiI, const float *dR,
                             const float *dI, float *realRhoPhi, float *imagRhoPhi)
{
    for (int k = 0; k < numK; k++) {
        float a = phiR[k] * dR[k], b = phiI[k] * dI[k];
        float c = phiR[k] * dI[k], d = phiI[k] * dR[k];
        realRhoPhi[k] = a + b;
        imagRhoPhi[k] = c - d;
    }
}

/* src/ori_kernel/mrif_kernel.cu:77-152 with the k loop running over all numK
 * samples (the reference's "FHGrid < 1" loop stops after the first grid of 256,
 * :84-85).  kvals is the AoS table {Kx,Ky,Kz,RhoPhiR,RhoPhiI}
 * (src/header/mrif_header.h:23-29).  Block positions as orc_mriq_gptb
 * (src/gptb_kernel/mrif_kernel.cu:113-125 index reconstruction). */
static void orc_mrif_voxel(int k0, int k1, const float *kvals, const float *x, const float *y,
                           const float *z, float *outR, float *outI, int xi, int f64)
{
    const float PIx2 = 6.2831853071795864769252867665590058f;
    if (f64) {
        double sx = x[xi], sy = y[xi], sz = z[xi];
        double r = outR[xi], i = outI[xi];
        for (int k = k0; k < k1; k++) {
            const float *kv = kvals + 5 * (size_t)k;
            double arg = 6.2831853071795864769252867665590058 *
                         ((double)kv[0] * sx + (double)kv[1] * sy + (double)kv[2] * sz);
            double c = cos(arg), sn = sin(arg);
            r += (double)kv[3] * c - (double)kv[4] * sn;
            i += (double)kv[4] * c + (double)kv[3] * sn;
        }
        outR[xi] = (float)r;
        outI[xi] = (float)i;
    } else {
        float sx = x[xi], sy = y[xi], sz = z[xi];
        float r = outR[xi], i = outI[xi];
        for (int k = k0; k < k1; k++) {
            const float *kv = kvals + 5 * (size_t)k;
            float a = kv[0] * sx, b = kv[1] * sy, c = kv[2] * sz;
            float d = a + b;
            d = d + c;
            float arg = PIx2 * d;
            float cs = cosf(arg), sn = sinf(arg);
            float rc = kv[3] * cs, is = kv[4] * sn;
            float ic = kv[4] * cs, rs = kv[3] * sn;
            float re = rc - is, im = ic + rs;
            r = r + re;
            i = i + im;
        }
        outR[xi] = r;
        outI[xi] = i;
    }
}

ORC_API void orc_mrif_gptb(int numK, const float *kvals, const float *x, const float *y,
                           const float *z, float *outR, float *outI, int gdx, int gdy, int kchunk,
                           int start, int end, int f64)
{
#pragma omp parallel for schedule(static)
    for (int bx = 0; bx < gdx; bx++) {
        int first = start + ((bx - start % gdx) + gdx) % gdx;
        for (int pos = first; pos < end; pos += gdx) {
            int chunk = (pos / gdx) % gdy;
            long k0 = (long)chunk * kchunk, k1 = k0 + kchunk;
            if (k0 > numK) k0 = numK;
            if (k1 > numK) k1 = numK;
            for (int t = 0; t < 256; t++)
                orc_mrif_voxel((int)k0, (int)k1, kvals, x, y, z, outR, outI, bx * 256 + t, f64);
        }
    }
}

/* ------------------------------------------------------------------------ */
/* cp                                                                       */
/* ------------------------------------------------------------------------ */

/* src/ori_kernel/cp_kernel.cu:185-209 initatoms: glibc srand(54321), four
 * rand() per atom in the order x,y,z,q.  The box is dim3 (unsigned) so
 * gridspacing*volsize truncates: 0.1f*4096 -> 409, 0.1f*1 -> 0. */
ORC_API void orc_cp_initatoms(float *atoms, int count, unsigned volx, unsigned voly, unsigned volz,
                              float gridspacing)
{
    unsigned sizex = (unsigned)(gridspacing * volx);
    unsigned sizey = (unsigned)(gridspacing * voly);
    unsigned sizez = (unsigned)(gridspacing * volz);
    srand(54321);
    for (int i = 0; i < count; i++) {
        int addr = i * 4;
        atoms[addr] = (rand() / (float)RAND_MAX) * sizex;
        atoms[addr + 1] = (rand() / (float)RAND_MAX) * sizey;
        atoms[addr + 2] = (rand() / (float)RAND_MAX) * sizez;
        atoms[addr + 3] = (float)(((rand() / (float)RAND_MAX) * 2.0) - 1.0);
    }
}

/* src/ori_kernel/cp_kernel.cu:159-179 copyatomstoconstbuf: z is replaced by
 * (zplane - z)^2. */
ORC_API void orc_cp_atoms_to_const(const float *atoms, int count, float zplane, float *atominfo)
{
    for (int i = 0; i < count * 4; i += 4) {
        atominfo[i] = atoms[i];
        atominfo[i + 1] = atoms[i + 1];
        float dz = zplane - atoms[i + 2];
        atominfo[i + 2] = dz * dz;
        atominfo[i + 3] = atoms[i + 3];
    }
}

/* src/gptb_kernel/cp_kernel.cu:8-96 (= ori_cp, src/ori_kernel/cp_kernel.cu:26-79,
 * with blockIdx reconstructed): grid (gdx,gdy) of (16,8) blocks, each thread 8
 * x-points 16 apart.  energygrid has row pitch gdx*16*8.
 *
 * Block positions [start,end) of a (gdx,gdy,gdz) grid, index reconstruction as in
 * the reference's 3-D kernels (block_id_z = pos / (x*y) % z): position p computes,
 * for block p % (gdx*gdy), the x-points n in [part*8/gdz, (part+1)*8/gdz) of every
 * thread, part = (p / (gdx*gdy)) % gdz; dx of point n is reached by the chain of
 * additions of the 8-point loop.  gdz = 1: a position is a whole block.  Positions
 * of one block are applied in ascending order. */
ORC_API void orc_cp_gptb(int numatoms, float gridspacing, float *energygrid, const float *atominfo,
                         int gdx, int gdy, int gdz, int start, int end)
{
    const int BX = 16, BY = 8, UNROLLX = 8;
    const int blocks = gdx * gdy;
    const int per_part = UNROLLX / gdz;
#pragma omp parallel for schedule(static)
    for (int blk = 0; blk < blocks; blk++) {
        int first = start + ((blk - start % blocks) + blocks) % blocks;
        for (int pos = first; pos < end; pos += blocks) {
            unsigned bx = (unsigned)pos % (unsigned)gdx;
            unsigned by = ((unsigned)pos / (unsigned)gdx) % (unsigned)gdy;
            int part = (pos / blocks) % gdz;
            int n0 = part * per_part, n1 = n0 + per_part;
            for (unsigned ty = 0; ty < (unsigned)BY; ty++) {
                for (unsigned tx = 0; tx < (unsigned)BX; tx++) {
                    unsigned xindex = bx * BX * UNROLLX + tx;
                    unsigned yindex = by * BY + ty;
                    unsigned outaddr = ((unsigned)gdx * BX * UNROLLX) * yindex + xindex;
                    float coory = gridspacing * yindex;
                    float coorx = gridspacing * xindex;
                    float e[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                    float gridspacing_u = gridspacing * BX;
                    for (int a = 0; a < numatoms; a++) {
                        const float *at = atominfo + 4 * a;
                        float dy = coory - at[1];
                        float dy2 = dy * dy;
                        float dyz2 = dy2 + at[2];
                        float dx = coorx - at[0];
                        for (int n = 0; n < n1; n++) {
                            if (n >= n0) {
                                float dx2 = dx * dx;
                                float r2 = dx2 + dyz2;
                                float inv = 1.0f / sqrtf(r2);
                                float contrib = at[3] * inv;
                                e[n] = e[n] + contrib;
                            }
                            dx = dx + gridspacing_u;
                        }
                    }
                    for (int n = n0; n < n1; n++) {
                        float *p = &energygrid[outaddr + (unsigned)n * BX];
                        *p = *p + e[n];
                    }
                }
            }
        }
    }
}

/* ------------------------------------------------------------------------ */
/* conv -> GEMM helpers                                                     */
/* ------------------------------------------------------------------------ */

/* src/TaskManager.cu:92-123 get_mnk_from_cudnn_args: 14 ints
 * {n,c,h,w, k,c,kh,kw, pad_h,pad_w, stride_h,stride_w, dil_h,dil_w}. */
ORC_API void orc_mnk_from_conv_args(const int a[14], int mnk[3])
{
    int height_col = (a[2] + 2 * a[8] - (a[12] * (a[6] - 1) + 1)) / a[10] + 1;
    int width_col = (a[3] + 2 * a[9] - (a[13] * (a[7] - 1) + 1)) / a[11] + 1;
    mnk[0] = a[0] * height_col * width_col;
    mnk[1] = a[4];
    mnk[2] = a[6] * a[7] * a[1];
}

/* src/TaskManager.cu:48-82 im2col_gpu_kernel_ (Caffe im2col, NCHW): n =
 * channels*height_col*width_col work items (the batch dimension is folded into
 * channels by the caller). */
ORC_API void orc_im2col(int n, const float *data_im, int height, int width, int kernel_h,
                        int kernel_w, int pad_h, int pad_w, int stride_h, int stride_w,
                        int dilation_h, int dilation_w, int height_col, int width_col,
                        float *data_col)
{
    for (int i = 0; i < n; i++) {
        int h_index = i / width_col;
        int h_col = h_index % height_col;
        int w_col = i % width_col;
        int c_im = h_index / height_col;
        int c_col = c_im * kernel_h * kernel_w;
        int h_offset = h_col * stride_h - pad_h;
        int w_offset = w_col * stride_w - pad_w;
        float *col = data_col + ((size_t)c_col * height_col + h_col) * width_col + w_col;
        const float *im = data_im + ((long)c_im * height + h_offset) * width + w_offset;
        for (int ki = 0; ki < kernel_h; ki++) {
            for (int kj = 0; kj < kernel_w; kj++) {
                int h_im = h_offset + ki * dilation_h;
                int w_im = w_offset + kj * dilation_w;
                *col = (h_im >= 0 && w_im >= 0 && h_im < height && w_im < width)
                           ? im[ki * dilation_h * width + kj * dilation_w]
                           : 0.0f;
                col += (size_t)height_col * width_col;
            }
        }
    }
}

/* ------------------------------------------------------------------ sgemm
 * src/ori_kernel/sgemm_kernel.cu:9-44 (general_ptb_sgemm: src/gptb_kernel/sgemm_kernel.cu:3-77):
 * C[m + n ldc] = C[m + n ldc] * beta + alpha * sum_k A[m + k lda] * B[n + k ldb], lda = ldc = M,
 * ldb = N, alpha = beta = 2, k ascending, each step c = fma(a, b, c) -- what nvcc's default
 * -fmad=true makes of "c[kk] += a * b_s[j][kk]".  A block is 128 rows m by 16 columns n.
 *
 * Positions [start, end) of the (gdx, gdy, gdz) grid: position p adds, to block p % (gdx*gdy),
 * k part (p / (gdx*gdy)) % gdz, i.e. k in [part*chunk, min((part+1)*chunk, K)) (the last part
 * runs to K).  gdz = 1: a position is a block's whole k loop, the reference's kernel.  Part 0
 * starts from zero, other parts from what the block's previous part left in W (M x N floats,
 * laid out as C); the last part scales and updates C.  Positions of one block are applied in
 * ascending order. */
ORC_API void orc_sgemm_gptb(const float *A, const float *B, float *C, float *W, int M, int N, int K, int gdx,
                            int gdy, int gdz, int chunk, int start, int end)
{
    const int TILE_M = 128, TILE_N = 16;
    const float alpha = 2.0f, beta = 2.0f;
    const int blocks = gdx * gdy;
#pragma omp parallel for schedule(dynamic)
    for (int blk = 0; blk < blocks; blk++) {
        int first = start + ((blk - start % blocks) + blocks) % blocks;
        for (int pos = first; pos < end; pos += blocks) {
            const int bx = pos % gdx, by = (pos / gdx) % gdy, part = (pos / blocks) % gdz;
            const int k0 = gdz > 1 ? (part * chunk < K ? part * chunk : K) : 0;
            const int k1 = (gdz == 1 || part == gdz - 1) ? K : ((part + 1) * chunk < K ? (part + 1) * chunk : K);
            for (int mid = 0; mid < TILE_M; mid++) {
                const size_t m = (size_t)bx * TILE_M + mid;
                const size_t t = (size_t)M * by * TILE_N + m;
                float c[16];
                for (int i = 0; i < TILE_N; i++) c[i] = k0 == 0 ? 0.0f : W[t + (size_t)i * M];
                for (int k = k0; k < k1; k++) {
                    const float a = A[m + (size_t)k * M];
                    const float *b = B + (size_t)by * TILE_N + (size_t)k * N;
                    for (int i = 0; i < TILE_N; i++) c[i] = fmaf(a, b[i], c[i]);
                }
                for (int i = 0; i < TILE_N; i++) {
                    if (k1 == K) {
                        const float scaled_old = C[t + (size_t)i * M] * beta;
                        const float scaled_sum = alpha * c[i];
                        C[t + (size_t)i * M] = scaled_old + scaled_sum;
                    } else {
                        W[t + (size_t)i * M] = c[i];
                    }
                }
            }
        }
    }
}

/* ------------------------------------------------------------------ fft
 * src/ori_kernel/fft_kernel.cu:11-61, src/header/fft_header.h:13-67 (g_general_ptb_fft:
 * src/gptb_kernel/fft_kernel.cu:3-75): a block of FFT_T = 128 threads transforms 256 complex
 * points in place.  Thread j holds v[r] = data[j + r*128], r = 0, 1; for Ns = 1, 2, .., 128:
 * angle = -2 pi (j % Ns) / (Ns * 2) (evaluated in double, rounded to float), v[r] *= (cos(r*angle),
 * sin(r*angle)) with the float cos and sin, butterfly (v0 + v1, v0 - v1), then every thread writes
 * v[r] to work[expand(j, Ns, 2) + r*Ns] and reads v[r] = work[j + r*128] (expand(j, 128, 2) = j),
 * expand(i, N1, N2) = (i / N1) * N1 * N2 + i % N1.  Complex product: (a.x b.x - a.y b.y,
 * a.x b.y + a.y b.x).  The library's cosf/sinf stand for CUDA's: bits of the twiddles may differ
 * from either device's.
 *
 * Positions [start, end): position p transforms batch entry p % grid. */
ORC_API void orc_fft_gptb(float *data, int grid, int start, int end)
{
    enum { N = 256, T = 128 };
    const double pi = 3.14159265358979323846;   /* M_PI of math.h */
    for (int pos = start; pos < end; pos++) {
        float *d = data + (size_t)(pos % grid) * N * 2;
        float vx[T][2], vy[T][2];
        for (int j = 0; j < T; j++)
            for (int r = 0; r < 2; r++) {
                vx[j][r] = d[2 * (j + r * T)];
                vy[j][r] = d[2 * (j + r * T) + 1];
            }
        for (int Ns = 1; Ns < N; Ns *= 2) {
            float sr[N], si[N];
            for (int j = 0; j < T; j++) {
                const float angle = (float)(-2 * pi * (j % Ns) / (Ns * 2));
                for (int r = 0; r < 2; r++) {
                    const float bx = cosf(r * angle), by = sinf(r * angle);
                    const float ax = vx[j][r], ay = vy[j][r];
                    const float p0 = ax * bx, p1 = ay * by, p2 = ax * by, p3 = ay * bx;
                    vx[j][r] = p0 - p1;
                    vy[j][r] = p2 + p3;
                }
                const float tx = vx[j][0], ty = vy[j][0];
                vx[j][0] = tx + vx[j][1];
                vy[j][0] = ty + vy[j][1];
                vx[j][1] = tx - vx[j][1];
                vy[j][1] = ty - vy[j][1];
                const int idxD = (j / Ns) * Ns * 2 + (j % Ns);
                for (int r = 0; r < 2; r++) {
                    sr[idxD + r * Ns] = vx[j][r];
                    si[idxD + r * Ns] = vy[j][r];
                }
            }
            for (int j = 0; j < T; j++) {
                const int idxS = (j / T) * T * 2 + (j % T);
                for (int r = 0; r < 2; r++) {
                    vx[j][r] = sr[idxS + r * T];
                    vy[j][r] = si[idxS + r * T];
                }
            }
        }
        for (int j = 0; j < T; j++)
            for (int r = 0; r < 2; r++) {
                d[2 * (j + r * T)] = vx[j][r];
                d[2 * (j + r * T) + 1] = vy[j][r];
            }
    }
}

/* source[i] = rand() / (float)RAND_MAX * 2 - 1 after srand(54321), x then y of each point
 * (src/ori_kernel/fft_kernel.cu:93-103) */
ORC_API void orc_fft_source(float *data, int values)
{
    srand(54321);
    for (int i = 0; i < values; i++) data[i] = (rand() / (float)RAND_MAX) * 2 - 1;
}

/* ------------------------------------------------------------------ cutcp
 * src/ori_kernel/cutcp_kernel.cu:19-158 (general_ptb_cutcp: src/gptb_kernel/cutcp_kernel.cu:12-183):
 * thread (tx, ty, tz) of region (xr, yr, zr) owns the lattice points (8 xr + tx, 8 yr + ty + 2 e,
 * 8 zr + tz), e = 0..3.  It walks the bins centre + nbr[n], n ascending, and in a bin the atoms until
 * the first with charge 0:
 *   dx = ax - x; dz = az - z; dxdz2 = dx*dx + dz*dz; dy = ay - y; r2 = dy*dy + dxdz2;
 *   if (r2 < cutoff2) { s = 1 - r2 * inv_cutoff2; energy_e += aq * rsqrt(r2) * s * s; }  dy -= 2h; ...
 * centre = floor((8 r + 4) * h / 4) per dimension.  1.0f / sqrtf stands for CUDA's rsqrtf (an
 * approximation of about an ulp on either device).  Energies are stored, not accumulated.
 *
 * Positions [start, end) of a grid of regions (columns) by parts of the list (rows; parts = 1: a
 * position is a region's whole list in ascending order, the reference's kernel): position p adds part
 * (p / regions) % parts, the entries part, part + parts, part + 2 parts, ..., to region r = p % regions =
 * (r / (gdy gdz), (r / gdz) % gdy, r % gdz).  Part 0 starts from zero, other parts from the energies
 * the region holds.  Positions of one region are applied in ascending order. */
ORC_API void orc_cutcp_gptb(int binDim_x, int binDim_y, const float *binZero, float h, float cutoff2, float inv_cutoff2,
                            float *regionZero, const int *nbr, int nbr_len, int gdx, int gdy, int gdz, int parts,
                            int start, int end)
{
    const int regions = gdx * gdy * gdz;
#pragma omp parallel for schedule(dynamic)
    for (int r = 0; r < regions; r++) {
        const int xr = r / (gdy * gdz), yr = (r / gdz) % gdy, zr = r % gdz;
        float *region = regionZero + (size_t)((zr * gdy + yr) * gdx + xr) * 512;
        const int bx = (int)floorf((8 * xr + 4) * h * 0.25f);
        const int by = (int)floorf((8 * yr + 4) * h * 0.25f);
        const int bz = (int)floorf((8 * zr + 4) * h * 0.25f);
        int first = start + ((r - start % regions) + regions) % regions;
        for (int pos = first; pos < end; pos += regions) {
            const int part = (pos / regions) % parts;
            for (int tid = 0; tid < 128; tid++) {
                const int tx = tid & 7, ty = (tid >> 3) & 1, tz = tid >> 4;
                const float x = (8 * xr + tx) * h, y = (8 * yr + ty) * h, z = (8 * zr + tz) * h;
                float *mine = region + (tid >> 4) * 64 + (tid & 15);
                float energy[4] = {0.f, 0.f, 0.f, 0.f};
                if (part > 0)
                    for (int e = 0; e < 4; e++) energy[e] = mine[16 * e];
                for (int n = part; n < nbr_len; n += parts) {
                    const int i = bx + nbr[3 * n], j = by + nbr[3 * n + 1], k = bz + nbr[3 * n + 2];
                    const float *bin = binZero + ((long long)(k * binDim_y + j) * binDim_x + i) * 32;
                    for (int a = 0; a < 8; a++) {
                        const float aq = bin[4 * a + 3];
                        if (0.f == aq) break;
                        const float dx = bin[4 * a] - x;
                        const float dz = bin[4 * a + 2] - z;
                        const float dxdz2 = dx * dx + dz * dz;
                        float dy = bin[4 * a + 1] - y;
                        for (int e = 0; e < 4; e++) {
                            const float r2 = dy * dy + dxdz2;
                            if (r2 < cutoff2) {
                                const float s = (1.f - r2 * inv_cutoff2);
                                energy[e] += aq * (1.0f / sqrtf(r2)) * s * s;
                            }
                            dy -= 2.0f * h;
                        }
                    }
                }
                for (int e = 0; e < 4; e++) mine[16 * e] = energy[e];
            }
        }
    }
}

/* prepare_input (src/header/cutcp_header.h:111-300): bin dimensions, neighbour list and the atoms
 * hashed into bins of 4 Angstroms, 8 to a bin, in the order given.  bins: binDim x*y*z * 32 floats,
 * zeroed by the caller; nbr: room for 1331 triples.  Returns the neighbour count, -1 where the
 * reference gives up.  counts: atoms whose bin was full, atoms outside or without charge. */
ORC_API int orc_cutcp_prepare(const float *atoms, int natoms, const float *lo, int nx, int ny, int nz, float h,
                              float cutoff, int *binDim, int *padding, float *bins, int *nbr, int *counts)
{
    const int lnx = 8 * (int)ceilf(nx / 8.f), lny = 8 * (int)ceilf(ny / 8.f), lnz = 8 * (int)ceilf(nz / 8.f);
    const int c = (int)ceil(cutoff * 0.25f);
    *padding = c;
    binDim[0] = (int)ceil(lnx * h * 0.25f) + 2 * c;
    binDim[1] = (int)ceil(lny * h * 0.25f) + 2 * c;
    binDim[2] = (int)ceil(lnz * h * 0.25f) + 2 * c;
    float s;
    if (ceilf(4.f / (8 * h)) == floorf(4.f / (8 * h))) {
        s = sqrtf(3);
        if (2 * c + 1 > 11) return -1;
    } else if (8 * h <= 2 * 4.f) {
        s = 2.f * sqrtf(3);
        if (2 * c + 3 > 11) return -1;
    } else {
        return -1;
    }
    const float r2 = (cutoff + s * 4.f) * (cutoff + s * 4.f);
    int cnt = 0;
    for (int k = -c; k <= c; k++)
        for (int j = -c; j <= c; j++)
            for (int i = -c; i <= c; i++) {
                if ((i * i + j * j + k * k) * 4.f * 4.f >= r2) continue;
                if (nbr) nbr[3 * cnt] = i, nbr[3 * cnt + 1] = j, nbr[3 * cnt + 2] = k;
                cnt++;
            }
    if (!bins) return cnt;
    const long long nbins = (long long)binDim[0] * binDim[1] * binDim[2];
    int *fill = (int *)calloc((size_t)nbins, sizeof(int));
    counts[0] = counts[1] = 0;
    for (int n = 0; n < natoms; n++) {
        const float px = atoms[4 * n] - lo[0], py = atoms[4 * n + 1] - lo[1], pz = atoms[4 * n + 2] - lo[2];
        const float q = atoms[4 * n + 3];
        const int i = (int)floorf(px * 0.25f), j = (int)floorf(py * 0.25f), k = (int)floorf(pz * 0.25f);
        if (i >= -c && i < binDim[0] - c && j >= -c && j < binDim[1] - c && k >= -c && k < binDim[2] - c && q != 0) {
            const long long index = ((long long)(k + c) * binDim[1] + (j + c)) * binDim[0] + (i + c);
            if (fill[index] < 8) {
                float *slot = bins + index * 32 + 4 * fill[index];
                slot[0] = px, slot[1] = py, slot[2] = pz, slot[3] = q;
                fill[index]++;
            } else {
                counts[0]++;
            }
        } else {
            counts[1]++;
        }
    }
    free(fill);
    return cnt;
}


/* ------------------------------------------------------------------ nn
 * src/ori_kernel/nn_kernel.cu:9-17 (general_ptb_nn: src/gptb_kernel/nn_kernel.cu:3-23): thread t of
 * block (bx, by) owns record globalId = blockDim.x * (gridDim.x * by + bx) + t and writes
 * sqrt((lat - r.lat) * (lat - r.lat) + (lng - r.lng) * (lng - r.lng)) in float if globalId <
 * numRecords.  Positions [start, end): bx = p % gx, by = (p / gx) % gy. */
ORC_API void orc_nn_gptb(const float *locations, float *distances, int numRecords, float lat, float lng, int gx,
                         int gy, int bdx, int start, int end)
{
    for (int pos = start; pos < end; ++pos) {
        const int bx = (int)((unsigned)pos % (unsigned)gx);
        const int by = (int)(((unsigned)pos / (unsigned)gx) % (unsigned)gy);
        for (int t = 0; t < bdx; ++t) {
            const long long id = (long long)bdx * ((long long)gx * by + bx) + t;
            if (id >= numRecords) continue;
            const float dlat = lat - locations[2 * id];
            const float dlng = lng - locations[2 * id + 1];
            distances[id] = sqrtf(dlat * dlat + dlng * dlng);
        }
    }
}

/* ------------------------------------------------------------------ hot3d
 * src/ori_kernel/hot3d_kernel.cu:9-60 (general_ptb_hot3d: src/gptb_kernel/hot3d_kernel.cu:3-62):
 * thread (tx, ty) of block (bx, by) owns column i = bdx bx + tx, j = bdy by + ty and walks it from
 * layer 0 up; the neighbour of an edge cell is the cell itself, below the bottom layer and above
 * the top layer likewise.  Per cell, float, summed left to right:
 *   cc t + cw W + ce E + cs S + cn N + cb below + ct above + sdc p + ct 80. */
ORC_API void orc_hot3d_gptb(const float *p, const float *tIn, float *tOut, float sdc, int nx, int ny, int nz,
                            float ce, float cw, float cn, float cs, float ct, float cb, float cc, int gx, int gy,
                            int bdx, int bdy, int start, int end)
{
    const float amb_temp = 80.0f;
    const long long xy = (long long)nx * ny;
    for (int pos = start; pos < end; ++pos) {
        const int bx = (int)((unsigned)pos % (unsigned)gx);
        const int by = (int)(((unsigned)pos / (unsigned)gx) % (unsigned)gy);
        for (int ty = 0; ty < bdy; ++ty)
            for (int tx = 0; tx < bdx; ++tx) {
                const int i = bdx * bx + tx, j = bdy * by + ty;
                if (i >= nx || j >= ny) continue;
                for (int k = 0; k < nz; ++k) {
                    const long long c = i + (long long)j * nx + k * xy;
                    const long long W = i == 0 ? c : c - 1, E = i == nx - 1 ? c : c + 1;
                    const long long N = j == 0 ? c : c - nx, S = j == ny - 1 ? c : c + nx;
                    const float below = tIn[k == 0 ? c : c - xy], above = tIn[k == nz - 1 ? c : c + xy];
                    float v = cc * tIn[c];
                    v = v + cw * tIn[W];
                    v = v + ce * tIn[E];
                    v = v + cs * tIn[S];
                    v = v + cn * tIn[N];
                    v = v + cb * below;
                    v = v + ct * above;
                    v = v + sdc * p[c];
                    v = v + ct * amb_temp;
                    tOut[c] = v;
                }
            }
    }
}

/* the step's coefficients, src/ori_kernel/hot3d_kernel.cu:84-116 (float variables, double constants) */
ORC_API void orc_hot3d_coefficients(int numCols, int numRows, int layers, float out[8])
{
    const float t_chip = 0.0005f, chip_height = 0.016f, chip_width = 0.016f;
    float dx = chip_height / numRows, dy = chip_width / numCols, dz = t_chip / layers;
    float Cap = 0.5 * 1.75e6 * t_chip * dx * dy;
    float Rx = dy / (2.0 * 100 * t_chip * dx);
    float Ry = dx / (2.0 * 100 * t_chip * dy);
    float Rz = dz / (100 * dx * dy);
    float max_slope = 3.0e6 / (0.5 * t_chip * 1.75e6);
    float dt = 0.001 / max_slope;
    float stepDivCap = dt / Cap;
    float ce = stepDivCap / Rx, cn = stepDivCap / Ry, ct = stepDivCap / Rz;
    float cc = 1.0 - (2.0 * ce + 2.0 * cn + 3.0 * ct);
    out[0] = stepDivCap, out[1] = ce, out[2] = ce, out[3] = cn, out[4] = cn, out[5] = ct, out[6] = ct, out[7] = cc;
}

/* ------------------------------------------------------------------ path
 * src/ori_kernel/path_kernel.cu:9-86 (general_ptb_path: src/gptb_kernel/path_kernel.cu:3-93):
 * block bx works on the 256 columns from blkX = (256 - 2 iteration) bx - border; thread tx holds
 * column blkX + tx.  prev[] starts as the source row where the column is on the grid.  Row i
 * (0 <= i < iteration): threads with i + 1 <= tx <= 254 - i whose tx lies in [validXmin,
 * validXmax] set result[tx] = min(prev[W], prev[tx], prev[E]) + wall[cols (startStep + i) + xidx],
 * W = max(tx - 1, validXmin), E = min(tx + 1, validXmax); all but the last row then copy result to
 * prev.  The threads that computed in the last row write result to gpuResults.
 * Positions [start, end): bx = p (no wrap in the reference). */
ORC_API void orc_path_gptb(int iteration, const int *wall, const int *src, int *results, int cols, int startStep,
                           int border, int start, int end)
{
    enum { BS = 256 };
    for (int bx = start; bx < end; ++bx) {
        int prev[BS], result[BS], computed[BS];
        const int small_block_cols = BS - iteration * 2;
        const int blkX = small_block_cols * bx - border;
        const int blkXmax = blkX + BS - 1;
        const int validXmin = blkX < 0 ? -blkX : 0;
        const int validXmax = blkXmax > cols - 1 ? BS - 1 - (blkXmax - cols + 1) : BS - 1;
        for (int tx = 0; tx < BS; ++tx) {
            const int xidx = blkX + tx;
            prev[tx] = (xidx >= 0 && xidx <= cols - 1) ? src[xidx] : 0;
            result[tx] = 0;
            computed[tx] = 0;
        }
        for (int i = 0; i < iteration; ++i) {
            for (int tx = 0; tx < BS; ++tx) {
                computed[tx] = 0;
                if (tx >= i + 1 && tx <= BS - i - 2 && tx >= validXmin && tx <= validXmax) {
                    int W = tx - 1, E = tx + 1;
                    if (W < validXmin) W = validXmin;
                    if (E > validXmax) E = validXmax;
                    int shortest = prev[W] <= prev[tx] ? prev[W] : prev[tx];
                    shortest = shortest <= prev[E] ? shortest : prev[E];
                    computed[tx] = 1;
                    result[tx] = shortest + wall[(long long)cols * (startStep + i) + blkX + tx];
                }
            }
            if (i == iteration - 1) break;
            for (int tx = 0; tx < BS; ++tx)
                if (computed[tx]) prev[tx] = result[tx];
        }
        for (int tx = 0; tx < BS; ++tx)
            if (computed[tx]) results[blkX + tx] = result[tx];
    }
}

/* the reference's grid: rand() % 10 after srand(9), row by row (src/ori_kernel/path_kernel.cu:113-119) */
ORC_API void orc_path_source(int *cells, long long n)
{
    srand(9);
    for (long long i = 0; i < n; ++i) cells[i] = rand() % 10;
}


/* ------------------------------------------------------------------ lava
 * src/ori_kernel/lava_kernel.cu:9-141 (general_ptb_lava: src/gptb_kernel/lava_kernel.cu:3-140);
 * the box list as src/ori_kernel/lava_kernel.cu:176-224 builds it.  Layouts of
 * src/header/lava_header.h:16-45. */
typedef struct { float v, x, y, z; } orc_four_vector;
typedef struct { int x, y, z; int number; long offset; } orc_nei_str;
typedef struct { int x, y, z; int number; long offset; int nn; orc_nei_str nei[26]; } orc_box_str;

ORC_API int orc_lava_box_bytes(void) { return (int)sizeof(orc_box_str); }

/* boxes1d^3 boxes, x fastest; the neighbours of a box in the order l (z), m (y), n (x) = -1, 0, 1 */
ORC_API void orc_lava_boxes(int boxes1d, void *out)
{
    orc_box_str *box = (orc_box_str *)out;
    int nh = 0;
    for (int i = 0; i < boxes1d; i++)
        for (int j = 0; j < boxes1d; j++)
            for (int k = 0; k < boxes1d; k++) {
                memset(&box[nh], 0, sizeof(orc_box_str));
                box[nh].x = k, box[nh].y = j, box[nh].z = i;
                box[nh].number = nh;
                box[nh].offset = (long)nh * 100;
                box[nh].nn = 0;
                for (int l = -1; l < 2; l++)
                    for (int m = -1; m < 2; m++)
                        for (int n = -1; n < 2; n++) {
                            const int inside = i + l >= 0 && j + m >= 0 && k + n >= 0 && i + l < boxes1d &&
                                               j + m < boxes1d && k + n < boxes1d;
                            if (!inside || (l == 0 && m == 0 && n == 0)) continue;
                            orc_nei_str *ne = &box[nh].nei[box[nh].nn];
                            ne->x = k + n, ne->y = j + m, ne->z = i + l;
                            ne->number = ne->z * boxes1d * boxes1d + ne->y * boxes1d + ne->x;
                            ne->offset = (long)ne->number * 100;
                            box[nh].nn++;
                        }
                nh++;
            }
}

/* Positions [start, end) of the grid boxes x 27: position p adds part (p / boxes) % 27 of box
 * p % boxes (part 0 = the home box, part k = neighbour k - 1 of the list) onto fv, every home
 * particle walking the part's 100 particles in order, all in float with expf. */
ORC_API void orc_lava_gptb(float alpha, const void *boxes_, const float *rv_, const float *qv, float *fv_,
                           int number_boxes, int start, int end)
{
    const orc_box_str *box = (const orc_box_str *)boxes_;
    const orc_four_vector *rv = (const orc_four_vector *)rv_;
    orc_four_vector *fv = (orc_four_vector *)fv_;
    const float a2 = 2.0 * alpha * alpha;
    for (int pos = start; pos < end; ++pos) {
        const int bx = pos % number_boxes, k = (pos / number_boxes) % 27;
        if (k >= 1 + box[bx].nn) continue;
        const int pointer = k == 0 ? bx : box[bx].nei[k - 1].number;
        const orc_four_vector *rA = rv + box[bx].offset, *rB = rv + box[pointer].offset;
        const float *qB = qv + box[pointer].offset;
        orc_four_vector *fA = fv + box[bx].offset;
        for (int w = 0; w < 100; ++w)
            for (int j = 0; j < 100; ++j) {
                const float dot = rA[w].x * rB[j].x + rA[w].y * rB[j].y + rA[w].z * rB[j].z;
                const float r2 = rA[w].v + rB[j].v - dot;
                const float u2 = a2 * r2;
                const float vij = expf(-u2);
                const float fs = 2 * vij;
                const float dx = rA[w].x - rB[j].x, dy = rA[w].y - rB[j].y, dz = rA[w].z - rB[j].z;
                const float fxij = fs * dx, fyij = fs * dy, fzij = fs * dz;
                fA[w].v += qB[j] * vij;
                fA[w].x += qB[j] * fxij;
                fA[w].y += qB[j] * fyij;
                fA[w].z += qB[j] * fzij;
            }
    }
}
