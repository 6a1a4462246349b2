/*
 * tacker_amd.h -- C-ABI of libtacker_amd.so (MI355X / gfx950).
 *
 * Two layers, both plain C (pointers, sizes, ints; no C++ or torch types):
 *
 *  1. tk*        : the thin device layer the host runtime (Kernel / GPTBKernel /
 *                  MixKernel / Creator / TaskManager) is written against.  It
 *                  replaces the CUDA runtime + driver calls the reference makes
 *                  directly (cudaMalloc, cudaLaunchKernel, cuModuleLoad, ...).
 *                  Two implementations exist: the HIP one (tk_hip.cpp, in
 *                  libtacker_amd.so) and a recording fake (tk_fake.cpp, in
 *                  libtacker_host_fake.so) used by CPU-only tests.
 *  2. tacker_*   : the entry points of the hot path.  Each one drives the same
 *                  C++ objects a reference caller would build by hand and
 *                  launches the same device function; the comment on each names
 *                  the reference interface it stands in for.
 *
 * Every function returns 0 on success and a non-zero code on failure unless
 * stated otherwise; tkGetErrorString / tacker_last_error give the text.
 * All device pointers are ordinary HIP device pointers (hipMalloc, torch, ...).
 * Streams are hipStream_t passed as void* (NULL = the default stream).
 * The library is single-host-thread like the reference (GPTBKernel::executeImpl
 * pushes/pops its own parameter vector, src/GPTBKernel.h:99-119).
 */
#ifndef TACKER_AMD_H
#define TACKER_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TK_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------- */
/* 1. thin device layer                                                       */
/* ------------------------------------------------------------------------- */

typedef void *tkStream_t;
typedef void *tkEvent_t;
typedef void *tkModule_t;
typedef void *tkFunction_t;
typedef struct tkDim3 {
    unsigned x, y, z;
} tkDim3;

enum { TK_MEMCPY_H2D = 1, TK_MEMCPY_D2H = 2, TK_MEMCPY_D2D = 3 };
enum {
    TK_SUCCESS = 0,
    TK_ERROR_INVALID_VALUE = 1,
    TK_ERROR_NOT_FOUND = 2,      /* unknown kernel / symbol / function key */
    TK_ERROR_UNSUPPORTED = 3,    /* shape the gfx950 kernels do not cover */
    TK_ERROR_DEVICE = 4          /* a HIP call failed; see tkGetErrorString */
};

/* replaces initCUDA (src/main.cu:166-184): select the device, create a context */
TK_API int tkInit(int device);
TK_API const char *tkGetErrorString(int code);
/* number of compute units (replaces the SM_NUM macro, src/header/pets_common.h:4-6) */
TK_API int tkGetCuCount(int *cu_count);
TK_API int tkGetDeviceName(char *buf, size_t len);

TK_API int tkMalloc(void **ptr, size_t bytes);                           /* cudaMalloc */
TK_API int tkFree(void *ptr);                                            /* cudaFree */
/* How often tkMalloc and tkFree have been called in this process (either pointer may be null).
 * No counterpart in the reference: a caller that must not allocate (stream capture, a serving
 * loop) reads it before and after a call to see that the library kept to that. */
TK_API int tkAllocationCalls(long long *mallocs, long long *frees);
TK_API int tkMemcpy(void *dst, const void *src, size_t bytes, int kind); /* cudaMemcpy */
TK_API int tkMemcpyAsync(void *dst, const void *src, size_t bytes, int kind, tkStream_t s);
TK_API int tkMemset(void *ptr, int value, size_t bytes);                 /* cudaMemset */
/* cudaMemcpyToSymbol for the two constant tables of the path: "ck" (mri-q k
 * table, src/ori_kernel/mriq_kernel.cu:9) and "atominfo" (cp atoms,
 * src/ori_kernel/cp_kernel.cu:23). */
TK_API int tkMemcpyToSymbol(const char *symbol, const void *src, size_t bytes, size_t offset);
/* cudaMemcpyFromSymbol; also serves "tk_spin_fail", the word a role-local
 * barrier raises when it gives up waiting. */
TK_API int tkMemcpyFromSymbol(void *dst, const char *symbol, size_t bytes, size_t offset);

TK_API int tkStreamCreate(tkStream_t *s);
TK_API int tkStreamDestroy(tkStream_t s);
TK_API int tkStreamSynchronize(tkStream_t s);
TK_API int tkDeviceSynchronize(void);
TK_API int tkEventCreate(tkEvent_t *e);
TK_API int tkEventDestroy(tkEvent_t e);
TK_API int tkEventRecord(tkEvent_t e, tkStream_t s);
TK_API int tkEventSynchronize(tkEvent_t e);
TK_API int tkEventElapsedTime(float *ms, tkEvent_t start, tkEvent_t stop);

/* A stream's work recorded once and launched as one graph afterwards (no counterpart in the
 * reference, whose query loop issues its launches one by one): everything enqueued on s between
 * tkStreamBeginCapture and tkStreamEndCapture -- kernel launches of either kind; no synchronisation
 * and no memory-set calls may fall in between, and s must not be the null stream -- becomes an
 * executable graph that tkGraphLaunch enqueues as a whole. */
typedef void *tkGraphExec_t;
TK_API int tkStreamBeginCapture(tkStream_t s);
TK_API int tkStreamEndCapture(tkStream_t s, tkGraphExec_t *exec);
TK_API int tkGraphLaunch(tkGraphExec_t exec, tkStream_t s);
TK_API int tkGraphExecDestroy(tkGraphExec_t exec);

/* cudaLaunchKernel (src/GPTBKernel.h:109, src/MixKernel.h:100): func is a value
 * of the function registry, args is an array of pointers to each argument. */
TK_API int tkLaunchKernel(const void *func, tkDim3 grid, tkDim3 block, void **args, size_t shmem,
                          tkStream_t stream);

/* cuModuleLoad / cuModuleGetFunction / cuLaunchKernel (src/ModuleCenter.cu): code
 * objects (.hsaco / .co) instead of cubins. */
TK_API int tkModuleLoad(tkModule_t *m, const char *path);
TK_API int tkModuleUnload(tkModule_t m);
TK_API int tkModuleGetFunction(tkFunction_t *f, tkModule_t m, const char *name);
TK_API int tkModuleLaunchKernel(tkFunction_t f, tkDim3 grid, tkDim3 block, void **args,
                                size_t shmem, tkStream_t stream);

/* Fills the string-keyed device-function registry (the global `fmap` of
 * src/main.cu:108-159) without the host translation unit including device
 * sources: insert(key, function, ctx) is called once per kernel. Keys on the
 * hot path: ori_{stencil,lbm,mriq,mrif,cp,sgemm,fft,cutcp}, gptb_{tzgemm,stencil,lbm,mriq,mrif,cp,sgemm,fft,cutcp},
 * tzgemm_{stencil,lbm,mriq,mrif,cp,sgemm,fft,cutcp}, plus variant keys "<key>@<variant>". */
typedef void (*tk_kernel_insert_fn)(const char *key, const void *func, void *ctx);
TK_API int tk_register_kernels(tk_kernel_insert_fn insert, void *ctx);

/* ------------------------------------------------------------------------- */
/* 2. hot-path entry points                                                   */
/* ------------------------------------------------------------------------- */

/* One-time set-up: tkInit(device), registry, kinfo JSON ("" or NULL = the
 * built-in gfx950 table). Replaces main()'s read_json + initCUDA + fmap
 * initialiser (src/main.cu:108-159,266-281). Idempotent. */
TK_API int tacker_init(int device, const char *kinfo_json_path);
TK_API const char *tacker_last_error(void);

/* getTZGEMMGridDim (src/tzgemm_kernel.h:30-48): out = {M_GLOBAL, N_GLOBAL,
 * K_GLOBAL, tiles}, dimensions floored to multiples of 128 (min 128), tiles in
 * units of the reference's 64x64 CTA tile. */
TK_API int tacker_tzgemm_grid_dim(int m, int n, int k, int out[4]);

/* No counterpart in the reference (its tzgemm is one CTA per tile whatever the shape). Shapes
 * with few tiles and a long reduction (the batch-1 layers of src/dnn/: 32-128 tiles, K up to
 * 25088) cut the reduction of a tile over `parts` workgroups; the partial tiles and one arrival
 * counter per tile live in a workspace the library binds to the output buffer C on the first
 * GEMM that writes it; the kernels, whose parameter lists are the reference's, find it by looking
 * C up in a device-resident table the binding fills (nothing is bound when parts == 1).
 * tacker_tzgemm_parts: the number of parts for (m, n, k) rounded as tacker_tzgemm_grid_dim
 * rounds them -- a function of the shape only, so fused and unfused launches add in the same
 * order. tacker_tzgemm_workspace_bytes: size of that workspace, 0 when parts == 1.
 * A kernel object built on C is a user of C's binding until it is destroyed; a binding without
 * users stays for the next object on the same C and is taken out (after a device synchronisation,
 * least recently used first) when a new binding needs its place: at most 512 bindings, at most
 * 1 GiB held by bindings without users.
 * tacker_tzgemm_workspace_stats: bindings in the table, those with a user, bytes they hold.
 * tacker_tzgemm_release_workspaces: synchronises the device and frees them all; only when no
 * kernel object that uses one is left. */
TK_API int tacker_tzgemm_parts(int m, int n, int k);
TK_API long long tacker_tzgemm_workspace_bytes(int m, int n, int k);
TK_API int tacker_tzgemm_workspace_stats(int *bindings, int *in_use, long long *bytes);
TK_API int tacker_tzgemm_release_workspaces(void);

/* general_ptb_tzgemm through GPTBKernel (src/gptb_kernel/tzgemm_kernel.cu:430-449,
 * src/GPTBKernel.h:99-119, src/TaskManager.cu:238-248): C[M][N] f32 =
 * 1.1 * A[M][K] f16 * (B[N][K] f16)^T for the 64x64 tiles [tile_start, tile_end).
 * M, N, K must already be multiples of 128. launch_grid = number of persistent
 * workgroups (0 = one per tile group, capped at 2 per CU). */
TK_API int tacker_gptb_tzgemm(const void *A, const void *B, float *C, int M, int N, int K,
                              int tile_start, int tile_end, int launch_grid, tkStream_t stream);

/* No counterpart in the reference. tacker_gptb_tzgemm for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc):
 * same arguments, same kernel code, same bits in C, but the workspace of the shapes whose
 * reduction is shared by workgroups is a static device array of the library
 * (TACKER_TZGEMM_STATIC_SCRATCH_BYTES, held by each GPU the library runs on until the process
 * ends) instead of a buffer bound to C, and the call itself allocates nothing (no hipMalloc /
 * hipFree, no kernel objects with device state; the counters are cleared by a small kernel, not a
 * memset, so the call can be captured). A shape whose workspace
 * (tacker_tzgemm_workspace_bytes) exceeds the array is refused with TK_ERROR_UNSUPPORTED.
 * Every call on a GPU shares that GPU's array: calls that overlap in time on one GPU (two
 * streams, two threads) race on it -- serialise them. */
#define TACKER_TZGEMM_STATIC_SCRATCH_BYTES ((8u << 20) + (64u << 10))
TK_API int tacker_gptb_tzgemm_static_scratch(const void *A, const void *B, float *C, int M, int N,
                                             int K, int tile_start, int tile_end, int launch_grid,
                                             tkStream_t stream);

/* ori_stencil through OriSTENCILKernel::executeImpl
 * (src/ori_kernel/stencil_kernel.cu:9-94,189-201): one Jacobi sweep A0 -> Anext. */
TK_API int tacker_ori_stencil(float c0, float c1, const float *A0, float *Anext, int nx, int ny,
                              int nz, tkStream_t stream);
/* general_ptb_stencil through GPTBKernel (src/gptb_kernel/stencil_kernel.cu:3-104,
 * src/Creator.cu:179-192): block positions [block_start, block_end) of a grid of
 * (ceil(nx/64), ceil(ny/4), runs) positions, runs = ceil((nz-2) / TACKER_STENCIL_Z_RUN): position
 * p computes run p / blocks of block p % blocks (blocks = the ori grid's ceil(nx/64) *
 * ceil(ny/4)), a run being TACKER_STENCIL_Z_RUN centre planes of the block's march along z --
 * the reference's 3-D index reconstruction over a grid whose z cuts that march, so that a
 * range can be as short as the GEMM it rides with.  [0, tacker_stencil_blocks(nx, ny, nz)) is
 * one sweep (ori_stencil bit for bit), and so is any set of ranges that tiles it. launch_grid
 * workgroups of launch_block threads (0 = the Creator default for this GPU). */
#define TACKER_STENCIL_Z_RUN 8
TK_API int tacker_stencil_blocks(int nx, int ny, int nz);
TK_API int tacker_gptb_stencil(float c0, float c1, const float *A0, float *Anext, int nx, int ny,
                               int nz, int block_start, int block_end, int launch_grid,
                               int launch_block, tkStream_t stream);

/* ori_lbm / general_ptb_lbm (src/ori_kernel/lbm_kernel.cu:9-154,
 * src/gptb_kernel/lbm_kernel.cu:3-178): one D3Q19 collide+scatter step. src and
 * dst point at entry plane 0 of cell (0,0,0) of a 20*sx*sy*sz float SoA grid.
 * Blocks are rows (y,z): block = y + sy*z. */
TK_API int tacker_ori_lbm(const float *src, float *dst, int sx, int sy, int sz, tkStream_t stream);
TK_API int tacker_gptb_lbm(const float *src, float *dst, int sx, int sy, int sz, int block_start,
                           int block_end, int launch_grid, int launch_block, tkStream_t stream);

/* ori_ComputePhiMag (src/ori_kernel/mriq_kernel.cu:47-54) */
TK_API int tacker_mriq_phimag(const float *phiR, const float *phiI, float *phiMag, int numK,
                              tkStream_t stream);
/* cudaMemcpyToSymbol(ck, ...) (src/ori_kernel/mriq_kernel.cu:254-256): host table
 * of numK {Kx,Ky,Kz,PhiMag} records, numK <= TACKER_MRIQ_MAX_K. */
#define TACKER_MRIQ_MAX_K 4096
TK_API int tacker_mriq_set_kvalues(const float *kvals_host, int numK);
/* ori_mriq / g_general_ptb_mriq (src/ori_kernel/mriq_kernel.cu:56-105,
 * src/gptb_kernel/mriq_kernel.cu:3-70). numX multiple of 256. ori_mriq adds all numK
 * samples to every voxel. The GPTB form works on block positions [block_start, block_end)
 * of a grid of (numX / 256) voxel blocks by ceil(numK / TACKER_MRIQ_K_CHUNK) chunks of the
 * k table: position p adds chunk p / (numX / 256) to voxel block p % (numX / 256) -- the
 * reference's host loop over k chunks (mriq_kernel.cu:258-283) as the y index of the GPTB
 * grid. [0, tacker_mriq_blocks(numK, numX)) equals ori_mriq bit for bit, and so does any
 * sequence of launches whose ranges tile it in ascending order. */
#define TACKER_MRIQ_K_CHUNK 128
TK_API int tacker_mriq_blocks(int numK, int numX);
TK_API int tacker_ori_mriq(int numK, const float *x, const float *y, const float *z, float *Qr,
                           float *Qi, int numX, tkStream_t stream);
TK_API int tacker_gptb_mriq(int numK, const float *x, const float *y, const float *z, float *Qr,
                            float *Qi, int numX, int block_start, int block_end, int launch_grid,
                            int launch_block, tkStream_t stream);

/* ComputeRhoPhiGPU (src/ori_kernel/mrif_kernel.cu:62-75): RhoPhi = conj(phi) * d per k sample. */
TK_API int tacker_mrif_rhophi(int numK, const float *phiR, const float *phiI, const float *dR,
                              const float *dI, float *realRhoPhi, float *imagRhoPhi,
                              tkStream_t stream);
/* cudaMemcpyToSymbol(c, ...) (src/ori_kernel/mrif_kernel.cu:304): host table of numK
 * {Kx,Ky,Kz,RhoPhiR,RhoPhiI} records, numK <= TACKER_MRIF_MAX_K. */
#define TACKER_MRIF_MAX_K 4096
TK_API int tacker_mrif_set_kvalues(const float *kvals_host, int numK);
/* ori_mrif / general_ptb_mrif (src/ori_kernel/mrif_kernel.cu:77-152,
 * src/gptb_kernel/mrif_kernel.cu:96-170). numX multiple of 256. ori_mrif adds all numK
 * samples to every voxel (the reference stops after the first grid of 256). Block positions
 * of the GPTB form are laid out as MRI-Q's: (numX / 256) voxel blocks by
 * ceil(numK / TACKER_MRIF_K_CHUNK) chunks of the k table, the reference's loop over grids of
 * the table (mrif_kernel.cu:84-85) as the y index. [0, tacker_mrif_blocks(numK, numX))
 * equals ori_mrif bit for bit, and so does any sequence of launches whose ranges tile it in
 * ascending order. */
#define TACKER_MRIF_K_CHUNK 128
TK_API int tacker_mrif_blocks(int numK, int numX);
TK_API int tacker_ori_mrif(int numK, const float *x, const float *y, const float *z, float *outR,
                           float *outI, int numX, tkStream_t stream);
TK_API int tacker_gptb_mrif(int numK, const float *x, const float *y, const float *z, float *outR,
                            float *outI, int numX, int block_start, int block_end, int launch_grid,
                            int launch_block, tkStream_t stream);

/* ori_sgemm / general_ptb_sgemm (src/ori_kernel/sgemm_kernel.cu:9-44,
 * src/gptb_kernel/sgemm_kernel.cu:3-77): C = 2 C + 2 A B in fp32; A is K rows of M floats (lda = M),
 * B K rows of N floats (ldb = N), C N columns of M floats (ldc = M); M a multiple of 128, N of 16.
 * k ascends per element of C, every step one fused multiply-add.  Block positions of the GPTB form:
 * the reference's (M / 128) x (N / 16) blocks by ceil(K / TACKER_SGEMM_K_CHUNK) parts of the k loop as
 * the z index; between parts a block's partial results rest in a workspace of M x N floats that the
 * library binds to C when a kernel object is built on it (tacker_tzgemm_release_workspaces frees
 * it).  [0, tacker_sgemm_blocks(M, N, K)) equals ori_sgemm bit for bit, and so does any sequence
 * of launches whose ranges tile it in ascending order. */
#define TACKER_SGEMM_K_CHUNK 64
TK_API int tacker_sgemm_blocks(int M, int N, int K);
TK_API int tacker_ori_sgemm(const float *A, const float *B, float *C, int M, int N, int K,
                            tkStream_t stream);
TK_API int tacker_gptb_sgemm(const float *A, const float *B, float *C, int M, int N, int K,
                             int block_start, int block_end, int launch_grid, int launch_block,
                             tkStream_t stream);

/* ori_fft / g_general_ptb_fft (src/ori_kernel/fft_kernel.cu:11-61, src/gptb_kernel/fft_kernel.cu:3-75):
 * `batches` forward transforms of 256 complex points each, radix 2, in place; data holds
 * batches x 256 (re, im) pairs of floats.  One block position per transform; a position past the
 * batch wraps (position % batches).  A transform is served by one wavefront (launch_block a
 * multiple of 64) where the reference launches 128 threads.  Twiddles are correctly rounded table
 * values: results agree with the reference's within rounding (about 1e-5 absolute for inputs in
 * [-1, 1]), not bit for bit. */
#define TACKER_FFT_POINTS 256
TK_API int tacker_ori_fft(float *data, int batches, tkStream_t stream);
TK_API int tacker_gptb_fft(float *data, int batches, int block_start, int block_end, int launch_grid,
                           int launch_block, tkStream_t stream);

/* ori_nn / general_ptb_nn (src/ori_kernel/nn_kernel.cu:9-17, src/gptb_kernel/nn_kernel.cu:3-23;
 * Rodinia nn): distances[i] = sqrtf((lat - lat_i)^2 + (lng - lng_i)^2) for numRecords records,
 * locations = numRecords {lat, lng} pairs of floats (the reference's LatLong).  One block position
 * per 256 records, tacker_nn_blocks(numRecords) of them.  fp32 in the order of the reference's
 * source with an IEEE square root: bit-identical to a CPU evaluation. */
TK_API int tacker_nn_blocks(int numRecords);
TK_API int tacker_ori_nn(const float *locations, float *distances, int numRecords, float lat, float lng,
                         tkStream_t stream);
TK_API int tacker_gptb_nn(const float *locations, float *distances, int numRecords, float lat, float lng,
                          int block_start, int block_end, int launch_grid, int launch_block,
                          tkStream_t stream);

/* ori_hot3d / general_ptb_hot3d (src/ori_kernel/hot3d_kernel.cu:9-60,
 * src/gptb_kernel/hot3d_kernel.cu:3-62; Rodinia hotspot3D): one time step of nx x ny x nz cells,
 * p = dissipated power, tIn / tOut = temperature before / after (distinct arrays), x fastest.  nx a
 * multiple of 64, ny of 4, nz >= 2; (nx / 64) * (ny / 4) block positions of 64 x 4 columns.  The
 * step's coefficients follow from the cell counts (src/ori_kernel/hot3d_kernel.cu:84-116);
 * tacker_hot3d_coefficients writes {sdc, ce, cw, cn, cs, ct, cb, cc}.  fp32 in the order of the
 * reference's source: bit-identical to a CPU evaluation. */
TK_API int tacker_hot3d_coefficients(int nx, int ny, int nz, float out[8]);
TK_API int tacker_ori_hot3d(const float *p, const float *tIn, float *tOut, int nx, int ny, int nz,
                            tkStream_t stream);
TK_API int tacker_gptb_hot3d(const float *p, const float *tIn, float *tOut, int nx, int ny, int nz,
                             int block_start, int block_end, int launch_grid, int launch_block,
                             tkStream_t stream);

/* ori_path / general_ptb_path (src/ori_kernel/path_kernel.cu:9-86,
 * src/gptb_kernel/path_kernel.cu:3-93; Rodinia pathfinder): `iteration` rows (1 .. 127) of
 * results[x] = wall[row][x] + min(src[x-1], src[x], src[x+1]) starting at row startStep of the
 * wall (the grid without its first row: (rows - 1) x cols ints), src and results rows of cols ints.
 * tacker_path_blocks(cols, iteration) block positions of 256 - 2 * iteration result columns each,
 * served by one wavefront each (launch_block a multiple of 64).  Integer work: the reference's
 * bits. */
TK_API int tacker_path_blocks(int cols, int iteration);
TK_API int tacker_ori_path(int iteration, const int *wall, const int *src, int *results, int cols, int rows,
                           int startStep, tkStream_t stream);
TK_API int tacker_gptb_path(int iteration, const int *wall, const int *src, int *results, int cols, int rows,
                            int startStep, int block_start, int block_end, int launch_grid,
                            int launch_block, tkStream_t stream);

/* ori_lava / general_ptb_lava (src/ori_kernel/lava_kernel.cu:9-141,
 * src/gptb_kernel/lava_kernel.cu:3-140; Rodinia lavaMD): boxes1d^3 boxes of 100 particles; rv = per
 * particle {v, x, y, z}, qv = its charge, fv = {potential, force x, y, z}, onto which every particle's
 * sums over the particles of its own box and of the up to 26 boxes around it are added (rv and fv
 * 16-byte aligned, distinct).  The box list (the reference's box_str array,
 * src/ori_kernel/lava_kernel.cu:176-224) is built inside; tacker_lava_boxes writes it to a host
 * buffer of boxes1d^3 * 656 bytes.  Block positions: boxes x 27 -- position p adds part
 * (p / boxes) % 27 of box p % boxes (part 0 = the box itself, part k = its k-th neighbour), so
 * ranges must be applied in ascending order to add a box's parts in the reference's order;
 * tacker_lava_blocks = boxes1d^3 * 27.  A box is served by one wavefront (launch_block a multiple of
 * 64) where the reference launches 128 threads.  fp32 in the order of the reference's source with
 * the hardware's exponential: results agree with a CPU evaluation within rounding
 * (|d| <= 2e-3 + 2e-5 |ref| for charges and coordinates in [0.1, 1]), not bit for bit. */
TK_API int tacker_lava_blocks(int boxes1d);
TK_API int tacker_lava_boxes(int boxes1d, void *out, size_t out_bytes);
TK_API int tacker_ori_lava(float alpha, int boxes1d, const float *rv, const float *qv, float *fv,
                           tkStream_t stream);
TK_API int tacker_gptb_lava(float alpha, int boxes1d, const float *rv, const float *qv, float *fv,
                            int block_start, int block_end, int launch_grid, int launch_block,
                            tkStream_t stream);

/* prepare_input (src/header/cutcp_header.h:111-300): hashes natoms atoms {x, y, z, q} into bins of
 * 4 x 4 x 4 Angstroms, 8 atoms to a bin, around a lattice of nx x ny x nz points of spacing h whose
 * lowest corner is lo, and lists the bin offsets a region of 8 x 8 x 8 points has to visit for the
 * given cutoff.  binDim[3], *padding (bins added on every side) and *nbr_len are always written;
 * bins (binDim[0] * binDim[1] * binDim[2] * 32 floats, x fastest) and nbr (*nbr_len triples, at most
 * 1331) when not NULL; counts[0] = atoms left out because their bin was full (the reference leaves
 * those to the CPU), counts[1] = atoms outside the bins or without charge.  Host memory only. */
TK_API int tacker_cutcp_prepare_input(const float *atoms, int natoms, const float lo[3], int nx, int ny,
                                      int nz, float h, float cutoff, int binDim[3], int *padding,
                                      float *bins, int *nbr, int *nbr_len, int counts[2]);
/* cudaMemcpyToSymbol(NbrListLen / NbrList) (src/ori_kernel/cutcp_kernel.cu:241-242) */
TK_API int tacker_cutcp_set_neighbours(const int *ijk, int len);
/* ori_cutcp / general_ptb_cutcp (src/ori_kernel/cutcp_kernel.cu:19-158,
 * src/gptb_kernel/cutcp_kernel.cu:12-183): the cutoff potential of the binned atoms on regions_x x
 * regions_y x regions_z regions of 8 x 8 x 8 lattice points, 512 floats per region, region (x, y, z)
 * at ((z regions_y + y) regions_x + x) * 512.  binZeroAddr points at bin (0, 0, 0) of the lattice,
 * behind the padding bins (device memory, read only).  Block positions of the GPTB form: the regions
 * in the order of the reference's GPTB kernel (x slowest) by the parts of TACKER_CUTCP_NBR_CHUNK
 * entries of the neighbour list loaded last, position p adding part p / regions to region
 * p % regions; a part other than the first goes on from the energies in memory.
 * [0, tacker_cutcp_blocks(...)) equals ori_cutcp bit for bit, and so does any sequence of launches
 * whose ranges tile it in ascending order.  A wavefront serves half a region (launch_block a
 * multiple of 64).  The hardware's reciprocal square root stands for CUDA's rsqrtf: results agree
 * with the reference's within rounding, not bit for bit. */
#define TACKER_CUTCP_NBR_CHUNK 32
TK_API int tacker_cutcp_blocks(int regions_x, int regions_y, int regions_z);
TK_API int tacker_ori_cutcp(int binDim_x, int binDim_y, const float *binZeroAddr, float h, float cutoff2,
                            float inv_cutoff2, float *regionZeroAddr, int regions_x, int regions_y,
                            int regions_z, tkStream_t stream);
TK_API int tacker_gptb_cutcp(int binDim_x, int binDim_y, const float *binZeroAddr, float h, float cutoff2,
                             float inv_cutoff2, float *regionZeroAddr, int regions_x, int regions_y,
                             int regions_z, int block_start, int block_end, int launch_grid,
                             int launch_block, tkStream_t stream);

/* copyatomstoconstbuf (src/ori_kernel/cp_kernel.cu:159-179): host array of
 * count (<= 64) {x,y,z,q}; z is replaced by (zplane - z)^2 on the way. */
TK_API int tacker_cp_set_atoms(const float *atoms_host, int count, float zplane);
/* initatoms (src/ori_kernel/cp_kernel.cu:185-209): glibc srand(54321) stream. */
TK_API int tacker_cp_initatoms(float *atoms_host, int count, unsigned volx, unsigned voly,
                               unsigned volz, float gridspacing);
/* ori_cp / g_general_ptb_cp (src/ori_kernel/cp_kernel.cu:26-79,
 * src/gptb_kernel/cp_kernel.cu:8-96): energygrid[voly][volx] += potential of the
 * atoms set by tacker_cp_set_atoms; volx multiple of 128, voly multiple of 8.
 * ori_cp runs the (volx/128, voly/8) blocks of 128 x 8 points. The GPTB form works on
 * block positions [block_start, block_end) of a (volx/128, voly/8, TACKER_CP_X_PARTS)
 * grid: position p computes part p / blocks of block p % blocks, a part being 2 of the 8
 * x points each thread of the block owns (the reference's 3-D index reconstruction over a
 * grid whose z splits the unrolled points). [0, tacker_cp_blocks(volx, voly)) equals
 * ori_cp bit for bit, and so does any set of ranges that tiles it. */
#define TACKER_CP_X_PARTS 4
TK_API int tacker_cp_blocks(int volx, int voly);
/* No counterpart in the reference. The cp kernels evaluate 1.0f / sqrtf(r2) with a short
 * instruction sequence where r2 is in [2^-20, 2^20) and with the general IEEE expansions
 * elsewhere; this runs the short sequence on the GPU for every float with bit pattern in
 * [lo_bits, hi_bits) and writes to *mismatches how many results differ from
 * 1.0f / sqrtf(x) in any bit (0 for the whole range [0x35800000, 0x49800000)). */
TK_API int tacker_cp_inv_sqrt_selftest(unsigned lo_bits, unsigned hi_bits, unsigned long long *mismatches);
TK_API int tacker_ori_cp(int numatoms, float gridspacing, float *energygrid, int volx, int voly,
                         tkStream_t stream);
TK_API int tacker_gptb_cp(int numatoms, float gridspacing, float *energygrid, int volx, int voly,
                          int block_start, int block_end, int launch_grid, int launch_block,
                          tkStream_t stream);

/* The fused launches: <be>_tzgemm_mix through MixKernel
 * (src/mix_kernel/tzgemm_{stencil,lbm,mriq,cp}.cu, src/MixKernel.h:55-104,
 * src/TaskManager.cu:253-264).  One launch carries the vector kernel's blocks
 * [be_start, be_end) and the GEMM tiles [tile_start, tile_end).  variant selects
 * the fused code path ("" or NULL = the kinfo default; "wg" = workgroup-split;
 * "wave" = wave-split inside each workgroup). launch_grid / launch_block 0 =
 * kinfo's gridsize * CUs / blocksize. */
TK_API int tacker_mix_tzgemm_stencil(float c0, float c1, const float *A0, float *Anext, int nx,
                                     int ny, int nz, int be_start, int be_end, const void *A,
                                     const void *B, float *C, int M, int N, int K, int tile_start,
                                     int tile_end, const char *variant, int launch_grid,
                                     int launch_block, tkStream_t stream);
TK_API int tacker_mix_tzgemm_lbm(const float *src, float *dst, int sx, int sy, int sz, int be_start,
                                 int be_end, const void *A, const void *B, float *C, int M, int N,
                                 int K, int tile_start, int tile_end, const char *variant,
                                 int launch_grid, int launch_block, tkStream_t stream);
TK_API int tacker_mix_tzgemm_mriq(int numK, const float *x, const float *y, const float *z,
                                  float *Qr, float *Qi, int numX, int be_start, int be_end,
                                  const void *A, const void *B, float *C, int M, int N, int K,
                                  int tile_start, int tile_end, const char *variant,
                                  int launch_grid, int launch_block, tkStream_t stream);
/* src/mix_kernel/tzgemm_mrif.cu */
TK_API int tacker_mix_tzgemm_mrif(int numK, const float *x, const float *y, const float *z,
                                  float *outR, float *outI, int numX, int be_start, int be_end,
                                  const void *A, const void *B, float *C, int M, int N, int K,
                                  int tile_start, int tile_end, const char *variant,
                                  int launch_grid, int launch_block, tkStream_t stream);
/* src/mix_kernel/tzgemm_sgemm.cu: the best-effort SGEMM (sA, sB, sC, sM, sN, sK) first, then the
 * latency-critical GEMM, as MixKernel concatenates them */
TK_API int tacker_mix_tzgemm_sgemm(const float *sA, const float *sB, float *sC, int sM, int sN, int sK,
                                   int be_start, int be_end, const void *A, const void *B, float *C,
                                   int M, int N, int K, int tile_start, int tile_end,
                                   const char *variant, int launch_grid, int launch_block,
                                   tkStream_t stream);
/* src/mix_kernel/tzgemm_cutcp.cu */
TK_API int tacker_mix_tzgemm_cutcp(int binDim_x, int binDim_y, const float *binZeroAddr, float h,
                                   float cutoff2, float inv_cutoff2, float *regionZeroAddr, int regions_x,
                                   int regions_y, int regions_z, int be_start, int be_end, const void *A,
                                   const void *B, float *C, int M, int N, int K, int tile_start,
                                   int tile_end, const char *variant, int launch_grid, int launch_block,
                                   tkStream_t stream);
/* src/mix_kernel/tzgemm_fft.cu */
TK_API int tacker_mix_tzgemm_fft(float *data, int batches, int be_start, int be_end, const void *A,
                                 const void *B, float *C, int M, int N, int K, int tile_start,
                                 int tile_end, const char *variant, int launch_grid, int launch_block,
                                 tkStream_t stream);
/* src/mix_kernel/tzgemm_nn.cu, tzgemm_hot3d.cu, tzgemm_path.cu, tzgemm_lava.cu */
TK_API int tacker_mix_tzgemm_lava(float alpha, int boxes1d, const float *rv, const float *qv, float *fv,
                                  int be_start, int be_end, const void *A, const void *B, float *C, int M,
                                  int N, int K, int tile_start, int tile_end, const char *variant,
                                  int launch_grid, int launch_block, tkStream_t stream);
TK_API int tacker_mix_tzgemm_nn(const float *locations, float *distances, int numRecords, float lat,
                                float lng, int be_start, int be_end, const void *A, const void *B,
                                float *C, int M, int N, int K, int tile_start, int tile_end,
                                const char *variant, int launch_grid, int launch_block, tkStream_t stream);
TK_API int tacker_mix_tzgemm_hot3d(const float *p, const float *tIn, float *tOut, int nx, int ny, int nz,
                                   int be_start, int be_end, const void *A, const void *B, float *C, int M,
                                   int N, int K, int tile_start, int tile_end, const char *variant,
                                   int launch_grid, int launch_block, tkStream_t stream);
TK_API int tacker_mix_tzgemm_path(int iteration, const int *wall, const int *src, int *results, int cols,
                                  int rows, int startStep, int be_start, int be_end, const void *A,
                                  const void *B, float *C, int M, int N, int K, int tile_start,
                                  int tile_end, const char *variant, int launch_grid, int launch_block,
                                  tkStream_t stream);
TK_API int tacker_mix_tzgemm_cp(int numatoms, float gridspacing, float *energygrid, int volx,
                                int voly, int be_start, int be_end, const void *A, const void *B,
                                float *C, int M, int N, int K, int tile_start, int tile_end,
                                const char *variant, int launch_grid, int launch_block,
                                tkStream_t stream);

/* im2col_gpu_kernel_ and convertFp32ToFp16_ (src/TaskManager.cu:48-90) */
TK_API int tacker_im2col(const float *data_im, int channels, int height, int width, int kernel_h,
                         int kernel_w, int pad_h, int pad_w, int stride_h, int stride_w,
                         int dilation_h, int dilation_w, float *data_col, tkStream_t stream);
TK_API int tacker_convert_fp32_to_fp16(void *out_f16, const float *in, int n, tkStream_t stream);
/* get_mnk_from_cudnn_args (src/TaskManager.cu:92-123) */
TK_API int tacker_mnk_from_conv_args(const int args[14], int mnk[3]);

/* kinfo lookups (src/json.cc:9-42): get_kernel_info / fget_kernel_info; a missing
 * key gives JSON_NOT_FOUND = -32767. */
TK_API int tacker_get_kernel_info(const char *kernel, const char *key);
TK_API float tacker_fget_kernel_info(const char *kernel, const char *key);

/* ---- object API: the class layer itself, one handle per C++ object ---------- */
typedef void *tacker_kernel_t;

/* createKernel (src/Creator.cu:21-337) for the names cp, cutcp, fft, lbm, mrif, mriq, sgemm, stencil,
 * tzgemm: the memoised GPTBKernel that owns seeded device buffers exactly as the
 * reference's Ori*Kernel::initParams builds them. Never destroy these. */
TK_API tacker_kernel_t tacker_create_kernel(const char *name);

/* Ori*Kernel objects over caller-owned device buffers (the reference's
 * Ori*Kernel(id) constructors allocate their own; see tacker_create_kernel). */
TK_API tacker_kernel_t tacker_ori_stencil_create(float c0, float c1, const float *A0, float *Anext,
                                                 int nx, int ny, int nz);
TK_API tacker_kernel_t tacker_ori_lbm_create(const float *src, float *dst, int sx, int sy, int sz);
TK_API tacker_kernel_t tacker_ori_mriq_create(int numK, const float *x, const float *y,
                                              const float *z, float *Qr, float *Qi, int numX);
TK_API tacker_kernel_t tacker_ori_sgemm_create(const float *A, const float *B, float *C, int M, int N,
                                               int K);
TK_API tacker_kernel_t tacker_ori_fft_create(float *data, int batches);
TK_API tacker_kernel_t tacker_ori_nn_create(const float *locations, float *distances, int numRecords,
                                            float lat, float lng);
TK_API tacker_kernel_t tacker_ori_hot3d_create(const float *p, const float *tIn, float *tOut, int nx, int ny,
                                               int nz);
TK_API tacker_kernel_t tacker_ori_lava_create(float alpha, int boxes1d, const float *rv, const float *qv,
                                              float *fv);
TK_API tacker_kernel_t tacker_ori_path_create(int iteration, const int *wall, const int *src, int *results,
                                              int cols, int rows, int startStep);
TK_API tacker_kernel_t tacker_ori_cutcp_create(int binDim_x, int binDim_y, const float *binZeroAddr, float h,
                                               float cutoff2, float inv_cutoff2, float *regionZeroAddr,
                                               int regions_x, int regions_y, int regions_z);
TK_API tacker_kernel_t tacker_ori_mrif_create(int numK, const float *x, const float *y,
                                              const float *z, float *outR, float *outI, int numX);
TK_API tacker_kernel_t tacker_ori_cp_create(int numatoms, float gridspacing, float *energygrid,
                                            int volx, int voly);
/* OriTZGEMMKernel(id, m, n, k) (src/tzgemm_kernel.h:56-147); m, n, k are rounded
 * by getTZGEMMGridDim's rule. A == NULL selects the global ori_wmma_* buffers. */
TK_API tacker_kernel_t tacker_ori_tzgemm_create(const void *A, const void *B, float *C, int m, int n,
                                                int k);
/* The global operand buffers ori_wmma_A / _B / _C (src/TaskManager.cu:19-46) as they are now:
 * device pointers and the bytes allocated for each (they grow when a larger shape is created, so
 * ask after creating the kernel). A and B hold seeded halves, C is where such kernels write. */
TK_API int tacker_global_gemm_buffers(const void **A, const void **B, float **C, long long bytes[3]);
/* new GPTBKernel(id, name, "gptb_<name>", ori, dim3(launch_grid), dim3(launch_block),
 * start, end) (src/GPTBKernel.h:14-70). launch_grid / launch_block 0 = the
 * Creator geometry for this GPU. */
TK_API tacker_kernel_t tacker_gptb_create(tacker_kernel_t ori, int launch_grid, int launch_block,
                                          int ptb_start_block_pos, int ptb_end_block_pos);
TK_API int tacker_gptb_set_range(tacker_kernel_t gptb, int ptb_start_block_pos, int ptb_end_block_pos);
/* new MixKernel(id, "tzgemm_<be>", be, tz, grid, block, be_start, be_end,
 * tile_start, tile_end) with grid and block from kinfo (src/TaskManager.cu:253-264). */
TK_API tacker_kernel_t tacker_mix_create(tacker_kernel_t be_gptb, tacker_kernel_t tz_gptb,
                                         int be_start, int be_end, int tile_start, int tile_end,
                                         const char *variant, int launch_grid, int launch_block);
TK_API int tacker_mix_set_range(tacker_kernel_t mix, int be_start, int be_end, int tile_start,
                                int tile_end);
/* new MixKernel(id, "<first>_<second>", first, second, grid, block, start1, end1, start2, end2)
 * for two best-effort kernels, first < second alphabetically, with grid and block from
 * kinfo (the constructor calls inside createMixKernel, src/Creator.cu:346-356).
 * tacker_mix_set_range applies to the result: (start1, end1, start2, end2). */
TK_API tacker_kernel_t tacker_be_pair_create(tacker_kernel_t first_gptb, tacker_kernel_t second_gptb,
                                             int start1, int end1, int start2, int end2,
                                             const char *variant, int launch_grid);
/* createMixKernel(name) (src/Creator.cu:341-816): the memoised fused pair "<a>_<b>" of the
 * memoised kernels createKernel(a), createKernel(b) over their full ranges. Never destroy. */
TK_API tacker_kernel_t tacker_create_mix_kernel(const char *name);
/* mixcublasSgemm(gemm_args, gptb_cd_kernel, cd_start_blk, cd_end_blk) (src/TaskManager.cu:309-400):
 * one fused launch of the GEMM {M, N, K} (rounded up to whole tiles, on the global operand buffers,
 * see tacker_global_gemm_buffers) with block positions [cd_start_blk, cd_end_blk) of the best-effort
 * GPTB kernel; an empty range launches the GEMM alone.  What TaskManager calls for a latency-critical
 * kernel that declares mixable = 1 and brings no operands of its own. */
TK_API int tacker_mix_cublas_sgemm(const int mnk[3], tacker_kernel_t be_gptb, int cd_start_blk,
                                   int cd_end_blk, tkStream_t stream);
/* mixcudnnConvolutionForward(cudnn_args, ...) (src/TaskManager.cu:125-306): the same for a
 * convolution given by its 14 integers {n, c, h, w, k, c, r, s, pad_h, pad_w, stride_h, stride_w,
 * dilation_h, dilation_w}: im2col of the library's scratch image on the stream, then the fused
 * launch of the GEMM {n*ho*wo, k, r*s*c} (get_mnk_from_cudnn_args, src/TaskManager.cu:92-123). */
TK_API int tacker_mix_cudnn_convolution_forward(const int cudnn_args[14], tacker_kernel_t be_gptb,
                                                int cd_start_blk, int cd_end_blk, tkStream_t stream);
/* ModuleCenter::registerModule(moduleName, cubinPath) (src/ModuleCenter.cu:8-19): load a gfx950 code
 * object (what `hipcc --genco` writes; the build leaves the library's own kernels as
 * lib/tacker_kernels.hsaco and lib/tacker_kernels_large.hsaco) under a name.  The object's copies of
 * the device symbols the host fills by name (mri-q / mri-fhd / cp constant tables, the GEMM's
 * workspace table, the failure word) are filled from the library's at load and written along with
 * them from then on, so kernels launched from it see what tacker_*_set_* and the runtime publish. */
TK_API int tacker_register_module(const char *module_name, const char *code_object_path);
/* ModuleCenter::getFunction(moduleName, functionName) != nullptr (src/ModuleCenter.cu:21-43) */
TK_API int tacker_module_has_function(const char *module_name, const char *function_name);
/* lmode DRIVER_LAUNCH (src/Kernel.h:7-10,39) for a GPTB or fused kernel object: take its device
 * function from a registered code object by the function's name there (the loadKernel of
 * src/ori_kernel/cp_kernel.cu:423-434; e.g. "general_ptb_stencil") and launch through
 * tkModuleLaunchKernel from then on.  TK_ERROR_NOT_FOUND leaves the object as it was. */
TK_API int tacker_kernel_use_module(tacker_kernel_t kernel, const char *module_name,
                                    const char *function_name);
/* Kernel::execute(stream) */
TK_API int tacker_kernel_execute(tacker_kernel_t kernel, tkStream_t stream);
/* exchange the input and output grid of a stencil / lbm ori object (the
 * ping-pong between iterations); fused and GPTB objects built on it follow,
 * because their parameter vectors alias the ori object's fields */
TK_API int tacker_kernel_swap_buffers(tacker_kernel_t ori);
/* out = {launch grid x, launch block x, ptb_start, ptb_end, number of kernel
 * parameters, smem, ori grid x, ori grid y} (start/end are 0 for non-GPTB objects) */
TK_API int tacker_kernel_info(tacker_kernel_t kernel, int out[8]);
/* copies `bytes` (4 or 8) of kernel parameter `index` -- entry `index` of Kernel::kernelParams
 * (src/Kernel.h:36), the void*-per-argument vector every launch passes to the driver -- into
 * `out`.  How a caller reaches the buffers an Ori*Kernel(id) constructor allocated itself. */
TK_API int tacker_kernel_param(tacker_kernel_t kernel, int index, void *out, int bytes);
TK_API int tacker_kernel_destroy(tacker_kernel_t kernel);
/* value of the device word kernels raise when they have to give up; reading clears it.
 * Bit 0: a role-local barrier of a wave-split fused kernel stopped waiting (its poll is
 * bounded). Bit 1: a GEMM whose reduction is shared by workgroups found no workspace bound to
 * its C (a hand-made launch on a buffer the library never saw) and left C untouched.
 * 0 = neither ever happened */
TK_API int tacker_spin_fail_flag(int *flag);
/* host half conversion used for the synthetic GEMM operands (round to nearest even) */
TK_API uint16_t tacker_float_to_half_bits(float f);
/* the seeded generator behind every synthetic input: fills out[n] with uniform
 * [lo,hi) floats of the stream started by seed */
TK_API int tacker_rng_uniform(uint64_t seed, float lo, float hi, float *out, size_t n);

/* ---- the latency-critical task and the scheduler ------------------------------ */
typedef void *tacker_task_t;
typedef void *tacker_task_manager_t;

/* createTask (src/main.cu:227-244): "vgg16" builds VGG16 at batch 1 with
 * random-initialised f16 weights; height/width 0 = 224. */
TK_API tacker_task_t tacker_task_create(const char *model, int height, int width);
TK_API int tacker_task_destroy(tacker_task_t task);
/* Task::initExecution + every kernel's execute(stream) (the warm-up loop of
 * src/main.cu:290-297) */
TK_API int tacker_task_execute(tacker_task_t task, tkStream_t stream);
/* Task::initExecution alone (src/Task.h:24 of the reference; VGG16's copies the query's input to
 * the device, synchronously) */
TK_API int tacker_task_stage_input(tacker_task_t task);
/* The task's launches recorded from `stream` into one graph (no counterpart in the reference, which
 * launches a query kernel by kernel): every kernel's execute(stream) between tkStreamBeginCapture
 * and tkStreamEndCapture, none of them run.  Call tacker_task_execute once before, so that no
 * kernel still has a buffer to allocate; per query then tacker_task_stage_input + tkGraphLaunch.
 * The graph holds the task's buffers by address: destroy it (tkGraphExecDestroy) before the task. */
TK_API int tacker_task_capture(tacker_task_t task, tkStream_t stream, tkGraphExec_t *exec);
TK_API int tacker_task_kernel_count(tacker_task_t task);
/* name (up to name_cap bytes), mixable flag, getArgs() (up to 14 ints, count in *nargs) */
TK_API int tacker_task_kernel_info(tacker_task_t task, int index, char *name, int name_cap,
                                   int *mixable, int args[14], int *nargs);
/* VGG16 only: the buffer layer conv_index writes (0..12 the convolutions, 13..15 the three fully
 * connected layers, whose result is one row: H = W = 1): device pointer and dims = {H, W, channels,
 * channel stride}.  It holds the raw GEMM output 1.1 * A * B^T; the layer that reads it adds the bias
 * and rectifies.  logits = the first `count` floats of the last layer's buffer */
TK_API int tacker_task_activation(tacker_task_t task, int conv_index, float **ptr, int dims[4]);
TK_API int tacker_task_logits(tacker_task_t task, const float **ptr, long *stride, int *count);
/* VGG16 only: weights (f16 [dims[0]][dims[1]] = [Cout padded][9*Cin padded], k =
 * (kh*3+kw)*Cin + c) and bias (f32 [dims[0]]) of convolution conv_index; 13..15: of the fully
 * connected layers ([out padded][in padded]; the last one has no bias: NULL) */
TK_API int tacker_task_conv_params(tacker_task_t task, int conv_index, void **weights, float **bias,
                                   int dims[2]);
TK_API int tacker_task_input(tacker_task_t task, float **host_ptr, int *bytes);

/* TaskManager(lc_task, be1, be2) (src/TaskManager.h:7-18) */
TK_API tacker_task_manager_t tacker_task_manager_create(tacker_task_t lc_task, const char *be_task1,
                                                        const char *be_task2);
TK_API int tacker_task_manager_destroy(tacker_task_manager_t tm);
/* the constants the reference hard-codes: 50 ms budget, 4 ms guard, 5 warm-up,
 * 10 profiling and 5 co-located queries (src/TaskManager.cu:430,446,569-586);
 * a negative value keeps the current setting */
TK_API int tacker_task_manager_configure(tacker_task_manager_t tm, float qos_budget_ms, float guard_ms,
                                         int warmup_queries, int profile_queries, int queries,
                                         int verbose);
/* executeAllTasks (second_stage != 0) or execute_with_one_cd_kernel; mode 0 = Aker
 * (ratio-limited BE slice per GEMM), 1 = Tacker (whole BE kernel per GEMM) */
TK_API int tacker_task_manager_run(tacker_task_manager_t tm, int mode, tkStream_t stream,
                                   int second_stage);
/* out = {lc_solo_ms, be1_solo_ms, be2_solo_ms, be_blocks_executed, mix_times,
 * mixable_times, time_earned_ms, qos_headroom_left_ms, stage1_be_ms, stage2_be_ms,
 * be_task_finish_num, n co-located latencies, n solo latencies} */
TK_API int tacker_task_manager_report(tacker_task_manager_t tm, float out[13]);
/* No counterpart in the reference (its hot loop, src/TaskManager.cu:586-640, fuses every mixable
 * kernel of every query): an LC kernel whose fused launch lost against "LC alone, then the BE
 * share alone" `limit` times in a row is launched alone from then on, with one more fused launch
 * every 64 queries (Aker mode only).  Default 3; 0 restores the reference's behaviour. */
TK_API int tacker_task_manager_set_fusion_strikes(tacker_task_manager_t tm, int limit);
/* No counterpart in the reference (it takes tiles x block_ratio(K) from kinfo,
 * src/TaskManager.cu:593-600): with on != 0 an Aker-mode run first times, for every mixable LC
 * kernel, its fused launch with be_total / 256, / 128, ... best-effort blocks and then co-locates
 * the count that earned most among those that kept the fused launch within (1 + max_stretch) of
 * the kernel alone (none: the kernel runs alone).  For layers that leave most CUs without a tile.
 * tacker_task_manager_calibrated_blocks copies the counts of the last run (one per LC kernel). */
TK_API int tacker_task_manager_set_calibration(tacker_task_manager_t tm, int on, float max_stretch);
TK_API int tacker_task_manager_calibrated_blocks(tacker_task_manager_t tm, int *out, int cap);
/* No counterpart in the reference.  With query_stretch > 0 the calibration pass chooses for the
 * query as a whole: per LC kernel at most one of the (count, form) options it timed, such that
 * what the fused launches add to their kernels sums to at most query_stretch of the query's solo
 * time and the earned time is the largest possible (max_stretch of
 * tacker_task_manager_set_calibration then only bounds a single kernel).  A layer that earns
 * little for the latency it adds leaves its share to one that earns more.  0 (default): the best
 * count per kernel.  passes (default 3, at least 1): timed fused launches per option; the slices
 * of the timed launches advance through the best-effort kernel as the co-located queries' do. */
TK_API int tacker_task_manager_set_calibration_budget(tacker_task_manager_t tm, float query_stretch, int passes);
/* The calibration pass can also choose, per LC kernel, among generated forms of the fused kernel:
 * `variants` is a comma-separated list of variant names ("default" = the form kinfo names for the
 * pair, e.g. "default,wave_256"); forms the pair was not generated in are skipped.  A short layer
 * can earn more in a form with fewer best-effort waves per workgroup (a 512-thread workgroup is
 * cheaper to launch than a 768-thread one).  tacker_task_manager_calibrated_variant copies the form
 * kept for LC kernel `kernel` in the last run ("" = default) and returns its length, -1 on error. */
TK_API int tacker_task_manager_set_calibration_variants(tacker_task_manager_t tm, const char *variants);
TK_API int tacker_task_manager_calibrated_variant(tacker_task_manager_t tm, int kernel, char *out, int cap);
/* LC kernels barred from fusion at the end of the last run */
TK_API int tacker_task_manager_fusion_disabled(tacker_task_manager_t tm);
/* "[Mix] BE task1 + task2 took ..." (src/TaskManager.cu:693): average time of the fused launch of
 * the two best-effort kernels measured by the last run with a second stage; 0 if none ran. */
TK_API float tacker_task_manager_be_mix_ms(tacker_task_manager_t tm);
/* No counterpart in the reference (its query latency is a sum of per-kernel intervals with a
 * synchronisation after each, src/TaskManager.cu:620-624): after the co-located queries, run
 * `queries` more of each kind -- every kernel alone, and with the best-effort blocks the last
 * co-located query carried -- with nothing between the launches of a query, each timed by one
 * pair of events and by the host's steady clock.  0 (default) = off. */
TK_API int tacker_task_manager_set_end_to_end(tacker_task_manager_t tm, int queries);
/* which = 0: per-query latency of the co-located queries (sum of per-kernel intervals), 1: of the
 * solo profiling queries; end-to-end queries (tacker_task_manager_set_end_to_end): 2 co-located and
 * 3 solo by events, 4 co-located and 5 solo by the host clock; 6 and 7: the solo query recorded once
 * from a stream and launched as one graph per query (tkStreamBeginCapture .. tkGraphLaunch), by
 * events and by the host clock -- no counterpart in the reference, which launches kernel by kernel */
TK_API int tacker_task_manager_latencies(tacker_task_manager_t tm, int which, float *out, int cap);

/* the scheduler's arithmetic on its own (src/TaskManager.cu:586-640) */
TK_API float tacker_qos_block_ratio(const char *be_name, int K_GLOBAL);
/* No counterpart in the reference (its Tacker mode always fuses the whole best-effort kernel,
 * src/TaskManager.cu:599): kinfo's measured gain (serial time / fused time) of a fused launch that
 * carries the whole best-effort kernel, 1 when kinfo holds none. Below 1 the scheduler carries the
 * Aker-mode slice in Tacker mode too. */
TK_API float tacker_qos_whole_kernel_gain(const char *be_name);
/* mode: 0 = Aker, 1 = Tacker (enum ExecutionMode) */
TK_API int tacker_qos_colocated_blocks(int mode, const char *be_name, int tiles, int K_GLOBAL,
                                       int be_total_blocks);
TK_API int tacker_qos_must_run_solo(float budget_ms, float guard_ms, float qos_headroom,
                                    float lc_time_remaining);
/* out = {counted_as_mixed, charged_ms, earned_ms} */
TK_API int tacker_qos_account(int mixable, float measured_ms, float solo_lc_ms, float be_ms,
                              int cd_blocks, int be_total_blocks, float out[3]);

#ifdef __cplusplus
}
#endif
#endif /* TACKER_AMD_H */
