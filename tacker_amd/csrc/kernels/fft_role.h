// FFT role: Parboil's batched 256-point complex transform (src/ori_kernel/fft_kernel.cu:11-61,
// src/gptb_kernel/fft_kernel.cu:3-75 of the reference), one transform per block position, in place.
//
// The reference gives a transform to a block of 128 threads: thread j holds the two points
// j and j + 128, and each of the 8 radix-2 stages multiplies the second by a twiddle, takes the
// butterfly and exchanges the 256 values through shared memory between two block barriers.  A role
// of a fused kernel cannot use the block barrier (it would wait for the other role's waves), so here
// one wavefront serves a transform: lane l plays the reference's threads l and l + 64, the exchange
// goes through 2 KiB of LDS that belong to the wave, and the wave's own program order is all the
// synchronisation there is (LDS serves a wave's accesses in order).  Same stages, same butterflies,
// same operation order per value; the twiddles come from a table of correctly rounded values where
// the reference calls cos and sin on a rounded angle.
#pragma once
#include <hip/hip_runtime.h>

#include "../header/fft_header.h"
#include "role_common.h"

namespace tk {

typedef float fft_c32 __attribute__((ext_vector_type(2)));   // (re, im)
typedef __attribute__((address_space(3))) fft_c32 fft_lds_c32;

// exp(-2 pi i k / 256), k = 0 .. 127: stage Ns uses entry (j % Ns) * (128 / Ns)
// (angle = -2 pi (j % Ns) / (2 Ns), src/ori_kernel/fft_kernel.cu:35)
static __device__ const float fft_twiddle[FFT_T][2] = {
    {1.0f, -0.0f}, {0.999698818f, -0.024541229f}, {0.99879545f, -0.0490676761f}, {0.997290432f, -0.0735645667f},
    {0.99518472f, -0.0980171412f}, {0.992479563f, -0.122410677f}, {0.989176512f, -0.146730468f}, {0.985277653f, -0.170961887f},
    {0.980785251f, -0.195090324f}, {0.975702107f, -0.219101235f}, {0.970031261f, -0.242980182f}, {0.963776052f, -0.266712755f},
    {0.956940353f, -0.290284663f}, {0.949528158f, -0.313681751f}, {0.941544056f, -0.336889863f}, {0.932992816f, -0.359895051f},
    {0.923879504f, -0.382683426f}, {0.914209783f, -0.405241311f}, {0.903989315f, -0.427555084f}, {0.893224299f, -0.449611336f},
    {0.881921291f, -0.471396744f}, {0.870086968f, -0.492898196f}, {0.857728601f, -0.514102757f}, {0.84485358f, -0.534997642f},
    {0.831469595f, -0.555570245f}, {0.817584813f, -0.575808167f}, {0.803207517f, -0.59569931f}, {0.78834641f, -0.615231574f},
    {0.773010433f, -0.634393275f}, {0.757208824f, -0.653172851f}, {0.740951121f, -0.671558976f}, {0.724247098f, -0.689540565f},
    {0.707106769f, -0.707106769f}, {0.689540565f, -0.724247098f}, {0.671558976f, -0.740951121f}, {0.653172851f, -0.757208824f},
    {0.634393275f, -0.773010433f}, {0.615231574f, -0.78834641f}, {0.59569931f, -0.803207517f}, {0.575808167f, -0.817584813f},
    {0.555570245f, -0.831469595f}, {0.534997642f, -0.84485358f}, {0.514102757f, -0.857728601f}, {0.492898196f, -0.870086968f},
    {0.471396744f, -0.881921291f}, {0.449611336f, -0.893224299f}, {0.427555084f, -0.903989315f}, {0.405241311f, -0.914209783f},
    {0.382683426f, -0.923879504f}, {0.359895051f, -0.932992816f}, {0.336889863f, -0.941544056f}, {0.313681751f, -0.949528158f},
    {0.290284663f, -0.956940353f}, {0.266712755f, -0.963776052f}, {0.242980182f, -0.970031261f}, {0.219101235f, -0.975702107f},
    {0.195090324f, -0.980785251f}, {0.170961887f, -0.985277653f}, {0.146730468f, -0.989176512f}, {0.122410677f, -0.992479563f},
    {0.0980171412f, -0.99518472f}, {0.0735645667f, -0.997290432f}, {0.0490676761f, -0.99879545f}, {0.024541229f, -0.999698818f},
    {0.0f, -1.0f}, {-0.024541229f, -0.999698818f}, {-0.0490676761f, -0.99879545f}, {-0.0735645667f, -0.997290432f},
    {-0.0980171412f, -0.99518472f}, {-0.122410677f, -0.992479563f}, {-0.146730468f, -0.989176512f}, {-0.170961887f, -0.985277653f},
    {-0.195090324f, -0.980785251f}, {-0.219101235f, -0.975702107f}, {-0.242980182f, -0.970031261f}, {-0.266712755f, -0.963776052f},
    {-0.290284663f, -0.956940353f}, {-0.313681751f, -0.949528158f}, {-0.336889863f, -0.941544056f}, {-0.359895051f, -0.932992816f},
    {-0.382683426f, -0.923879504f}, {-0.405241311f, -0.914209783f}, {-0.427555084f, -0.903989315f}, {-0.449611336f, -0.893224299f},
    {-0.471396744f, -0.881921291f}, {-0.492898196f, -0.870086968f}, {-0.514102757f, -0.857728601f}, {-0.534997642f, -0.84485358f},
    {-0.555570245f, -0.831469595f}, {-0.575808167f, -0.817584813f}, {-0.59569931f, -0.803207517f}, {-0.615231574f, -0.78834641f},
    {-0.634393275f, -0.773010433f}, {-0.653172851f, -0.757208824f}, {-0.671558976f, -0.740951121f}, {-0.689540565f, -0.724247098f},
    {-0.707106769f, -0.707106769f}, {-0.724247098f, -0.689540565f}, {-0.740951121f, -0.671558976f}, {-0.757208824f, -0.653172851f},
    {-0.773010433f, -0.634393275f}, {-0.78834641f, -0.615231574f}, {-0.803207517f, -0.59569931f}, {-0.817584813f, -0.575808167f},
    {-0.831469595f, -0.555570245f}, {-0.84485358f, -0.534997642f}, {-0.857728601f, -0.514102757f}, {-0.870086968f, -0.492898196f},
    {-0.881921291f, -0.471396744f}, {-0.893224299f, -0.449611336f}, {-0.903989315f, -0.427555084f}, {-0.914209783f, -0.405241311f},
    {-0.923879504f, -0.382683426f}, {-0.932992816f, -0.359895051f}, {-0.941544056f, -0.336889863f}, {-0.949528158f, -0.313681751f},
    {-0.956940353f, -0.290284663f}, {-0.963776052f, -0.266712755f}, {-0.970031261f, -0.242980182f}, {-0.975702107f, -0.219101235f},
    {-0.980785251f, -0.195090324f}, {-0.985277653f, -0.170961887f}, {-0.989176512f, -0.146730468f}, {-0.992479563f, -0.122410677f},
    {-0.99518472f, -0.0980171412f}, {-0.997290432f, -0.0735645667f}, {-0.99879545f, -0.0490676761f}, {-0.999698818f, -0.024541229f},
};

// (a.x b.x - a.y b.y, a.x b.y + a.y b.x): operator* of src/header/fft_header.h:20
__device__ __forceinline__ fft_c32 fft_mul(fft_c32 a, fft_c32 b)
{
    fft_c32 r;
    r.x = a.x * b.x - a.y * b.y;
    r.y = a.x * b.y + a.y * b.x;
    return r;
}

// The nine twiddles a lane ever needs: stages Ns = 1 .. 64 use the same one for j = l and
// j = l + 64 (j % Ns is the same), the last stage (Ns = 128) one each.
struct FftLaneTwiddles {
    fft_c32 w[9];
};
__device__ __forceinline__ FftLaneTwiddles fft_lane_twiddles(int lane)
{
    FftLaneTwiddles t;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        const int k = (lane & ((1 << s) - 1)) << (7 - s);
        t.w[s].x = fft_twiddle[k][0];
        t.w[s].y = fft_twiddle[k][1];
    }
    t.w[8].x = fft_twiddle[lane + 64][0];
    t.w[8].y = fft_twiddle[lane + 64][1];
    return t;
}

// v[h][r]: point r of the reference's thread j = lane + 64 h.  work: the wave's 256 values of LDS.
__device__ __forceinline__ void fft_stages(fft_c32 (&v)[2][2], int lane, const FftLaneTwiddles &t, fft_lds_c32 *work)
{
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        const int Ns = 1 << s;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int j = lane + 64 * h;
            // v[0] is multiplied by (cos 0, sin 0) = (1, 0) in the reference: the value itself
            v[h][1] = fft_mul(v[h][1], (s == 7 && h == 1) ? t.w[8] : t.w[s]);
            const fft_c32 v0 = v[h][0];
            v[h][0] = v0 + v[h][1];
            v[h][1] = v0 - v[h][1];
            const int idxD = ((j >> s) << (s + 1)) + (j & (Ns - 1));   // GPU_expand(j, Ns, 2)
            work[idxD] = v[h][0];
            work[idxD + Ns] = v[h][1];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // GPU_expand(j, 128, 2) = j: thread j takes values j and j + 128
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            v[h][0] = work[lane + 64 * h];
            v[h][1] = work[lane + 64 * h + FFT_T];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
}

__device__ __forceinline__ void fft_load(fft_c32 (&v)[2][2], const fft_c32 *__restrict__ transform, int lane)
{
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int r = 0; r < 2; ++r) v[h][r] = transform[lane + 64 * h + FFT_T * r];
}

__device__ __forceinline__ void fft_store(const fft_c32 (&v)[2][2], fft_c32 *__restrict__ transform, int lane)
{
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int r = 0; r < 2; ++r) transform[lane + 64 * h + FFT_T * r] = v[h][r];
}

// the LDS of the calling wave: 256 complex values per wave of a role of up to WAVES wavefronts
template <int WAVES>
__device__ __forceinline__ fft_lds_c32 *fft_work_of_wave(int wave)
{
    __shared__ __align__(16) float fft_work[WAVES][FFT_N][2];
    return (fft_lds_c32 *)&fft_work[wave][0][0];
}

// grid_dimension_x: transforms in the batch (the reference's grid).  Block positions [start, end)
// are served by the role's role_blocks x (role_threads / 64) wavefronts in turn; a position past
// the batch wraps as the reference's block_pos % grid_dimension_x does.
template <int WAVES>
__device__ __forceinline__ void fft_role(float *__restrict__ data, int grid_dimension_x, int role_block, int role_blocks,
                                         int start, int end, int tid, int role_threads)
{
    const int waves = min(role_threads / FFT_WAVE, WAVES);
    const int wave = tid / FFT_WAVE;
    if (wave >= waves || start >= end || grid_dimension_x <= 0) return;
    const int lane = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    fft_lds_c32 *work = fft_work_of_wave<WAVES>(wave);
    fft_c32 *all = reinterpret_cast<fft_c32 *>(data);
    const FftLaneTwiddles t = fft_lane_twiddles(lane);
    const int stride = role_blocks * waves;
    int pos = start + role_block + role_blocks * wave;
    if (pos >= end) return;
    fft_c32 v[2][2], next[2][2];
    fft_load(v, all + (size_t)(pos % grid_dimension_x) * FFT_N, lane);
    for (;;) {
        const int pos_next = pos + stride;
        const bool more = pos_next < end;
        // the next transform's points are on their way while this one is computed
        if (more) fft_load(next, all + (size_t)(pos_next % grid_dimension_x) * FFT_N, lane);
        fft_stages(v, lane, t, work);
        fft_store(v, all + (size_t)(pos % grid_dimension_x) * FFT_N, lane);
        if (!more) break;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int r = 0; r < 2; ++r) v[h][r] = next[h][r];
        pos = pos_next;
    }
}

}  // namespace tk
