// Data-movement kernels of the latency-critical DNN task (VGG16, batch 1), whose
// convolutions and fully-connected layers run on tzgemm.
//
// The reference lowers a convolution with a Caffe NCHW im2col into an fp32 column
// buffer and then times ptb_tzgemm on unrelated global operands
// (src/include/dnn.h:554-803): a timing proxy.  Here the GEMM consumes the real
// activations, so im2col writes the operand tzgemm wants directly: A[M][K] f16
// with K contiguous, from NHWC fp32 activations.
#pragma once
#include <hip/hip_runtime.h>

// A[m][k] for m = (h*W + w), k = (kh*KW + kw)*C + c; zero for padding taps and for
// k in [KH*KW*C, K_pad).  Rows m >= H*W of A are never written (they stay zero).
// act is [H][W][c_stride] with c < C used.  3x3/stride-1 style parameters general.
// bias != nullptr: act is the raw output of the previous GEMM and its epilogue is applied
// on the way in, v = act + bias[c], then max(v, 0) if relu -- the values a separate
// bias/ReLU pass over act would have left there, without that pass.
// K_write (a multiple of 8, 0 = K_pad): only columns [0, K_write) of each row are written -- for an
// operand buffer of its own whose columns from K_write on were zeroed once and stay zero.
extern "C" __global__ void im2col_nhwc_f16(const float *act, int H, int W, int C, int c_stride,
                                           int KH, int KW, int pad, int stride, int Ho, int Wo,
                                           _Float16 *A, int K_pad, const float *bias, int relu, int K_write)
{
    typedef float f4 __attribute__((ext_vector_type(4)));
    typedef _Float16 h8 __attribute__((ext_vector_type(8)));
    const int k_real = KH * KW * C;
    if ((C & 7) == 0 && (c_stride & 3) == 0 && (K_pad & 7) == 0 && K_write == 0) {
        // 8 consecutive k share one tap (C is a multiple of 8): two 16-byte loads of the
        // activation, one 16-byte store of A, 32-bit index arithmetic
        const unsigned groups_per_row = (unsigned)K_pad >> 3;
        const unsigned total = (unsigned)(Ho * Wo) * groups_per_row;
        for (unsigned g = blockIdx.x * blockDim.x + threadIdx.x; g < total; g += blockDim.x * gridDim.x) {
            const unsigned m = g / groups_per_row;
            const int k = (int)(g - m * groups_per_row) << 3;
            h8 out = {0, 0, 0, 0, 0, 0, 0, 0};
            if (k < k_real) {
                const int tap = k / C;
                const int c = k - tap * C;
                const int kh = tap / KW, kw = tap - kh * KW;
                const int ho = (int)(m / (unsigned)Wo), wo = (int)(m - (unsigned)ho * (unsigned)Wo);
                const int h = ho * stride - pad + kh, w = wo * stride - pad + kw;
                if (h >= 0 && h < H && w >= 0 && w < W) {
                    const float *src = act + ((size_t)h * W + w) * c_stride + c;
                    f4 lo = *reinterpret_cast<const f4 *>(src);
                    f4 hi = *reinterpret_cast<const f4 *>(src + 4);
                    if (bias) {
                        lo += *reinterpret_cast<const f4 *>(bias + c);
                        hi += *reinterpret_cast<const f4 *>(bias + c + 4);
                        if (relu) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                lo[e] = lo[e] < 0.0f ? 0.0f : lo[e];
                                hi[e] = hi[e] < 0.0f ? 0.0f : hi[e];
                            }
                        }
                    }
                    out = h8{(_Float16)lo.x, (_Float16)lo.y, (_Float16)lo.z, (_Float16)lo.w,
                             (_Float16)hi.x, (_Float16)hi.y, (_Float16)hi.z, (_Float16)hi.w};
                }
            }
            *reinterpret_cast<h8 *>(A + (size_t)g * 8) = out;
        }
        return;
    }
    if ((K_pad & 7) == 0 && (K_write & 7) == 0 && (long)Ho * Wo * K_pad < (1L << 31)) {
        // any channel count (the first layer has 3): still one 16-byte store of A per thread and
        // 32-bit index arithmetic, the 8 values gathered one by one; groups past the real K
        // (most of the row when C is small) are just zeros
        const unsigned groups_per_row = (unsigned)(K_write > 0 ? K_write : K_pad) >> 3;
        const unsigned total = (unsigned)(Ho * Wo) * groups_per_row;
        for (unsigned g = blockIdx.x * blockDim.x + threadIdx.x; g < total; g += blockDim.x * gridDim.x) {
            const unsigned m = g / groups_per_row;
            const int k0 = (int)(g - m * groups_per_row) << 3;
            h8 out = {0, 0, 0, 0, 0, 0, 0, 0};
            if (k0 < k_real) {
                const int ho = (int)(m / (unsigned)Wo), wo = (int)(m - (unsigned)ho * (unsigned)Wo);
                // (kh, kw, c) of k0 by division, of the 7 that follow by counting up
                int tap = (int)((unsigned)k0 / (unsigned)C);
                int c = k0 - tap * C;
                int kh = (int)((unsigned)tap / (unsigned)KW), kw = tap - kh * KW;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    if (k0 + e < k_real) {
                        const int h = ho * stride - pad + kh, w = wo * stride - pad + kw;
                        if (h >= 0 && h < H && w >= 0 && w < W) {
                            float v = act[((size_t)h * W + w) * c_stride + c];
                            if (bias) {
                                v += bias[c];
                                if (relu && v < 0.0f) v = 0.0f;
                            }
                            out[e] = (_Float16)v;
                        }
                    }
                    if (++c == C) {
                        c = 0;
                        if (++kw == KW) {
                            kw = 0;
                            ++kh;
                        }
                    }
                }
            }
            *reinterpret_cast<h8 *>(A + (size_t)m * K_pad + k0) = out;
        }
        return;
    }
    const long total = (long)Ho * Wo * K_pad;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (long)blockDim.x * gridDim.x) {
        const int k = (int)(i % K_pad);
        const long m = i / K_pad;
        float v = 0.0f;
        if (k < k_real) {
            const int c = k % C;
            const int tap = k / C;
            const int kw = tap % KW, kh = tap / KW;
            const int wo = (int)(m % Wo), ho = (int)(m / Wo);
            const int h = ho * stride - pad + kh, w = wo * stride - pad + kw;
            if (h >= 0 && h < H && w >= 0 && w < W) {
                v = act[((long)h * W + w) * c_stride + c];
                if (bias) {
                    v += bias[c];
                    if (relu && v < 0.0f) v = 0.0f;
                }
            }
        }
        A[i] = (_Float16)v;
    }
}

// The same operand for a 3x3 / pad 1 / stride 1 convolution with C a multiple of 8, built the other
// way round: a thread takes 8 channels of one input pixel, reads them once (bias and ReLU applied as
// above) and stores them to the up to 9 rows of A whose window covers the pixel -- A[(ho*W + wo)][tap*C
// + c] with ho = h + 1 - kh, wo = w + 1 - kw.  The gather form reads every activation 9 times (18 bytes
// read per byte of A written); this one reads it once.  What no pixel writes is zero and is written by
// the thread of the row's own pixel: the taps of its window that fall outside the image, and the
// columns from 9*C up to K_pad.  Every element of rows < H*W is written exactly once.
// pool != 0: act is [2H][2W][c_stride] and the pixel is the maximum of its 2x2 cell, taken before the
// bias and the ReLU exactly as maxpool2x2_nhwc takes it -- the pooling layer between two
// convolutions without a launch and without its round trip through memory.
extern "C" __global__ void im2col3x3_scatter_nhwc_f16(const float *act, int H, int W, int C, int c_stride,
                                                      _Float16 *A, int K_pad, const float *bias, int relu,
                                                      int pool)
{
    typedef float f4 __attribute__((ext_vector_type(4)));
    typedef _Float16 h8 __attribute__((ext_vector_type(8)));
    const unsigned groups = (unsigned)C >> 3;                 // 8-channel groups of a pixel
    const unsigned total = (unsigned)(H * W) * groups;
    const unsigned row_groups = (unsigned)K_pad >> 3;
    const h8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    for (unsigned id = blockIdx.x * blockDim.x + threadIdx.x; id < total; id += blockDim.x * gridDim.x) {
        const unsigned p = id / groups;
        const int c = (int)(id - p * groups) << 3;
        const int h = (int)(p / (unsigned)W), w = (int)(p - (unsigned)h * (unsigned)W);
        f4 lo, hi;
        if (pool) {
            const size_t right = (size_t)c_stride, below = (size_t)(2 * W) * c_stride;
            const float *src = act + ((size_t)(2 * h) * (2 * W) + 2 * w) * c_stride + c;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const float *s4 = src + 4 * half;
                const f4 a = *reinterpret_cast<const f4 *>(s4);
                const f4 b = *reinterpret_cast<const f4 *>(s4 + right);
                const f4 d = *reinterpret_cast<const f4 *>(s4 + below);
                const f4 e = *reinterpret_cast<const f4 *>(s4 + below + right);
                f4 m;
#pragma unroll
                for (int i = 0; i < 4; ++i) m[i] = fmaxf(fmaxf(a[i], b[i]), fmaxf(d[i], e[i]));
                if (half == 0) lo = m;
                else hi = m;
            }
        } else {
            const float *src = act + (size_t)p * c_stride + c;
            lo = *reinterpret_cast<const f4 *>(src);
            hi = *reinterpret_cast<const f4 *>(src + 4);
        }
        if (bias) {
            lo += *reinterpret_cast<const f4 *>(bias + c);
            hi += *reinterpret_cast<const f4 *>(bias + c + 4);
            if (relu) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    lo[e] = lo[e] < 0.0f ? 0.0f : lo[e];
                    hi[e] = hi[e] < 0.0f ? 0.0f : hi[e];
                }
            }
        }
        const h8 v = {(_Float16)lo.x, (_Float16)lo.y, (_Float16)lo.z, (_Float16)lo.w,
                      (_Float16)hi.x, (_Float16)hi.y, (_Float16)hi.z, (_Float16)hi.w};
        _Float16 *own = A + (size_t)p * K_pad + c;             // this pixel's row, this channel group
#pragma unroll
        for (int kh = 0; kh < 3; ++kh)
#pragma unroll
            for (int kw = 0; kw < 3; ++kw) {
                const int tap = (kh * 3 + kw) * C;
                const int ho = h + 1 - kh, wo = w + 1 - kw;    // row whose tap (kh, kw) is this pixel
                if (ho >= 0 && ho < H && wo >= 0 && wo < W)
                    *reinterpret_cast<h8 *>(A + (size_t)(ho * W + wo) * K_pad + tap + c) = v;
                const int hs = h - 1 + kh, ws = w - 1 + kw;    // pixel under tap (kh, kw) of the own row
                if (hs < 0 || hs >= H || ws < 0 || ws >= W) *reinterpret_cast<h8 *>(own + tap) = zero;
            }
        for (unsigned g = 9 * groups + ((unsigned)c >> 3); g < row_groups; g += groups)
            *reinterpret_cast<h8 *>(A + (size_t)p * K_pad + (size_t)g * 8) = zero;
    }
}

// 2x2 / stride 2 max pooling, NHWC with channel stride ld.  The network itself pools while it builds
// the next operand (im2col3x3_scatter_nhwc_f16, pack_fc_input_pooled); this kernel is the plain
// statement of what they compute, and what the tests hold them against.  bias != nullptr: in is the raw
// output of the previous GEMM; out = max(in) + bias[c], then max(., 0) if relu, which is what
// pooling the biased, rectified values gives (x -> fl(x + b) and ReLU are non-decreasing).
extern "C" __global__ void maxpool2x2_nhwc(const float *in, int H, int W, int ld, float *out,
                                           const float *bias, int relu)
{
    const int Ho = H / 2, Wo = W / 2;
    const long total = (long)Ho * Wo * ld;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (long)blockDim.x * gridDim.x) {
        const int c = (int)(i % ld);
        const long p = i / ld;
        const int wo = (int)(p % Wo), ho = (int)(p / Wo);
        const float *src = in + ((long)(2 * ho) * W + 2 * wo) * ld + c;
        const float a = src[0], b = src[ld], d = src[(long)W * ld], e = src[(long)W * ld + ld];
        float v = fmaxf(fmaxf(a, b), fmaxf(d, e));
        if (bias) {
            v += bias[c];
            if (relu && v < 0.0f) v = 0.0f;
        }
        out[i] = v;
    }
}

// Fully-connected layers run as C[out][128] = W[out][K] * X[128][K]^T with the
// batch-1 activation in row 0 of X: pack an fp32 vector (taken with a stride, so
// it can be column 0 of the previous layer's output) into that f16 row, with an
// optional bias + ReLU on the way.
extern "C" __global__ void pack_fc_input(const float *src, long src_stride, const float *bias, int relu,
                                         int n, _Float16 *x_row)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
        float v = src[(long)i * src_stride];
        if (bias) v += bias[i];
        if (relu && v < 0.0f) v = 0.0f;
        x_row[i] = (_Float16)v;
    }
}

// The same row from the raw output of the last convolution, [2*Ho][W][ld] with C channels used, through
// the 2x2 max pooling that precedes the classifier: element i = (ho*Wo + wo)*C + c of the NHWC
// flattening is the maximum of its 2x2 cell, then + bias[c], then ReLU -- the operations of
// maxpool2x2_nhwc followed by pack_fc_input, in their order.
extern "C" __global__ void pack_fc_input_pooled(const float *in, int W, int ld, int C, const float *bias,
                                                int relu, int n, _Float16 *x_row)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
        const int c = i % C;
        const int p = i / C;
        const int Wo = W / 2;
        const int wo = p % Wo, ho = p / Wo;
        const float *src = in + ((long)(2 * ho) * W + 2 * wo) * ld + c;
        const float a = src[0], b = src[ld], d = src[(long)W * ld], e = src[(long)W * ld + ld];
        float v = fmaxf(fmaxf(a, b), fmaxf(d, e));
        if (bias) {
            v += bias[c];
            if (relu && v < 0.0f) v = 0.0f;
        }
        x_row[i] = (_Float16)v;
    }
}
