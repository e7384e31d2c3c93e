// The two paths of the convolution entry points for input channel counts that are not a multiple of the
// 16-byte chunk the implicit-GEMM gather works in (first layers with IC = 1 or 3, odd channel counts).
//
// Channel padding (pad_channels_kernel, at the end of this file): activations and weights are copied once with
// IC rounded up to the chunk, zero-filled, and the implicit gather runs on the copies.  Taken when the
// padded count is at most 8/3 of IC: the copy moves the input once, where a column buffer is written and
// read back kH*kW / stride^2 times as large (an 11x11 stride-4 IC = 3 layer at batch 32, FP32: 300 -> 136 us).
//
// Explicit im2col, for the thinner inputs (IC = 1, 2 in FP16, 1 in FP32), where padding would multiply
// the MFMA work by 4 to 8: the reference's own algorithm -- a column buffer followed by the GEMM
// (src_template/Ampere_FP16/im2col.cu:38-97, scripts/Ampere_FP16/Ampere_FP16_conv.py:431-446) -- on NHWC data:
//
//   col[m][k] = x[b][oh*stride - pad + kh][ow*stride - pad + kw][c],   m = (b*OH + oh)*OW + ow,
//                                                                      k = (kh*kW + kw)*IC + c,
//   zero where the tap falls outside the image and for the padding columns k >= K.
//
// The buffer is written in the operand layout the template's GEMM takes for A: row-major M x ldk for the
// FP16 templates (K contiguous), K x ldm for the FP32 template (M contiguous); the weights are repacked to
// the matching B layout (N x ldk with zero-padded K, or K x ldn).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "helix_fastdiv.h"

namespace helix_im2col {
namespace {   // internal linkage: every template library carries its own copy and exports none of it

using helix_fastdiv::FastDiv;

struct Geom {
    int H, W, IC, OH, OW, kW, stride, pad;
    int M, K;   // M = batch*OH*OW, K = kH*kW*IC
    FastDiv by_OW, by_OH, by_IC, by_kW;   // multiply-shift division by the run-time extents
};

inline Geom make_geom(int H, int W, int IC, int OH, int OW, int kW, int stride, int pad, int M, int K) {
    return Geom{H, W, IC, OH, OW, kW, stride, pad, M, K,
                helix_fastdiv::make(OW), helix_fastdiv::make(OH), helix_fastdiv::make(IC), helix_fastdiv::make(kW)};
}

// Output row m -> image base (in pixels) and the image coordinates of its top-left filter tap.
struct Pixel { int img, ih0, iw0; };

__device__ __forceinline__ Pixel pixel_of(const Geom& g, int m) {
    const int t = g.by_OW.div(m);
    const int ow = m - t * g.OW;
    const int b = g.by_OH.div(t);
    const int oh = t - b * g.OH;
    return Pixel{b * g.H * g.W, oh * g.stride - g.pad, ow * g.stride - g.pad};
}

// K-contiguous column buffer: col[m*ldk + k], k < ldk (ldk a multiple of VEC); one thread writes VEC
// consecutive k of one row with a single store.  The row is decomposed once per thread, the first k of the
// chunk once, and (channel, tap column, tap row) then step from element to element.
// `by_chunks` divides by ldk / VEC; M * (ldk / VEC) must fit 31 bits (checked by the caller).
template <typename T, int VEC>
__global__ void im2col_rows_kernel(const T* x, T* col, Geom g, int ldk, FastDiv by_chunks) {
    const int chunks = by_chunks.d;
    const int total = g.M * chunks;
    // the running index is 64-bit: total may lie within one grid stride of 2^31, where a 32-bit index would wrap
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x) {
        const int idx = (int)i;
        const int m = by_chunks.div(idx), k0 = (idx - m * chunks) * VEC;
        const Pixel px = pixel_of(g, m);
        int f = g.by_IC.div(k0);
        int c = k0 - f * g.IC;
        int kh = g.by_kW.div(f);
        int kw = f - kh * g.kW;
        T v[VEC];
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            const int ih = px.ih0 + kh, iw = px.iw0 + kw;
            const bool ok = (k0 + j < g.K) && ih >= 0 && ih < g.H && iw >= 0 && iw < g.W;
            v[j] = ok ? x[((size_t)px.img + (size_t)ih * g.W + iw) * g.IC + c] : (T)0;
            if (++c == g.IC) {
                c = 0;
                if (++kw == g.kW) { kw = 0; ++kh; }
            }
        }
        T* dst = col + (size_t)m * ldk + k0;
#pragma unroll
        for (int j = 0; j < VEC; j++) dst[j] = v[j];
    }
}

// M-contiguous column buffer: col[k*ldm + m], m < ldm.  blockIdx.y walks k (tap and channel are uniform per
// workgroup), consecutive threads write consecutive m.
template <typename T>
__global__ void im2col_cols_kernel(const T* x, T* col, Geom g, int ldm) {
    for (int k = blockIdx.y; k < g.K; k += gridDim.y) {
        const int f = g.by_IC.div(k);
        const int c = k - f * g.IC;
        const int kh = g.by_kW.div(f);
        const int kw = f - kh * g.kW;
        T* row = col + (size_t)k * ldm;
        for (int m = blockIdx.x * blockDim.x + threadIdx.x; m < ldm; m += gridDim.x * blockDim.x) {
            T v = (T)0;
            if (m < g.M) {
                const Pixel px = pixel_of(g, m);
                const int ih = px.ih0 + kh, iw = px.iw0 + kw;
                if (ih >= 0 && ih < g.H && iw >= 0 && iw < g.W) v = x[((size_t)px.img + (size_t)ih * g.W + iw) * g.IC + c];
            }
            row[m] = v;
        }
    }
}

// weights [N][K] -> [N][ldk], zero-padded
template <typename T>
__global__ void pack_weights_rows_kernel(const T* w, T* out, int N, int K, int ldk) {
    const size_t total = (size_t)N * ldk;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const int n = (int)(idx / ldk), k = (int)(idx % ldk);
        out[idx] = k < K ? w[(size_t)n * K + k] : (T)0;
    }
}

// weights [N][K] -> [K][ldn] (transposed), zero-padded
template <typename T>
__global__ void pack_weights_cols_kernel(const T* w, T* out, int N, int K, int ldn) {
    const size_t total = (size_t)K * ldn;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const int k = (int)(idx / ldn), n = (int)(idx % ldn);
        out[idx] = n < N ? w[(size_t)n * K + k] : (T)0;
    }
}

// rows x IC -> rows x ICp (ICp a multiple of VEC, >= IC), zero-filled tail; serves NHWC activations (one row
// per pixel) and [OC][kH][kW][IC] weights (one row per filter tap) alike.  One thread writes VEC consecutive
// channels of one row with a single store.  `by_chunks` divides by ICp / VEC; rows * (ICp / VEC) must fit 31 bits.
template <typename T, int VEC>
__global__ void pad_channels_kernel(const T* src, T* dst, int rows, int IC, int ICp, FastDiv by_chunks) {
    const int chunks = by_chunks.d;
    const int total = rows * chunks;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x) {
        const int idx = (int)i;
        const int r = by_chunks.div(idx), c0 = (idx - r * chunks) * VEC;
        const T* from = src + (size_t)r * IC + c0;
        struct alignas(sizeof(T) * VEC) Chunk { T v[VEC]; } chunk;
#pragma unroll
        for (int j = 0; j < VEC; j++) chunk.v[j] = (c0 + j < IC) ? from[j] : (T)0;
        *reinterpret_cast<Chunk*>(dst + (size_t)r * ICp + c0) = chunk;   // dst is aligned to the chunk by the caller
    }
}

// Channel count after padding to the gather chunk of VEC elements, and whether that path is the one taken:
// the padded count within 8/3 of IC and the padded activations within the 2 GiB a buffer descriptor spans.
inline int padded_channels(int IC, int vec) { return (IC + vec - 1) / vec * vec; }

inline bool pads_channels(int batch, int H, int W, int IC, int vec, int elem_bytes) {
    const int ICp = padded_channels(IC, vec);
    return IC % vec != 0 && 3LL * ICp <= 8LL * IC &&
           (long long)batch * H * W * ICp * elem_bytes < 0x7fffffffLL;
}

inline int grid_for(size_t total) {
    size_t b = (total + 255) / 256;
    return (int)(b > 65536 ? 65536 : (b < 1 ? 1 : b));
}

inline size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

}  // namespace
}  // namespace helix_im2col
