// Explicit im2col for the convolution entry points of the MI355X kernel templates: the path taken when the
// input channel count is not a multiple of the 16-byte chunk the implicit-GEMM gather works in (first layers
// with IC = 1 or 3, odd channel counts), where the reference's own algorithm -- a column buffer followed by
// the GEMM (src_template/Ampere_FP16/im2col.cu:38-97, scripts/Ampere_FP16/Ampere_FP16_conv.py:431-446) --
// is used as is, on NHWC data:
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

namespace helix_im2col {

struct Geom {
    int H, W, IC, OH, OW, kW, stride, pad;
    int M, K;   // M = batch*OH*OW, K = kH*kW*IC
};

template <typename T>
__device__ __forceinline__ T tap(const T* x, const Geom& g, int m, int k) {
    if (m >= g.M || k >= g.K) return (T)0;
    const int ow = m % g.OW;
    const int t = m / g.OW;
    const int oh = t % g.OH;
    const int b = t / g.OH;
    const int c = k % g.IC;
    const int f = k / g.IC;
    const int ih = oh * g.stride - g.pad + f / g.kW;
    const int iw = ow * g.stride - g.pad + f % g.kW;
    if (ih < 0 || ih >= g.H || iw < 0 || iw >= g.W) return (T)0;
    return x[(((size_t)b * g.H + ih) * g.W + iw) * g.IC + c];
}

// K-contiguous column buffer: col[m*ldk + k], k < ldk (ldk a multiple of VEC); one thread writes VEC
// consecutive k of one row with a single store.
template <typename T, int VEC>
__global__ void im2col_rows_kernel(const T* x, T* col, Geom g, int ldk) {
    const int chunks = ldk / VEC;
    const size_t total = (size_t)g.M * chunks;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const int m = (int)(idx / chunks), k0 = (int)(idx % chunks) * VEC;
        T v[VEC];
#pragma unroll
        for (int j = 0; j < VEC; j++) v[j] = tap(x, g, m, k0 + j);
        T* dst = col + (size_t)m * ldk + k0;
#pragma unroll
        for (int j = 0; j < VEC; j++) dst[j] = v[j];
    }
}

// M-contiguous column buffer: col[k*ldm + m], m < ldm; consecutive threads write consecutive m.
template <typename T>
__global__ void im2col_cols_kernel(const T* x, T* col, Geom g, int ldm) {
    const size_t total = (size_t)g.K * ldm;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const int k = (int)(idx / ldm), m = (int)(idx % ldm);
        col[idx] = tap(x, g, m, k);
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

inline int grid_for(size_t total) {
    size_t b = (total + 255) / 256;
    return (int)(b > 65536 ? 65536 : (b < 1 ? 1 : b));
}

inline size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

}  // namespace helix_im2col
