// Host side shared by every MI355X kernel template: the extern "C" entry points of
// include/helix_abi.h, written once on top of a small per-template interface (namespace tpl).
//
// A template translation unit defines, before including this file:
//   namespace tpl {
//     constexpr int kElemBytes;                       // 2 (FP16) or 4 (FP32)
//     const char* info_json();
//     size_t workspace_bytes(int M, int N, int K);
//     size_t conv_workspace_bytes(int B, int H, int W, int IC, int OC, int kH, int kW, int stride, int pad);
//     int gemm(const void*, const void*, void*, int M, int N, int K, int lda, int ldb, int ldc,
//              void* ws, size_t ws_bytes, hipStream_t);
//     int conv2d(const void*, const void*, void*, int B, int H, int W, int IC, int OC, int kH, int kW,
//                int stride, int pad, void* ws, size_t ws_bytes, hipStream_t);
//     void bench_layout(int M, int N, int K, size_t* a_elems, size_t* b_elems, size_t* c_elems,
//                       int* lda, int* ldb, int* ldc);
//   }
//
// The timing entry points follow the reference's measurement loop (warm-up launches, then a group
// of launches between two events, src_template/Ampere_FP16/gemm.cu:636-652) but initialise their
// buffers, which the reference leaves as returned by cudaMalloc (gemm.cu:630-634).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#include <float.h>
#include <vector>

#include "helix_abi.h"

#define HELIX_HIP_TRY(expr)                      \
    do {                                         \
        hipError_t _e = (expr);                  \
        if (_e != hipSuccess) return (int)_e;    \
    } while (0)

namespace helix_host {
namespace {   // internal linkage: a library exports the helix_* entry points only

// Deterministic fill: value = scale * u, u in [-1, 1) from an integer hash of the element index.
__global__ void fill_f16_kernel(_Float16* p, size_t n, float scale, uint32_t seed) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        uint32_t h = (uint32_t)i * 2654435761u + seed;
        h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
        float u = (float)(h & 0xffffu) * (1.0f / 32768.0f) - 1.0f;
        p[i] = (_Float16)(u * scale);
    }
}

__global__ void fill_f32_kernel(float* p, size_t n, float scale, uint32_t seed) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        uint32_t h = (uint32_t)i * 2654435761u + seed;
        h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
        float u = (float)(h & 0xffffu) * (1.0f / 32768.0f) - 1.0f;
        p[i] = u * scale;
    }
}

inline int fill(void* p, size_t n_elems, int elem_bytes, float scale, uint32_t seed, hipStream_t s) {
    if (n_elems == 0) return 0;
    int blocks = (int)((n_elems + 255) / 256);
    if (blocks > 4096) blocks = 4096;
    if (elem_bytes == 2)
        hipLaunchKernelGGL(fill_f16_kernel, dim3(blocks), dim3(256), 0, s, (_Float16*)p, n_elems, scale, seed);
    else
        hipLaunchKernelGGL(fill_f32_kernel, dim3(blocks), dim3(256), 0, s, (float*)p, n_elems, scale, seed);
    return (int)hipGetLastError();
}

struct DeviceBuffers {
    std::vector<void*> ptrs;
    ~DeviceBuffers() {
        for (void* p : ptrs)
            if (p) (void)hipFree(p);
    }
    int alloc(void** out, size_t bytes) {
        *out = nullptr;
        if (bytes == 0) bytes = 256;
        hipError_t e = hipMalloc(out, bytes);
        if (e != hipSuccess) return (int)e;
        ptrs.push_back(*out);
        return 0;
    }
};

template <typename Launch>
int time_launches(Launch&& launch, hipStream_t s, int warmup, int iters, double* avg_s) {
    if (iters <= 0 || warmup < 0 || !avg_s) return HELIX_ERR_INVALID_VALUE;
    for (int i = 0; i < warmup; i++) {
        int rc = launch(i);
        if (rc) return rc;
    }
    hipEvent_t start, stop;
    HELIX_HIP_TRY(hipEventCreate(&start));
    hipError_t e = hipEventCreate(&stop);
    if (e != hipSuccess) { (void)hipEventDestroy(start); return (int)e; }
    int rc = 0;
    float ms = 0.f;
    e = hipEventRecord(start, s);
    if (e == hipSuccess) {
        for (int i = 0; i < iters && rc == 0; i++) rc = launch(warmup + i);
        if (rc == 0) e = hipEventRecord(stop, s);
        if (rc == 0 && e == hipSuccess) e = hipEventSynchronize(stop);
        if (rc == 0 && e == hipSuccess) e = hipEventElapsedTime(&ms, start, stop);
    }
    (void)hipEventDestroy(start);
    (void)hipEventDestroy(stop);
    if (rc) return rc;
    if (e != hipSuccess) return (int)e;
    *avg_s = (double)ms / 1000.0 / (double)iters;
    return 0;
}

}  // namespace
}  // namespace helix_host

extern "C" {

int helix_info(char* json, int cap) {
    const char* s = tpl::info_json();
    int need = (int)strlen(s) + 1;
    if (json && cap >= need) memcpy(json, s, (size_t)need);
    return need;
}

size_t helix_workspace_bytes(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    return tpl::workspace_bytes(M, N, K);
}

size_t helix_conv_workspace_bytes(int batch, int H, int W, int IC, int OC, int kH, int kW, int stride, int pad) {
    if (batch <= 0 || H <= 0 || W <= 0 || IC <= 0 || OC <= 0 || kH <= 0 || kW <= 0 || stride <= 0 || pad < 0) return 0;
    if (H + 2 * pad < kH || W + 2 * pad < kW) return 0;
    return tpl::conv_workspace_bytes(batch, H, W, IC, OC, kH, kW, stride, pad);
}

int helix_gemm(const void* A, const void* B, void* C, int M, int N, int K, int lda, int ldb, int ldc,
               void* workspace, size_t workspace_bytes, void* stream) {
    if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0) return HELIX_ERR_INVALID_VALUE;
    return tpl::gemm(A, B, C, M, N, K, lda, ldb, ldc, workspace, workspace_bytes, (hipStream_t)stream);
}

int helix_conv2d(const void* x, const void* w, void* y, int batch, int H, int W, int IC, int OC, int kH, int kW,
                 int stride, int pad, void* workspace, size_t workspace_bytes, void* stream) {
    if (!x || !w || !y || batch <= 0 || H <= 0 || W <= 0 || IC <= 0 || OC <= 0 || kH <= 0 || kW <= 0 ||
        stride <= 0 || pad < 0)
        return HELIX_ERR_INVALID_VALUE;
    if (H + 2 * pad < kH || W + 2 * pad < kW) return HELIX_ERR_INVALID_VALUE;
    return tpl::conv2d(x, w, y, batch, H, W, IC, OC, kH, kW, stride, pad, workspace, workspace_bytes,
                       (hipStream_t)stream);
}

#ifndef HELIX_NO_STATIC_SCRATCH
}  // extern "C"

// Scratch memory of helix_gemm_static_scratch: the K-partition partial sums live in this array instead of in
// a caller-provided workspace.  Every GPU the library runs on holds its own copy of the array, at its own
// address, until the process ends.  In host code the name is only a handle for HIP_SYMBOL(); the memory is
// reached through the per-device pointer below.
//
// HELIX_TPL_SCRATCH_BYTES (a template may define it before including this file) is the size this library gives the
// array: HELIX_STATIC_SCRATCH_BYTES unless the template never asks for a workspace (tpl::workspace_bytes is 0 for
// every shape), in which case a token array keeps the symbol and the entry point's code path the same.
#ifndef HELIX_TPL_SCRATCH_BYTES
#define HELIX_TPL_SCRATCH_BYTES HELIX_STATIC_SCRATCH_BYTES
#endif
static_assert(HELIX_TPL_SCRATCH_BYTES <= HELIX_STATIC_SCRATCH_BYTES, "the documented maximum bounds every library");
static __device__ __align__(256) unsigned char scratch[HELIX_TPL_SCRATCH_BYTES];

namespace helix_host {
namespace {

constexpr int kMaxDevices = 64;
void* scratch_ptr[kMaxDevices];   // device address of `scratch` per device ordinal, filled on first use

// Device address of `scratch` on the current device (looked up once per device, with that device current).
inline int static_scratch(void** out) {
    int d = -1;
    HELIX_HIP_TRY(hipGetDevice(&d));
    if (d < 0 || d >= kMaxDevices) return HELIX_ERR_INVALID_VALUE;
    void* p = __atomic_load_n(&scratch_ptr[d], __ATOMIC_ACQUIRE);
    if (!p) {
        HELIX_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return HELIX_ERR_INVALID_VALUE;
        __atomic_store_n(&scratch_ptr[d], p, __ATOMIC_RELEASE);   // racing first calls store the same address
    }
    *out = p;
    return 0;
}

}  // namespace
}  // namespace helix_host

extern "C" {

int helix_gemm_static_scratch(const void* A, const void* B, void* C, int M, int N, int K, int lda, int ldb, int ldc,
                              void* stream) {
    if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0) return HELIX_ERR_INVALID_VALUE;
    const size_t need = tpl::workspace_bytes(M, N, K);
    if (need > (size_t)HELIX_TPL_SCRATCH_BYTES) return HELIX_ERR_WORKSPACE;
    void* ws = nullptr;
    int rc = helix_host::static_scratch(&ws);
    if (rc) return rc;
    // Nothing to clear: a K-partitioned launch writes every partial sum of its M x N x partitions block before
    // its reduction pass reads that block, and reads nothing else of the array.
    return tpl::gemm(A, B, C, M, N, K, lda, ldb, ldc, ws, (size_t)HELIX_TPL_SCRATCH_BYTES, (hipStream_t)stream);
}
#else
int helix_gemm_static_scratch(const void*, const void*, void*, int, int, int, int, int, int, void*) {
    return HELIX_ERR_UNSUPPORTED;   // vendor comparator: the vendor library manages (and may allocate) its own workspace
}
#endif

int helix_gemm_timed(const void* A, const void* B, void* C, int M, int N, int K, int lda, int ldb, int ldc,
                     void* workspace, size_t workspace_bytes, void* stream, int warmup, int iters,
                     double* avg_s) {
    hipStream_t s = (hipStream_t)stream;
    auto launch = [&](int) { return helix_gemm(A, B, C, M, N, K, lda, ldb, ldc, workspace, workspace_bytes, stream); };
    return helix_host::time_launches(launch, s, warmup, iters, avg_s);
}

int helix_conv2d_timed(const void* x, const void* w, void* y, int batch, int H, int W, int IC, int OC, int kH,
                       int kW, int stride, int pad, void* workspace, size_t workspace_bytes, void* stream,
                       int warmup, int iters, double* avg_s) {
    hipStream_t s = (hipStream_t)stream;
    auto launch = [&](int) {
        return helix_conv2d(x, w, y, batch, H, W, IC, OC, kH, kW, stride, pad, workspace, workspace_bytes, stream);
    };
    return helix_host::time_launches(launch, s, warmup, iters, avg_s);
}

int helix_bench(int M, int N, int K, int warmup, int iters, int outer, size_t rotate_bytes, double* min_s,
                double* avg_s, double* max_s) {
    if (M <= 0 || N <= 0 || K <= 0 || iters <= 0 || outer <= 0 || warmup < 0) return HELIX_ERR_INVALID_VALUE;
    size_t ae, be, ce;
    int lda, ldb, ldc;
    tpl::bench_layout(M, N, K, &ae, &be, &ce, &lda, &ldb, &ldc);
    const int eb = tpl::kElemBytes;
    size_t nrot = 1;
    if (rotate_bytes > 0 && be * eb > 0) {
        nrot = (rotate_bytes + be * eb - 1) / (be * eb);
        if (nrot < 1) nrot = 1;
        if (nrot > 64) nrot = 64;
    }
    helix_host::DeviceBuffers bufs;
    void *A, *C, *ws;
    std::vector<void*> Bs(nrot);
    int rc;
    if ((rc = bufs.alloc(&A, ae * eb))) return rc;
    for (size_t r = 0; r < nrot; r++)
        if ((rc = bufs.alloc(&Bs[r], be * eb))) return rc;
    if ((rc = bufs.alloc(&C, ce * eb))) return rc;
    size_t wsb = tpl::workspace_bytes(M, N, K);
    if ((rc = bufs.alloc(&ws, wsb))) return rc;
    if ((rc = helix_host::fill(A, ae, eb, 0.5f, 1u, nullptr))) return rc;
    for (size_t r = 0; r < nrot; r++)
        if ((rc = helix_host::fill(Bs[r], be, eb, 0.5f, 2u + (uint32_t)r, nullptr))) return rc;
    if ((rc = helix_host::fill(C, ce, eb, 0.0f, 3u, nullptr))) return rc;
    HELIX_HIP_TRY(hipDeviceSynchronize());

    auto launch = [&](int i) {
        return tpl::gemm(A, Bs[(size_t)i % nrot], C, M, N, K, lda, ldb, ldc, ws, wsb, nullptr);
    };
    double mn = DBL_MAX, mx = 0.0, tot = 0.0;
    for (int o = 0; o < outer; o++) {
        double t;
        rc = helix_host::time_launches(launch, nullptr, o == 0 ? warmup : 0, iters, &t);
        if (rc) return rc;
        mn = t < mn ? t : mn;
        mx = t > mx ? t : mx;
        tot += t;
    }
    if (min_s) *min_s = mn;
    if (avg_s) *avg_s = tot / outer;
    if (max_s) *max_s = mx;
    return 0;
}

int helix_bench_conv(int batch, int IC, int H, int W, int OC, int kH, int kW, int stride, int pad, int warmup,
                     int iters, int outer, double* min_s, double* avg_s, double* max_s) {
    if (batch <= 0 || IC <= 0 || H <= 0 || W <= 0 || OC <= 0 || kH <= 0 || kW <= 0 || stride <= 0 || pad < 0 ||
        iters <= 0 || outer <= 0 || warmup < 0)
        return HELIX_ERR_INVALID_VALUE;
    if (H + 2 * pad < kH || W + 2 * pad < kW) return HELIX_ERR_INVALID_VALUE;
    int OH = (H + 2 * pad - kH) / stride + 1, OW = (W + 2 * pad - kW) / stride + 1;
    size_t xe = (size_t)batch * H * W * IC, we = (size_t)OC * kH * kW * IC, ye = (size_t)batch * OH * OW * OC;
    const int eb = tpl::kElemBytes;
    helix_host::DeviceBuffers bufs;
    void *x, *w, *y, *ws;
    int rc;
    if ((rc = bufs.alloc(&x, xe * eb))) return rc;
    if ((rc = bufs.alloc(&w, we * eb))) return rc;
    if ((rc = bufs.alloc(&y, ye * eb))) return rc;
    size_t wsb = tpl::conv_workspace_bytes(batch, H, W, IC, OC, kH, kW, stride, pad);
    if ((rc = bufs.alloc(&ws, wsb))) return rc;
    if ((rc = helix_host::fill(x, xe, eb, 0.5f, 1u, nullptr))) return rc;
    if ((rc = helix_host::fill(w, we, eb, 0.5f, 2u, nullptr))) return rc;
    if ((rc = helix_host::fill(y, ye, eb, 0.0f, 3u, nullptr))) return rc;
    HELIX_HIP_TRY(hipDeviceSynchronize());
    auto launch = [&](int) { return tpl::conv2d(x, w, y, batch, H, W, IC, OC, kH, kW, stride, pad, ws, wsb, nullptr); };
    double mn = DBL_MAX, mx = 0.0, tot = 0.0;
    for (int o = 0; o < outer; o++) {
        double t;
        rc = helix_host::time_launches(launch, nullptr, o == 0 ? warmup : 0, iters, &t);
        if (rc) return rc;
        mn = t < mn ? t : mn;
        mx = t > mx ? t : mx;
        tot += t;
    }
    if (min_s) *min_s = mn;
    if (avg_s) *avg_s = tot / outer;
    if (max_s) *max_s = mx;
    return 0;
}

}  // extern "C"
