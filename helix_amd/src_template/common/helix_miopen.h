// Vendor comparator behind the common C ABI: MIOpen forward convolution on the templates' own layouts --
// NHWC activations, [OC][kH][kW][IC] weights, NHWC output -- so the benchmark wrappers can print a vendor column
// next to the template's.  Included by MI355X_FP16/miopen_f16.hip and MI355X_FP32/miopen_f32.hip after they
// define MIOPEN_ELEM_TYPE (miopenHalf / miopenFloat) and MIOPEN_ELEM_BYTES.
//
// Role in the reference: src_template/Ampere_FP16/cudnn_fp16.cu:109-380 and Ampere_FP32/cudnn_fp32.cu -- tensor,
// filter and convolution descriptors (:227-281), cudnnFindConvolutionForwardAlgorithm (:283), workspace, timed
// cudnnConvolutionForward launches (:339-372).  Differences: the library keeps one plan per problem (descriptors,
// the algorithm MIOpen's own search found fastest, workspace size) and exports helix_conv2d / helix_bench_conv
// instead of printing a line.
#pragma once

#include <hip/hip_runtime.h>
#include <miopen/miopen.h>
#include <stdint.h>
#include <stdio.h>

#include <array>
#include <map>
#include <mutex>

#include "helix_abi.h"

namespace tpl {

constexpr int kElemBytes = MIOPEN_ELEM_BYTES;

inline const char* info_json() {
    return "{\"family\": \"miopen\", \"arch\": \"gfx950\", \"vendor\": \"miopenConvolutionForward, algorithm from "
           "miopenFindConvolutionForwardAlgorithm\", \"layout_a\": \"NHWC\", \"layout_b\": \"[OC][kH][kW][IC]\", "
           "\"layout_c\": \"NHWC\", \"k_multiple\": 1, \"ld_multiple\": 1}";
}

inline size_t workspace_bytes(int, int, int) { return 0; }

inline void bench_layout(int M, int N, int K, size_t* ae, size_t* be, size_t* ce, int* lda, int* ldb, int* ldc) {
    *ae = (size_t)M * K; *be = (size_t)N * K; *ce = (size_t)M * N;
    *lda = K; *ldb = K; *ldc = N;
}

inline int gemm(const void*, const void*, void*, int, int, int, int, int, int, void*, size_t, hipStream_t) {
    return HELIX_ERR_UNSUPPORTED;
}

struct Plan {
    miopenTensorDescriptor_t x = nullptr, w = nullptr, y = nullptr;
    miopenConvolutionDescriptor_t conv = nullptr;
    miopenConvFwdAlgorithm_t algo = miopenConvolutionFwdAlgoGEMM;
    size_t ws_bytes = 0;   // workspace the search was given and the chosen algorithm may use
    bool searched = false;
    int status = 0;        // non-zero: the problem could not be described to MIOpen
};

inline miopenHandle_t handle() {
    static miopenHandle_t h = nullptr;
    if (!h && miopenCreate(&h) != miopenStatusSuccess) h = nullptr;
    return h;
}

inline std::mutex& plan_mutex() {
    static std::mutex m;
    return m;
}

// Descriptors and workspace size of one problem (no GPU work); the algorithm search happens at the first run.
inline Plan& plan_for(int batch, int H, int W, int IC, int OC, int kH, int kW, int stride, int pad) {
    static std::map<std::array<int, 9>, Plan> plans;
    const std::array<int, 9> key{batch, H, W, IC, OC, kH, kW, stride, pad};
    auto it = plans.find(key);
    if (it != plans.end()) return it->second;
    Plan& p = plans[key];
    miopenHandle_t h = handle();
    if (!h) { p.status = HELIX_ERR_UNSUPPORTED; return p; }
    const int OH = (H + 2 * pad - kH) / stride + 1, OW = (W + 2 * pad - kW) / stride + 1;
    // lens are always given in N, C, H, W order; the layout argument says how they lie in memory
    const int xl[4] = {batch, IC, H, W}, wl[4] = {OC, IC, kH, kW}, yl[4] = {batch, OC, OH, OW};
    bool ok = miopenCreateTensorDescriptor(&p.x) == miopenStatusSuccess &&
              miopenCreateTensorDescriptor(&p.w) == miopenStatusSuccess &&
              miopenCreateTensorDescriptor(&p.y) == miopenStatusSuccess &&
              miopenCreateConvolutionDescriptor(&p.conv) == miopenStatusSuccess;
    ok = ok && miopenSetNdTensorDescriptorWithLayout(p.x, MIOPEN_ELEM_TYPE, miopenTensorNHWC, xl, 4) == miopenStatusSuccess;
    ok = ok && miopenSetNdTensorDescriptorWithLayout(p.w, MIOPEN_ELEM_TYPE, miopenTensorNHWC, wl, 4) == miopenStatusSuccess;
    ok = ok && miopenSetNdTensorDescriptorWithLayout(p.y, MIOPEN_ELEM_TYPE, miopenTensorNHWC, yl, 4) == miopenStatusSuccess;
    ok = ok && miopenInitConvolutionDescriptor(p.conv, miopenConvolution, pad, pad, stride, stride, 1, 1) == miopenStatusSuccess;
    ok = ok && miopenConvolutionForwardGetWorkSpaceSize(h, p.w, p.x, p.conv, p.y, &p.ws_bytes) == miopenStatusSuccess;
    if (!ok) p.status = HELIX_ERR_INVALID_VALUE;
    return p;
}

inline size_t conv_workspace_bytes(int batch, int H, int W, int IC, int OC, int kH, int kW, int stride, int pad) {
    std::lock_guard<std::mutex> lock(plan_mutex());
    const Plan& p = plan_for(batch, H, W, IC, OC, kH, kW, stride, pad);
    return p.status ? 0 : p.ws_bytes;
}

inline int conv2d(const void* x, const void* w, void* y, int batch, int H, int W, int IC, int OC, int kH, int kW,
                  int stride, int pad, void* ws, size_t ws_bytes, hipStream_t s) {
    std::lock_guard<std::mutex> lock(plan_mutex());
    Plan& p = plan_for(batch, H, W, IC, OC, kH, kW, stride, pad);
    if (p.status) return p.status;
    if (p.ws_bytes > 0 && (!ws || ws_bytes < p.ws_bytes)) return HELIX_ERR_WORKSPACE;
    miopenHandle_t h = handle();
    if (miopenSetStream(h, s) != miopenStatusSuccess) return HELIX_ERR_INVALID_VALUE;
    if (!p.searched) {
        // MIOpen times its applicable algorithms on these very buffers (y is overwritten) and returns them
        // fastest first
        miopenConvAlgoPerf_t perf[4];
        int found = 0;
        miopenStatus_t st = miopenFindConvolutionForwardAlgorithm(h, p.x, x, p.w, w, p.conv, p.y, y, 4, &found, perf, ws,
                                                                  p.ws_bytes, false);
        if (st != miopenStatusSuccess || found < 1) return 1000 + (int)st;
        p.algo = perf[0].fwd_algo;
        p.searched = true;
    }
    const float alpha = 1.f, beta = 0.f;
    miopenStatus_t st = miopenConvolutionForward(h, &alpha, p.x, x, p.w, w, p.conv, p.algo, &beta, p.y, y, ws, p.ws_bytes);
    return st == miopenStatusSuccess ? 0 : 1000 + (int)st;
}

}  // namespace tpl

#define HELIX_NO_STATIC_SCRATCH   // the vendor library owns its workspace
#include "helix_host.h"
