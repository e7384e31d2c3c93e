// Vendor comparator behind the common C ABI: rocBLAS FP32 GEMM with the operand layouts of the FP32 template
// -- A stored K x M, B stored K x N, C[M x N], all row-major -- so the benchmark wrappers can print a vendor
// column next to the template's.
//
// Role in the reference: src_template/Ampere_FP32/cublas_f32.cu:28-43 (cublasGemmEx, FP32) and the cublasSgemm
// check inside sgemm.cu:468.
#include <hip/hip_runtime.h>
#include <rocblas/rocblas.h>
#include <stdint.h>
#include <stdio.h>

#include "helix_abi.h"

namespace tpl {

constexpr int kElemBytes = 4;

inline const char* info_json() {
    return "{\"family\": \"rocblas_f32\", \"arch\": \"gfx950\", \"vendor\": \"rocblas_sgemm\", "
           "\"layout_a\": \"K x M row-major f32\", \"layout_b\": \"K x N row-major f32\", "
           "\"layout_c\": \"M x N row-major f32\", \"accumulate\": \"f32\", \"k_multiple\": 1, \"ld_multiple\": 1}";
}

inline size_t workspace_bytes(int, int, int) { return 0; }
inline size_t conv_workspace_bytes(int, int, int, int, int, int, int, int, int) { return 0; }

inline void bench_layout(int M, int N, int K, size_t* ae, size_t* be, size_t* ce, int* lda, int* ldb, int* ldc) {
    *ae = (size_t)K * M; *be = (size_t)K * N; *ce = (size_t)M * N;
    *lda = M; *ldb = N; *ldc = N;
}

inline rocblas_handle handle() {
    static rocblas_handle h = nullptr;
    if (!h && rocblas_create_handle(&h) != rocblas_status_success) h = nullptr;
    return h;
}

inline int gemm(const void* A, const void* B, void* C, int M, int N, int K, int lda, int ldb, int ldc, void*, size_t,
                hipStream_t s) {
    if (lda < M || ldb < N || ldc < N) return HELIX_ERR_INVALID_VALUE;
    rocblas_handle h = handle();
    if (!h) return HELIX_ERR_UNSUPPORTED;
    if (rocblas_set_stream(h, s) != rocblas_status_success) return HELIX_ERR_INVALID_VALUE;
    const float alpha = 1.f, beta = 0.f;
    // column-major view: C^T (N x M, ld ldc) = (B as N x K, ld ldb) * op_T(A as M x K, ld lda)
    rocblas_status st = rocblas_sgemm(h, rocblas_operation_none, rocblas_operation_transpose, N, M, K, &alpha,
                                      (const float*)B, ldb, (const float*)A, lda, &beta, (float*)C, ldc);
    return st == rocblas_status_success ? 0 : 1000 + (int)st;
}

inline int conv2d(const void*, const void*, void*, int, int, int, int, int, int, int, int, int, void*, size_t,
                  hipStream_t) {
    return HELIX_ERR_UNSUPPORTED;
}

}  // namespace tpl

#define HELIX_NO_STATIC_SCRATCH   // the vendor library owns its workspace
#include "helix_host.h"
