// Vendor comparator behind the common C ABI: rocBLAS FP16 GEMM (FP32 compute), same operand layouts as the
// FP16 template -- C[M x N] = A[M x K] * B[N x K]^T, row-major -- so the benchmark wrappers can print a vendor
// column next to the template's.
//
// Role in the reference: src_template/Ampere_FP16/cublas_f16.cu:28-44 (cublasGemmEx on row-major operands
// through the column-major identity C^T = B^T A^T) and its timing main (:46-105).  Differences: FP32 compute
// type (the reference asks for CUBLAS_COMPUTE_16F, :55), and the library exports helix_bench instead of
// printing a line.
#include <hip/hip_runtime.h>
#include <rocblas/rocblas.h>
#include <stdint.h>
#include <stdio.h>

#include "helix_abi.h"

namespace tpl {

constexpr int kElemBytes = 2;

inline const char* info_json() {
    return "{\"family\": \"rocblas_f16\", \"arch\": \"gfx950\", \"vendor\": \"rocblas_gemm_ex, f16 in / f32 compute / f16 out\", "
           "\"layout_a\": \"M x K row-major f16\", \"layout_b\": \"N x K row-major f16\", "
           "\"layout_c\": \"M x N row-major f16\", \"accumulate\": \"f32\", \"k_multiple\": 1, \"ld_multiple\": 1}";
}

inline size_t workspace_bytes(int, int, int) { return 0; }
inline size_t conv_workspace_bytes(int, int, int, int, int, int, int, int, int) { return 0; }

inline void bench_layout(int M, int N, int K, size_t* ae, size_t* be, size_t* ce, int* lda, int* ldb, int* ldc) {
    *ae = (size_t)M * K; *be = (size_t)N * K; *ce = (size_t)M * N;
    *lda = K; *ldb = K; *ldc = N;
}

inline rocblas_handle handle() {
    static rocblas_handle h = nullptr;
    if (!h && rocblas_create_handle(&h) != rocblas_status_success) h = nullptr;
    return h;
}

inline int gemm(const void* A, const void* B, void* C, int M, int N, int K, int lda, int ldb, int ldc, void*, size_t,
                hipStream_t s) {
    if (lda < K || ldb < K || ldc < N) return HELIX_ERR_INVALID_VALUE;
    rocblas_handle h = handle();
    if (!h) return HELIX_ERR_UNSUPPORTED;
    if (rocblas_set_stream(h, s) != rocblas_status_success) return HELIX_ERR_INVALID_VALUE;
    const float alpha = 1.f, beta = 0.f;
    // column-major view: C^T (N x M, ld ldc) = op_T(B as K x N, ld ldb) * (A as K x M, ld lda)
    rocblas_status st = rocblas_gemm_ex(h, rocblas_operation_transpose, rocblas_operation_none, N, M, K, &alpha, B,
                                        rocblas_datatype_f16_r, ldb, A, rocblas_datatype_f16_r, lda, &beta, C,
                                        rocblas_datatype_f16_r, ldc, C, rocblas_datatype_f16_r, ldc,
                                        rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0);
    return st == rocblas_status_success ? 0 : 1000 + (int)st;
}

inline int conv2d(const void*, const void*, void*, int, int, int, int, int, int, int, int, int, void*, size_t,
                  hipStream_t) {
    return HELIX_ERR_UNSUPPORTED;
}

}  // namespace tpl

#define HELIX_NO_STATIC_SCRATCH   // the vendor library owns its workspace
#include "helix_host.h"
