// MI355X (gfx950 / CDNA4) FP32 GEMV / skinny-GEMM template: no MFMA, HBM-bound weight streaming.
//
//   C[M x N] = A[M x K] * B[N x K]^T,  M small, B = the weight matrix, streamed once.  FP32 throughout.
//
// Role in the reference: src_template/Ampere_FP32/gemv_template_fp32.cu:153-253 (the float twin of the
// FP16 GEMV; the reference never builds it, scripts/Ampere_FP32/build_Ampere_FP32.py:59-61).
//
// Same structure as the FP16 GEMV of this backend: one wave64 owns ROWS weight rows, its lanes are
// spread along K and load 16 bytes (4 floats) per row per 256-wide K step with the non-temporal hint;
// M_TILE x ROWS FP32 partial sums per lane are reduced across the wave with a transposing butterfly.
// SPLIT_K > 1 partitions K over blockIdx.z through an FP32 workspace and a fixed-order reduction.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "helix_abi.h"

#ifndef SPLIT_K
#define SPLIT_K 1
#endif
#ifndef WAVES_PER_BLOCK
#define WAVES_PER_BLOCK 4
#endif
#ifndef K_UNROLL
#define K_UNROLL 2
#endif

namespace {

typedef float elem_t;
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int SPLITK = SPLIT_K;
constexpr int WPB = WAVES_PER_BLOCK;
constexpr int VEC = 4;           // floats per 128-bit load
constexpr int KSTEP = 64 * VEC;  // floats covered by one wave-wide 128-bit load

struct Params {
    const elem_t* A;  // M x K activations
    const elem_t* B;  // N x K weights
    elem_t* C;        // M x N
    float* ws;        // SPLIT_K > 1: [SPLIT_K][M][N]
    int M, N, K, lda, ldb, ldc;
};

__device__ __forceinline__ float dot4(floatx4 a, floatx4 b, float acc) {
#pragma unroll
    for (int i = 0; i < 4; i++) acc = __builtin_fmaf(a[i], b[i], acc);
    return acc;
}

__device__ __forceinline__ floatx4 load_stream(const elem_t* p) {
    return __builtin_nontemporal_load((const floatx4*)p);
}

// Transposing wave reduction.  On entry every lane holds V partial values; on exit val[0..] holds
// complete sums of the value indices returned by reduced_index().
template <int V, int O>
struct Reduce {
    static __device__ __forceinline__ void run(float* val, int lane) {
        if constexpr (O >= 1) {
            if constexpr (V >= 2) {
                constexpr int H = V / 2;
                const bool up = (lane & O) != 0;
#pragma unroll
                for (int i = 0; i < H; i++) {
                    const float lo = val[i], hi = val[i + H];
                    const float send = up ? lo : hi;
                    const float keep = up ? hi : lo;
                    val[i] = keep + __shfl_xor(send, O, 64);
                }
                Reduce<H, O / 2>::run(val, lane);
            } else {
                val[0] += __shfl_xor(val[0], O, 64);
                Reduce<1, O / 2>::run(val, lane);
            }
        }
    }
    // index of the value that ends up in val[i] of this lane
    static __device__ __forceinline__ int index(int i, int lane) {
        if constexpr (O >= 1 && V >= 2) {
            constexpr int H = V / 2;
            return ((lane & O) ? H : 0) + Reduce<H, O / 2>::index(i, lane);
        } else {
            return i;
        }
    }
    // number of values left in val[] after the reduction
    static constexpr int remaining() {
        if constexpr (O >= 1 && V >= 2) return Reduce<V / 2, O / 2>::remaining();
        else return V;
    }
    // lanes sharing one value after the reduction form groups of this many lanes (1 if V >= 64)
    static constexpr int dup() {
        if constexpr (O >= 1) {
            if constexpr (V >= 2) return Reduce<V / 2, O / 2>::dup();
            else return 2 * Reduce<1, O / 2>::dup();
        } else return 1;
    }
};

template <int MT, int ROWS>
__global__ __launch_bounds__(64 * WPB) void helix_gemv_f32_kernel(const Params p) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n0 = (blockIdx.x * WPB + wave) * ROWS;
    const int m0 = blockIdx.y * MT;
    if (n0 >= p.N) return;

    int k_begin = 0, k_end = p.K;
    if (SPLITK > 1) {
        const int steps = (p.K + KSTEP - 1) / KSTEP;
        const int per = (steps + SPLITK - 1) / SPLITK;
        k_begin = (int)blockIdx.z * per * KSTEP;
        k_end = k_begin + per * KSTEP;
        if (k_end > p.K) k_end = p.K;
    }

    const elem_t* wrow[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        const int n = (n0 + r) < p.N ? (n0 + r) : (p.N - 1);  // clamp: duplicates are never stored
        wrow[r] = p.B + (size_t)n * p.ldb;
    }
    const elem_t* xrow[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) {
        const int mm = (m0 + m) < p.M ? (m0 + m) : (p.M - 1);
        xrow[m] = p.A + (size_t)mm * p.lda;
    }

    float acc[MT * ROWS];
#pragma unroll
    for (int v = 0; v < MT * ROWS; v++) acc[v] = 0.f;

    int k = k_begin + lane * VEC;
    // main loop: K_UNROLL independent 512-wide steps per trip keep K_UNROLL*ROWS loads in flight per lane
    for (; k + (K_UNROLL - 1) * KSTEP < k_end; k += K_UNROLL * KSTEP) {
        floatx4 w[K_UNROLL][ROWS];
#pragma unroll
        for (int u = 0; u < K_UNROLL; u++)
#pragma unroll
            for (int r = 0; r < ROWS; r++) w[u][r] = load_stream(wrow[r] + k + u * KSTEP);
#pragma unroll
        for (int u = 0; u < K_UNROLL; u++)
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const floatx4 xv = *(const floatx4*)(xrow[m] + k + u * KSTEP);
#pragma unroll
                for (int r = 0; r < ROWS; r++) acc[m * ROWS + r] = dot4(w[u][r], xv, acc[m * ROWS + r]);
            }
    }
    for (; k < k_end; k += KSTEP) {
        floatx4 w[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; r++) w[r] = load_stream(wrow[r] + k);
#pragma unroll
        for (int m = 0; m < MT; m++) {
            const floatx4 xv = *(const floatx4*)(xrow[m] + k);
#pragma unroll
            for (int r = 0; r < ROWS; r++) acc[m * ROWS + r] = dot4(w[r], xv, acc[m * ROWS + r]);
        }
    }

    constexpr int V = MT * ROWS;
    typedef Reduce<V, 32> Red;
    Red::run(acc, lane);
    constexpr int REM = Red::remaining();
    constexpr int DUP = Red::dup();
    if (DUP > 1 && (lane & (DUP - 1)) != 0) return;  // one writer per value
#pragma unroll
    for (int i = 0; i < REM; i++) {
        const int v = Red::index(i, lane);
        const int m = m0 + v / ROWS, n = n0 + v % ROWS;
        if (m < p.M && n < p.N) {
            if (SPLITK > 1)
                p.ws[((size_t)blockIdx.z * p.M + m) * p.N + n] = acc[i];
            else
                p.C[(size_t)m * p.ldc + n] = acc[i];
        }
    }
}

__global__ void helix_gemv_splitk_reduce_kernel(const float* ws, elem_t* C, int M, int N, int ldc, int splits) {
    const size_t total = (size_t)M * N;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        float s = 0.f;
        for (int k = 0; k < splits; k++) s += ws[(size_t)k * total + idx];
        C[(idx / N) * ldc + (idx % N)] = s;
    }
}

}  // namespace

#include <stdio.h>

namespace tpl {

constexpr int kElemBytes = 4;

inline const char* info_json() {
    static char buf[768];
    static bool done = false;
    if (!done) {
        snprintf(buf, sizeof(buf),
                 "{\"family\": \"gemv_f32\", \"arch\": \"gfx950\", \"mfma\": \"none\", \"lds_stages\": 0, "
                 "\"block_rows\": 1, \"block_cols\": 128, \"wave_rows\": 0, \"wave_cols\": 0, \"split_k\": %d, "
                 "\"threads\": %d, \"lds_bytes\": 0, \"k_step\": %d, "
                 "\"layout_a\": \"M x K row-major f32 (activations)\", "
                 "\"layout_b\": \"N x K row-major f32 (streamed weights)\", \"layout_c\": \"M x N row-major f32\", "
                 "\"accumulate\": \"f32\", \"k_multiple\": 4, \"ld_multiple\": 4}",
                 SPLITK, 64 * WPB, KSTEP);
        done = true;
    }
    return buf;
}

inline size_t workspace_bytes(int M, int N, int K) {
    (void)K;
    return SPLITK > 1 ? (size_t)SPLITK * (size_t)M * (size_t)N * sizeof(float) : 0;
}

inline void bench_layout(int M, int N, int K, size_t* ae, size_t* be, size_t* ce, int* lda, int* ldb, int* ldc) {
    *ae = (size_t)M * K; *be = (size_t)N * K; *ce = (size_t)M * N;
    *lda = K; *ldb = K; *ldc = N;
}

template <int MT, int ROWS>
inline int launch_cfg(const Params& p, hipStream_t s) {
    const int waves = (p.N + ROWS - 1) / ROWS;
    dim3 grid((waves + WPB - 1) / WPB, (p.M + MT - 1) / MT, SPLITK), block(64 * WPB);
    hipLaunchKernelGGL((helix_gemv_f32_kernel<MT, ROWS>), grid, block, 0, s, p);
    return (int)hipGetLastError();
}

// rows per wave: as many as keep >= ~8 waves per CU in flight, bounded by the accumulator budget
template <int MT>
inline int launch_mt(const Params& p, hipStream_t s) {
    constexpr int RMAX = (128 / MT) < 8 ? (128 / MT) : 8;
    const int want = p.N / 2048;
    if (RMAX >= 8 && want >= 8) return launch_cfg<MT, 8>(p, s);
    if (RMAX >= 4 && want >= 4) return launch_cfg<MT, 4>(p, s);
    if (RMAX >= 2 && want >= 2) return launch_cfg<MT, 2>(p, s);
    return launch_cfg<MT, 1>(p, s);
}

inline int gemm(const void* A, const void* B, void* C, int M, int N, int K, int lda, int ldb, int ldc, void* ws,
                size_t ws_bytes, hipStream_t s) {
    if (K % 4 != 0 || lda % 4 != 0 || ldb % 4 != 0) return HELIX_ERR_INVALID_VALUE;
    if (lda < K || ldb < K || ldc < N) return HELIX_ERR_INVALID_VALUE;
    if (((uintptr_t)A & 15) || ((uintptr_t)B & 15) || ((uintptr_t)C & 3)) return HELIX_ERR_INVALID_VALUE;
    if ((M + 15) / 16 > 65535) return HELIX_ERR_INVALID_VALUE;
    if (SPLITK > 1) {
        if (!ws || ws_bytes < workspace_bytes(M, N, K)) return HELIX_ERR_WORKSPACE;
    }
    Params p{(const elem_t*)A, (const elem_t*)B, (elem_t*)C, (float*)ws, M, N, K, lda, ldb, ldc};
    int rc;
    // activation-row tile, like the reference's N_TILE pick from the skinny extent
    // (gemv_template_fp32.cu:233-251)
    if (M <= 1) rc = launch_mt<1>(p, s);
    else if (M <= 2) rc = launch_mt<2>(p, s);
    else if (M <= 4) rc = launch_mt<4>(p, s);
    else if (M <= 8) rc = launch_mt<8>(p, s);
    else rc = launch_mt<16>(p, s);
    if (rc) return rc;
    if (SPLITK > 1) {
        size_t total = (size_t)M * N;
        int blocks = (int)((total + 255) / 256);
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL(helix_gemv_splitk_reduce_kernel, dim3(blocks), dim3(256), 0, s, (const float*)ws,
                           (elem_t*)C, M, N, ldc, SPLITK);
        return (int)hipGetLastError();
    }
    return 0;
}

inline int conv2d(const void*, const void*, void*, int, int, int, int, int, int, int, int, int, void*, size_t,
                  hipStream_t) {
    return HELIX_ERR_UNSUPPORTED;
}

}  // namespace tpl

#include "helix_host.h"
