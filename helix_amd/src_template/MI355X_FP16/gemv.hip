// MI355X (gfx950 / CDNA4) FP16 GEMV / skinny-GEMM template: no MFMA, HBM-bound weight streaming.
//
//   C[M x N] = A[M x K] * B[N x K]^T,  M small (decode batch), B = the weight matrix, streamed once.
//   FP16 in, FP32 accumulate (v_dot2_f32_f16), FP16 out.
//
// Role in the reference: src_template/Ampere_FP16/gemv.cu:152-252 (`mySGemvKernel_Stage4` and its
// N_TILE dispatch) and gemv_splitK.cu:153-260.  The reference names the streamed matrix A (Mbig x K)
// and the skinny one B (Nsmall x K) and swaps M and N on the host so that M >= N (gemv.cu:384-386);
// here the streamed matrix is always the B operand of the common GEMM signature and callers with a
// tall-skinny problem swap operands themselves (C^T = B * A^T).
//
// Kernel structure
//   * one wave64 owns ROWS weight rows; its 64 lanes are spread along K, each lane loading 16 bytes
//     (8 halves) per row per 512-wide K step, so every load instruction covers one contiguous
//     1 KiB segment of a weight row (fully coalesced 128-bit loads, streamed with the non-temporal
//     hint so weights do not evict the activations from cache).
//   * the M_TILE activation rows are re-read per K step (they stay resident in L1/L2: M_TILE*K*2 bytes).
//   * M_TILE x ROWS FP32 partial sums per lane; after the K loop they are reduced across the wave with a
//     transposing butterfly (each exchange halves the number of live values, ~2 instructions per
//     value instead of 12 for one butterfly per value), then written by the lanes that own them.
//   * SPLIT_K > 1 partitions K over blockIdx.z; partials go to an FP32 workspace and a second kernel
//     sums them in fixed order (deterministic; the reference uses half atomics, gemv_splitK.cu:213-217).
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

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef int intx4 __attribute__((ext_vector_type(4)));

constexpr int SPLITK = SPLIT_K;
constexpr int WPB = WAVES_PER_BLOCK;
constexpr int KSTEP = 64 * 8;  // halves covered by one wave-wide 128-bit load

struct Params {
    const half_t* A;  // M x K activations
    const half_t* B;  // N x K weights
    half_t* C;        // M x N
    float* ws;        // SPLIT_K > 1: [SPLIT_K][M][N]
    int M, N, K, lda, ldb, ldc;
};

__device__ __forceinline__ float dot8(half8 a, half8 b, float acc) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
        half2_t x = {a[2 * i], a[2 * i + 1]};
        half2_t y = {b[2 * i], b[2 * i + 1]};
        acc = __builtin_amdgcn_fdot2(x, y, acc, false);
    }
    return acc;
}

__device__ __forceinline__ half8 load_stream(const half_t* p) {
    return __builtin_bit_cast(half8, __builtin_nontemporal_load((const intx4*)p));
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
__global__ __launch_bounds__(64 * WPB) void helix_gemv_f16_kernel(const Params p) {
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

    const half_t* wrow[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        const int n = (n0 + r) < p.N ? (n0 + r) : (p.N - 1);  // clamp: duplicates are never stored
        wrow[r] = p.B + (size_t)n * p.ldb;
    }
    const half_t* xrow[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) {
        const int mm = (m0 + m) < p.M ? (m0 + m) : (p.M - 1);
        xrow[m] = p.A + (size_t)mm * p.lda;
    }

    float acc[MT * ROWS];
#pragma unroll
    for (int v = 0; v < MT * ROWS; v++) acc[v] = 0.f;

    int k = k_begin + lane * 8;
    // main loop: K_UNROLL independent 512-wide steps per trip keep K_UNROLL*ROWS loads in flight per lane
    for (; k + (K_UNROLL - 1) * KSTEP < k_end; k += K_UNROLL * KSTEP) {
        half8 w[K_UNROLL][ROWS];
#pragma unroll
        for (int u = 0; u < K_UNROLL; u++)
#pragma unroll
            for (int r = 0; r < ROWS; r++) w[u][r] = load_stream(wrow[r] + k + u * KSTEP);
#pragma unroll
        for (int u = 0; u < K_UNROLL; u++)
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const half8 xv = *(const half8*)(xrow[m] + k + u * KSTEP);
#pragma unroll
                for (int r = 0; r < ROWS; r++) acc[m * ROWS + r] = dot8(w[u][r], xv, acc[m * ROWS + r]);
            }
    }
    for (; k < k_end; k += KSTEP) {
        half8 w[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; r++) w[r] = load_stream(wrow[r] + k);
#pragma unroll
        for (int m = 0; m < MT; m++) {
            const half8 xv = *(const half8*)(xrow[m] + k);
#pragma unroll
            for (int r = 0; r < ROWS; r++) acc[m * ROWS + r] = dot8(w[r], xv, acc[m * ROWS + r]);
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
                p.C[(size_t)m * p.ldc + n] = (half_t)acc[i];
        }
    }
}

__global__ void helix_gemv_splitk_reduce_kernel(const float* ws, half_t* C, int M, int N, int ldc, int splits) {
    const size_t total = (size_t)M * N;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        float s = 0.f;
        for (int k = 0; k < splits; k++) s += ws[(size_t)k * total + idx];
        C[(idx / N) * ldc + (idx % N)] = (half_t)s;
    }
}

}  // namespace

#include <stdio.h>

namespace tpl {

constexpr int kElemBytes = 2;

inline const char* info_json() {
    static char buf[768];
    static bool done = false;
    if (!done) {
        snprintf(buf, sizeof(buf),
                 "{\"family\": \"gemv_f16\", \"arch\": \"gfx950\", \"mfma\": \"none\", \"lds_stages\": 0, "
                 "\"block_rows\": 1, \"block_cols\": 128, \"wave_rows\": 0, \"wave_cols\": 0, \"split_k\": %d, "
                 "\"threads\": %d, \"lds_bytes\": 0, \"k_step\": %d, "
                 "\"layout_a\": \"M x K row-major f16 (activations)\", "
                 "\"layout_b\": \"N x K row-major f16 (streamed weights)\", \"layout_c\": \"M x N row-major f16\", "
                 "\"accumulate\": \"f32\", \"k_multiple\": 8, \"ld_multiple\": 8}",
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
    hipLaunchKernelGGL((helix_gemv_f16_kernel<MT, ROWS>), grid, block, 0, s, p);
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
    if (K % 8 != 0 || lda % 8 != 0 || ldb % 8 != 0) return HELIX_ERR_INVALID_VALUE;
    if (lda < K || ldb < K || ldc < N) return HELIX_ERR_INVALID_VALUE;
    if (((uintptr_t)A & 15) || ((uintptr_t)B & 15) || ((uintptr_t)C & 1)) return HELIX_ERR_INVALID_VALUE;
    if ((M + 15) / 16 > 65535) return HELIX_ERR_INVALID_VALUE;
    if (SPLITK > 1) {
        if (!ws || ws_bytes < workspace_bytes(M, N, K)) return HELIX_ERR_WORKSPACE;
    }
    Params p{(const half_t*)A, (const half_t*)B, (half_t*)C, (float*)ws, M, N, K, lda, ldb, ldc};
    int rc;
    // activation-row tile, like the reference's N_TILE pick from the skinny extent (gemv.cu:232-250)
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
                           (half_t*)C, M, N, ldc, SPLITK);
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
