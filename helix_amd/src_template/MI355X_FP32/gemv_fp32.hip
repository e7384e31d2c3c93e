// MI355X (gfx950 / CDNA4) FP32 GEMV / skinny-GEMM template: no MFMA, HBM-bound weight streaming.
//
//   C[M x N] = A[M x K] * B[N x K]^T,  M small, B = the weight matrix, streamed once.  FP32 throughout.
//
// Role in the reference: src_template/Ampere_FP32/gemv_template_fp32.cu:153-253 (the float twin of the
// FP16 GEMV; the reference never builds it, scripts/Ampere_FP32/build_Ampere_FP32.py:59-61).
//
// Same structure as the FP16 GEMV of this backend: a workgroup stages its M_TILE activation rows for
// its K range in LDS; each wave walks its own run of consecutive weight rows, ROWS at a time, with the
// 64 lanes spread along K (16 bytes = 4 floats per lane per 256-wide step, non-temporal loads, double
// buffered); M_TILE x ROWS FP32 partial sums per lane are reduced across the wave with a transposing
// butterfly.  K is partitioned over blockIdx.z (FP32 workspace + fixed-order reduction kernel) when the
// staged activations would exceed the LDS budget or SPLIT_K asks for it.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "helix_abi.h"

#ifndef SPLIT_K
#define SPLIT_K 1
#endif
#ifndef WAVES_PER_BLOCK
#define WAVES_PER_BLOCK 4
#endif
// (weight rows per pass, 512-wide K steps in flight) per activation-row tile
#ifndef GEMV_R1
#define GEMV_R1 1
#define GEMV_KU1 8
#endif
#ifndef GEMV_R2
#define GEMV_R2 1
#define GEMV_KU2 8
#endif
#ifndef GEMV_R4
#define GEMV_R4 1
#define GEMV_KU4 4
#endif
#ifndef GEMV_R4_WIDE
#define GEMV_R4_WIDE 2
#define GEMV_KU4_WIDE 4
#endif
#ifndef GEMV_R8
#define GEMV_R8 4
#define GEMV_KU8 2
#endif
#ifndef GEMV_R16
#define GEMV_R16 4
#define GEMV_KU16 1
#endif
#ifndef X_LDS_BYTES
#define X_LDS_BYTES 65536   // staged activations of one workgroup of WAVES_PER_BLOCK waves (two workgroups share a CU)
#endif
#ifndef X_LDS_BYTES_WIDE
#define X_LDS_BYTES_WIDE 131072   // ... of one workgroup of twice as many waves, alone on its CU: same waves per CU
#endif
#ifndef GEMV_MANY_WAVES_MT
#define GEMV_MANY_WAVES_MT 4   // activation-row tiles up to this one run 16 waves per compute unit instead of 8
#endif
#ifndef TARGET_WAVES
#define TARGET_WAVES 2048   // waves a launch aims for: 256 compute units x 8
#endif

namespace {

typedef float elem_t;
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef int intx4 __attribute__((ext_vector_type(4)));

constexpr int SPLITK = SPLIT_K;
constexpr int WPB = WAVES_PER_BLOCK;
constexpr int VEC = 4;           // floats per 128-bit load
constexpr int KSTEP = 64 * VEC;  // floats covered by one wave-wide 128-bit load

struct Params {
    const elem_t* A;  // M x K activations
    const elem_t* B;  // N x K weights
    elem_t* C;        // M x N
    float* ws;        // ksplit > 1: [ksplit][M][N] FP32 partial sums
    int M, N, K, lda, ldb, ldc;
    int kchunk;         // K range of one workgroup (multiple of KSTEP)
    int ksplit;         // number of K ranges (grid.z)
    int rows_per_wave;  // consecutive weight rows owned by one wave
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

// WAVES: waves per workgroup.  WAVES_PER_BLOCK when the staged activations leave room for two workgroups per
// CU, twice that when they need more than half of the LDS, so that a long K costs neither occupancy nor a
// K partition with its second kernel.
template <int MT, int ROWS, int KU, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void helix_gemv_f32_kernel(const Params p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    elem_t* xs = (elem_t*)smem;                      // [MT][kchunk] activations of this K range

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int m0 = blockIdx.y * MT;
    const int kchunk = p.kchunk;                     // multiple of KSTEP
    const int k_begin = (int)blockIdx.z * kchunk;
    const int k_end = (k_begin + kchunk) < p.K ? (k_begin + kchunk) : p.K;
    constexpr int TRIP = KU * KSTEP;                 // K extent of one trip: KU*ROWS loads per lane

    // ---- this wave's run of weight rows -----------------------------------------------------------------
    const int row_first = (blockIdx.x * WAVES + wave) * p.rows_per_wave;
    const int row_last = (row_first + p.rows_per_wave) < p.N ? (row_first + p.rows_per_wave) : p.N;

    const elem_t* wrow[ROWS];
    auto set_rows = [&](int n0) {
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            const int n = (n0 + r) < p.N ? (n0 + r) : (p.N - 1);   // clamp: duplicates are never stored
            wrow[r] = p.B + (size_t)n * p.ldb + lane * VEC;
        }
    };
    auto load_trip = [&](floatx4 (&w)[KU][ROWS], int kk) {
#pragma unroll
        for (int u = 0; u < KU; u++)
#pragma unroll
            for (int r = 0; r < ROWS; r++) w[u][r] = load_stream(wrow[r] + kk + u * KSTEP);
    };

    // The first trip of the first row group is requested before the activations are staged, and the
    // first trip of every later group before the previous group is reduced: the weight stream never
    // waits for anything but HBM.
    floatx4 wa[KU][ROWS], wb[KU][ROWS];
    const bool has_trip = (k_begin + TRIP <= k_end);
    if (row_first < row_last) {
        set_rows(row_first);
        if (has_trip) load_trip(wa, k_begin);
    }

    // ---- stage the activations: 16-byte chunks, zero beyond M and beyond K ----------------------------
    {
        const int chunks_per_row = kchunk / VEC;
        const int total = MT * chunks_per_row;
        for (int c = tid; c < total; c += 64 * WAVES) {
            const int m = c / chunks_per_row, kc = (c % chunks_per_row) * VEC;
            intx4 v = {0, 0, 0, 0};
            if (m0 + m < p.M && k_begin + kc < k_end) v = *(const intx4*)(p.A + (size_t)(m0 + m) * p.lda + k_begin + kc);
            *(intx4*)(xs + (size_t)m * kchunk + kc) = v;
        }
    }
    __syncthreads();

    const elem_t* xl = xs + lane * VEC;                // this lane's 4 floats of every 256-wide step
    float acc[MT * ROWS];
    auto dot_trip = [&](const floatx4 (&w)[KU][ROWS], int kk) {
#pragma unroll
        for (int u = 0; u < KU; u++)
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const floatx4 xv = *(const floatx4*)(xl + (size_t)m * kchunk + (kk - k_begin) + u * KSTEP);
#pragma unroll
                for (int r = 0; r < ROWS; r++) acc[m * ROWS + r] = dot4(w[u][r], xv, acc[m * ROWS + r]);
            }
    };

    for (int n0 = row_first; n0 < row_last; n0 += ROWS) {
#pragma unroll
        for (int v = 0; v < MT * ROWS; v++) acc[v] = 0.f;

        int k = k_begin;                              // wave-uniform; lane offset is in the pointers
        // double-buffered trips: the loads of trip t+1 are issued before the dot products of trip t
        if (has_trip) {
            for (; k + 3 * TRIP <= k_end; k += 2 * TRIP) {
                load_trip(wb, k + TRIP);
                dot_trip(wa, k);
                load_trip(wa, k + 2 * TRIP);
                dot_trip(wb, k + TRIP);
            }
            if (k + 2 * TRIP <= k_end) {
                load_trip(wb, k + TRIP);
                dot_trip(wa, k);
                dot_trip(wb, k + TRIP);
                k += 2 * TRIP;
            } else {
                dot_trip(wa, k);
                k += TRIP;
            }
        }
        // remainder (fewer than KU steps; the last one may be partial): all loads first, lanes beyond K
        // contribute zeros, then the dot products
        if (k < k_end) {
#pragma unroll
            for (int u = 0; u < KU; u++) {
                const int kk = k + u * KSTEP;
                const bool live = kk + lane * VEC < k_end;
#pragma unroll
                for (int r = 0; r < ROWS; r++) {
                    floatx4 z = {0.f, 0.f, 0.f, 0.f};
                    wb[u][r] = live ? load_stream(wrow[r] + kk) : z;
                }
            }
#pragma unroll
            for (int u = 0; u < KU; u++) {
                const int kk = k + u * KSTEP;
                if (kk < k_end) {   // wave-uniform: steps past the K range have no staged activations
#pragma unroll
                    for (int m = 0; m < MT; m++) {
                        const floatx4 xv = *(const floatx4*)(xl + (size_t)m * kchunk + (kk - k_begin));
#pragma unroll
                        for (int r = 0; r < ROWS; r++) acc[m * ROWS + r] = dot4(wb[u][r], xv, acc[m * ROWS + r]);
                    }
                }
            }
        }

        // request the next group's first trip, then reduce and store this group underneath it
        if (n0 + ROWS < row_last) {
            set_rows(n0 + ROWS);
            if (has_trip) load_trip(wa, k_begin);
        }

        constexpr int V = MT * ROWS;
        typedef Reduce<V, 32> Red;
        Red::run(acc, lane);
        constexpr int REM = Red::remaining();
        constexpr int DUP = Red::dup();
        if (DUP == 1 || (lane & (DUP - 1)) == 0) {   // one writer per value
#pragma unroll
            for (int i = 0; i < REM; i++) {
                const int v = Red::index(i, lane);
                const int m = m0 + v / ROWS, n = n0 + v % ROWS;
                if (m < p.M && n < row_last) {
                    if (p.ksplit > 1)
                        p.ws[((size_t)blockIdx.z * p.M + m) * p.N + n] = acc[i];
                    else
                        p.C[(size_t)m * p.ldc + n] = acc[i];
                }
            }
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
                 "\"threads\": %d, \"lds_bytes\": %d, \"k_step\": %d, "
                 "\"layout_a\": \"M x K row-major f32 (activations)\", "
                 "\"layout_b\": \"N x K row-major f32 (streamed weights)\", \"layout_c\": \"M x N row-major f32\", "
                 "\"accumulate\": \"f32\", \"k_multiple\": 4, \"ld_multiple\": 4}",
                 SPLITK, 64 * WPB, X_LDS_BYTES, KSTEP);
        done = true;
    }
    return buf;
}

constexpr int mtile_of(int M) { return M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : M <= 8 ? 8 : 16; }

// K partitioning: enough ranges that M_TILE activation rows of one range fit X_LDS_BYTES_WIDE, at least SPLIT_K
inline void k_partition(int M, int K, int* kchunk, int* ksplit) {
    const int mt = mtile_of(M);
    const int steps = (K + KSTEP - 1) / KSTEP;
    int max_steps = X_LDS_BYTES_WIDE / (mt * KSTEP * 4);
    if (max_steps < 1) max_steps = 1;
    int split = (steps + max_steps - 1) / max_steps;
    if (split < SPLITK) split = SPLITK;
    if (split > steps) split = steps;
    const int per = (steps + split - 1) / split;
    *kchunk = per * KSTEP;
    *ksplit = (steps + per - 1) / per;
}

inline size_t workspace_bytes(int M, int N, int K) {
    int kchunk, ksplit;
    k_partition(M, K, &kchunk, &ksplit);
    return ksplit > 1 ? (size_t)ksplit * (size_t)M * (size_t)N * sizeof(float) : 0;
}

inline void bench_layout(int M, int N, int K, size_t* ae, size_t* be, size_t* ce, int* lda, int* ldb, int* ldc) {
    *ae = (size_t)M * K; *be = (size_t)N * K; *ce = (size_t)M * N;
    *lda = K; *ldb = K; *ldc = N;
}

template <int MT, int ROWS, int KU, int WAVES>
inline int launch_waves(Params p, int lds, hipStream_t s) {
    const int waves = (p.N + p.rows_per_wave - 1) / p.rows_per_wave;
    static int attr_rc = (int)hipFuncSetAttribute((const void*)helix_gemv_f32_kernel<MT, ROWS, KU, WAVES>,
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (attr_rc) return attr_rc;
    dim3 grid((waves + WAVES - 1) / WAVES, (p.M + MT - 1) / MT, p.ksplit), block(64 * WAVES);
    hipLaunchKernelGGL((helix_gemv_f32_kernel<MT, ROWS, KU, WAVES>), grid, block, lds, s, p);
    return (int)hipGetLastError();
}

template <int MT, int ROWS, int KU>
inline int launch_cfg(Params p, hipStream_t s) {
    // Up to four activation rows leave the vector units idle most of the time: twice the waves per CU, in workgroups
    // of twice the size so that the activations are staged as often as before (measured 2 - 13 % on the decode shapes;
    // slower with the eight-row tile).
    const int lds = MT * p.kchunk * 4;
    const bool many = (MT <= GEMV_MANY_WAVES_MT) && lds <= X_LDS_BYTES;
    const long long target = many ? 2 * TARGET_WAVES : TARGET_WAVES;
    // consecutive rows per wave: a multiple of ROWS that brings the launch near the target number of waves
    long long want = ((long long)p.N * p.ksplit + target - 1) / target;
    if (want < 1) want = 1;
    p.rows_per_wave = (int)((want + ROWS - 1) / ROWS) * ROWS;
    if (many || lds > X_LDS_BYTES) return launch_waves<MT, ROWS, KU, 2 * WPB>(p, lds, s);
    return launch_waves<MT, ROWS, KU, WPB>(p, lds, s);
}

inline int gemm(const void* A, const void* B, void* C, int M, int N, int K, int lda, int ldb, int ldc, void* ws,
                size_t ws_bytes, hipStream_t s) {
    if (K % 4 != 0 || lda % 4 != 0 || ldb % 4 != 0) return HELIX_ERR_INVALID_VALUE;
    if (lda < K || ldb < K || ldc < N) return HELIX_ERR_INVALID_VALUE;
    if (((uintptr_t)A & 15) || ((uintptr_t)B & 15) || ((uintptr_t)C & 3)) return HELIX_ERR_INVALID_VALUE;
    if ((M + 15) / 16 > 65535) return HELIX_ERR_INVALID_VALUE;
    Params p{(const elem_t*)A, (const elem_t*)B, (elem_t*)C, (float*)ws, M, N, K, lda, ldb, ldc, 0, 1, 1};
    k_partition(M, K, &p.kchunk, &p.ksplit);
    if (p.ksplit > 65535) return HELIX_ERR_INVALID_VALUE;
    if (p.ksplit > 1) {
        if (!ws || ws_bytes < workspace_bytes(M, N, K)) return HELIX_ERR_WORKSPACE;
    }
    int rc;
    // activation-row tile, like the reference's N_TILE pick from the skinny extent (gemv_template_fp32.cu:233-251); wider
    // tiles take more weight rows per pass so that one LDS read of the activations feeds several rows
    switch (mtile_of(M)) {
        case 1: rc = launch_cfg<1, GEMV_R1, GEMV_KU1>(p, s); break;
        case 2: rc = launch_cfg<2, GEMV_R2, GEMV_KU2>(p, s); break;
        case 4:
            // four rows: one weight row per pass while the staged activations leave room for 16 waves per CU
            // (3 - 13 % faster there), two rows per pass when they fill the LDS and 8 waves share them
            if (4 * p.kchunk * 4 <= X_LDS_BYTES) rc = launch_cfg<4, GEMV_R4, GEMV_KU4>(p, s);
            else rc = launch_cfg<4, GEMV_R4_WIDE, GEMV_KU4_WIDE>(p, s);
            break;
        case 8: rc = launch_cfg<8, GEMV_R8, GEMV_KU8>(p, s); break;
        default: rc = launch_cfg<16, GEMV_R16, GEMV_KU16>(p, s); break;
    }
    if (rc) return rc;
    if (p.ksplit > 1) {
        size_t total = (size_t)M * N;
        int blocks = (int)((total + 255) / 256);
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL(helix_gemv_splitk_reduce_kernel, dim3(blocks), dim3(256), 0, s, (const float*)ws,
                           (elem_t*)C, M, N, ldc, p.ksplit);
        return (int)hipGetLastError();
    }
    return 0;
}

inline size_t conv_workspace_bytes(int, int, int, int, int, int, int, int, int) { return 0; }

inline int conv2d(const void*, const void*, void*, int, int, int, int, int, int, int, int, int, void*, size_t,
                  hipStream_t) {
    return HELIX_ERR_UNSUPPORTED;
}

}  // namespace tpl

#include "helix_host.h"
