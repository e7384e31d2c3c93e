// Parts shared by the FP16 MFMA tile templates of this directory (gemm.hip: copies staged through registers,
// GEMM and implicit-GEMM convolution; gemm_dtl.hip: direct-to-LDS copies, GEMM only): the compile-time tile
// parameters, the launch parameters, the workgroup -> output tile mapping, the epilogue, the split-K reduction
// and the host-side K-partition rule.
//
// Compile-time parameters (set with -D by the build script, one shared library per combination):
//   BLOCK_ROWS x BLOCK_COLS   workgroup tile of C           (reference BLOCK_ROWS / BLOCK_COLS,
//                                                            scripts/Ampere_FP16/build_Ampere_FP16.py:47-53)
//   WAVE_ROWS  x WAVE_COLS    tile of C owned by one wave64 (reference WARP_ROWS / WARP_COLS)
//   BLOCK_K                   K extent of one LDS stage
//   K_STAGES                  depth of the K pipeline       (reference K_STAGE)
//   SPLIT_K                   1: each workgroup walks all of K.  > 1: K is partitioned into 2 .. SPLIT_K ranges, as
//                             many as it takes to give every compute unit a workgroup; the FP32 partial sums go
//                             to the workspace and are added in partition order, by the last workgroup of a tile
//                             to finish (all partitions of a tile run on one XCD and meet in its L2) or, where
//                             that is not available, by a second kernel
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#ifndef SPLIT_K
#define SPLIT_K 1
#endif
#define HELIX_SPLITK_ENABLED (SPLIT_K > 1)

#include "helix_abi.h"
#include "helix_fastdiv.h"
#include "helix_splitk.h"

#ifndef BLOCK_ROWS
#define BLOCK_ROWS 256
#endif
#ifndef BLOCK_COLS
#define BLOCK_COLS 256
#endif
#ifndef WAVE_ROWS
#define WAVE_ROWS 128
#endif
#ifndef WAVE_COLS
#define WAVE_COLS 128
#endif
#ifndef BLOCK_K
#define BLOCK_K 64
#endif
#ifndef K_STAGES
#define K_STAGES 2
#endif
#ifndef SPLIT_K
#define SPLIT_K 1
#endif
#ifndef GROUP_ROWS
#define GROUP_ROWS 4
#endif

namespace {

typedef _Float16 half_t;
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef int intx4 __attribute__((ext_vector_type(4)));
typedef int intx2 __attribute__((ext_vector_type(2)));

constexpr int BM = BLOCK_ROWS, BN = BLOCK_COLS, WM = WAVE_ROWS, WN = WAVE_COLS, BK = BLOCK_K;
constexpr int STAGES = K_STAGES, SPLITK = SPLIT_K;
constexpr int WAVES_M = BM / WM, WAVES_N = BN / WN, NWAVES = WAVES_M * WAVES_N, NTHREADS = 64 * NWAVES;
constexpr int TM = WM / 16, TN = WN / 16;      // MFMA tiles per wave
constexpr int KSTEPS = BK / 32;                // 32-wide MFMA k-steps per K tile
constexpr int A_STAGE_BYTES = BM * BK * 2, B_STAGE_BYTES = BN * BK * 2;   // one K tile of each operand in LDS
constexpr int STAGE_BYTES = A_STAGE_BYTES + B_STAGE_BYTES;
// epilogue staging: one 32 x WAVE_COLS strip of halves per wave, rows padded by 16 bytes
constexpr int STRIP_LD = WN * 2 + 16;
constexpr int STRIP_BYTES = 32 * STRIP_LD;
constexpr int OOB_OFFSET = 0x7fffffff;         // byte offset beyond any buffer: the load returns zeros

static_assert(BM % WM == 0 && BN % WN == 0, "block tile must be a multiple of the wave tile");
static_assert(WM % 32 == 0 && WN % 16 == 0, "wave tile: rows in multiples of 32 (the epilogue pairs 16-row tiles), columns of 16");
static_assert(NTHREADS <= 1024, "bad thread count");
static_assert(SPLITK >= 1 && SPLITK <= 8, "SPLIT_K out of range");

using helix_fastdiv::FastDiv;   // division by a run-time constant as multiply and shift

struct ConvGeom {
    int H, W, IC, OH, OW, kW, stride, pad, M;  // M = batch*OH*OW
    FastDiv by_OW, by_OH, by_IC, by_kW;
};

struct Params {
    const half_t* A;   // GEMM: M x K (lda).  CONV: x, NHWC
    const half_t* B;   // N x K (ldb).        CONV: w, [OC][kH][kW][IC]
    half_t* C;         // M x N (ldc)
    float* ws;         // SPLIT_K > 1: [splits][M][N] FP32 partial sums
    int splits;        // K partitions of this launch (1 when SPLIT_K == 1)
    int M, N, K, lda, ldb, ldc;
    int tiles_m, tiles_n;
    unsigned a_bytes;  // CONV: size of x in bytes (bounds for the gather)
    helix_splitk::Plan plan;   // SPLIT_K > 1: how the partitions of a tile are added (common/helix_splitk.h)
    ConvGeom g;
};


// ---- workgroup id -> output tile and K range --------------------------------------------------------------
struct TileRange {
    int m0, n0, k_begin, k_end;
    int tile, split;   // output tile number and K partition of this workgroup
    bool idle;         // a workgroup id beyond the tiles of its XCD (grids are padded to whole rounds of 8 ids)
};

__device__ __forceinline__ TileRange tile_range_of_workgroup(const Params& p) {
    // workgroup id -> tile number (XCD-aware: ids are dealt round-robin to the 8 XCDs, and each XCD is given a
    // compact run of tile numbers) and K partition
    const helix_splitk::Unit u = helix_splitk::unit_of_workgroup(p.plan, p.tiles_m * p.tiles_n, p.splits);
    const int pid = u.tile;
    const int group_tiles = GROUP_ROWS * p.tiles_n;
    const int grp = pid / group_tiles;
    const int first_m = grp * GROUP_ROWS;
    const int gsize = (p.tiles_m - first_m) < GROUP_ROWS ? (p.tiles_m - first_m) : GROUP_ROWS;
    const int in_grp = pid % group_tiles;
    const int tile_m = first_m + in_grp % gsize;
    const int tile_n = in_grp / gsize;
    // K range of this workgroup (split-K partitions are multiples of BLOCK_K)
    int k_begin = 0, k_end = p.K;
    if (SPLITK > 1) {
        const int ktiles = (p.K + BK - 1) / BK;
        const int per_k = (ktiles + p.splits - 1) / p.splits;
        k_begin = u.split * per_k * BK;
        k_end = k_begin + per_k * BK;
        if (k_end > p.K) k_end = p.K;
        if (k_begin > p.K) k_begin = p.K;
    }
    return TileRange{tile_m * BM, tile_n * BN, k_begin, k_end, pid, u.split, u.idle};
}

// ---- epilogue: accumulators -> C (or the split-K workspace) -------------------------------------------------
// The MFMAs were issued with the B fragment as the first operand, so accumulator tile (i, j) holds the transposed
// 16x16 block: lane l owns tile row m = l % 16 and the four consecutive tile columns n = 4*(l/16) + {0,1,2,3}.

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

// FP32 partial sums of K partition `split` into the workspace: four consecutive columns per lane, one 16-byte
// store where that is aligned.
__device__ __forceinline__ void store_partial(floatx4 (&acc)[TM][TN], const Params& p, int m0, int n0, int split,
                                              int wave_m, int wave_n, int lane) {
    const int m_l = lane & 15, n_l = (lane >> 4) * 4;
    const bool vec_ok = (p.N % 4 == 0);
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int row = m0 + wave_m * WM + i * 16 + m_l;
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int col = n0 + wave_n * WN + j * 16 + n_l;
            if (row < p.M) {
                float* dst = p.ws + ((size_t)split * p.M + row) * p.N + col;
                if (vec_ok && col + 4 <= p.N) {
                    *(floatx4*)dst = acc[i][j];
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (col + e < p.N) dst[e] = acc[i][j][e];
                }
            }
        }
    }
}

// FP16 result through LDS: each wave rounds a 32 x WAVE_COLS strip into its private LDS region (8-byte writes),
// reads it back row-contiguous and stores 16 bytes per lane, so a store instruction covers whole
// 2*WAVE_COLS-byte row segments.
__device__ __forceinline__ void store_result(floatx4 (&acc)[TM][TN], const Params& p, int m0, int n0, int wave, int wave_m,
                                             int wave_n, int lane, unsigned char* smem) {
    const int m_l = lane & 15, n_l = (lane >> 4) * 4;
    __syncthreads();   // every wave is done reading the ring; the strips reuse its memory
    unsigned char* strip = smem + wave * STRIP_BYTES;
    // widest store the row stride and base address allow: 8, 4, 2 or 1 halves at a time
    const int valign = (int)(((uintptr_t)p.C >> 1) | (unsigned)p.ldc) & 7;
    const int vec = (valign == 0) ? 8 : (valign & 3) == 0 ? 4 : (valign & 1) == 0 ? 2 : 1;
    constexpr int CPR = WN / 8;                    // 16-byte chunks per strip row
#pragma unroll
    for (int ii = 0; ii < TM / 2; ii++) {
#pragma unroll
        for (int hh = 0; hh < 2; hh++) {
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const floatx4 a = acc[ii * 2 + hh][j];
                half4 h = {(half_t)a[0], (half_t)a[1], (half_t)a[2], (half_t)a[3]};
                *(half4*)(strip + (hh * 16 + m_l) * STRIP_LD + (j * 16 + n_l) * 2) = h;
            }
        }
        __builtin_amdgcn_wave_barrier();   // same-wave LDS traffic stays in program order
#pragma unroll
        for (int t = 0; t < (32 * CPR) / 64; t++) {
            const int idx = t * 64 + lane;
            const int r = idx / CPR, ch = idx % CPR;
            const intx4 v = *(const intx4*)(strip + r * STRIP_LD + ch * 16);
            const int row = m0 + wave_m * WM + ii * 32 + r;
            const int col = n0 + wave_n * WN + ch * 8;
            if (row < p.M && col < p.N) {
                half_t* dst = p.C + (size_t)row * p.ldc + col;
                // non-temporal: the result is not read again by this launch, and the operand panels keep their
                // place in the caches (measured: layers whose output is most of their traffic 6 - 10 % faster)
                if (vec == 8 && col + 8 <= p.N) {
                    __builtin_nontemporal_store(v, (intx4*)dst);
                } else if (vec == 4 && col + 8 <= p.N) {
                    __builtin_nontemporal_store(intx2{v[0], v[1]}, (intx2*)dst);
                    __builtin_nontemporal_store(intx2{v[2], v[3]}, (intx2*)dst + 1);
                } else if (vec == 2 && col + 8 <= p.N) {
#pragma unroll
                    for (int e = 0; e < 4; e++) ((int*)dst)[e] = v[e];
                } else {
                    const half8 hv = __builtin_bit_cast(half8, v);
#pragma unroll
                    for (int e = 0; e < 8; e++)
                        if (col + e < p.N) dst[e] = hv[e];
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
}

// The epilogue of a tile kernel: accumulators -> C, through the workspace when K is partitioned.  LDS_PER_WG: the
// kernel's LDS allocation (it bounds the workgroups per compute unit).
template <int LDS_PER_WG>
__device__ __forceinline__ void store_tile(floatx4 (&acc)[TM][TN], const Params& p, const TileRange& tr, int tid, int wave,
                                           int wave_m, int wave_n, int lane, unsigned char* smem) {
    if (SPLITK > 1) {
        store_partial(acc, p, tr.m0, tr.n0, tr.split, wave_m, wave_n, lane);
        constexpr int WG_PER_CU = (160 * 1024) / LDS_PER_WG;
        constexpr bool ROOMY = WG_PER_CU * NWAVES <= 8;            // at most two waves per SIMD: 256 registers each
        if (p.plan.fused)                                          // else helix_splitk_reduce_kernel adds the partials
            helix_splitk::sum_partitions_if_last<half_t, BM, BN, NTHREADS, SPLITK, ROOMY ? 32 : 16>(
                p.plan, p.ws, p.C, p.M, p.N, p.ldc, p.splits, tr.tile, tr.m0, tr.n0, tid, smem);
        return;
    }
    store_result(acc, p, tr.m0, tr.n0, wave, wave_m, wave_n, lane, smem);
}


// Sums the SPLIT_K FP32 partials in a fixed order and rounds once to FP16 (deterministic, unlike
// the reference's half2 atomics, src_template/Ampere_FP16/gemm_splitK.cu:495-506).
__global__ void helix_splitk_reduce_kernel(const float* ws, half_t* C, int M, int N, int ldc, int splits) {
    const size_t total = (size_t)M * N;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        float s = 0.f;
        for (int k = 0; k < splits; k++) s += ws[(size_t)k * total + idx];
        const size_t row = idx / N, col = idx % N;
        C[row * ldc + col] = (half_t)s;
    }
}

}  // namespace

namespace tpl {

constexpr int kElemBytes = 2;


// K partitions for an M x N x K problem: enough to hand every one of the 256 compute units a workgroup,
// at least 2 (the reference's split-K is always 2-way, gemm_splitK.cu:124-129), at most SPLIT_K, and
// never so many that a partition has fewer than two K tiles.
inline int split_factor(long long M, long long N, long long K) {
    if (SPLITK <= 1) return 1;
    const long long tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
    const long long ktiles = (K + BK - 1) / BK;
    long long s = 256 / (tiles > 0 ? tiles : 1);
    if (s > SPLITK) s = SPLITK;
    if (s > ktiles / 2) s = ktiles / 2;
    if (s < 2) s = 2;
    return (int)s;
}

inline size_t workspace_bytes(int M, int N, int K) {
    return SPLITK > 1 ? (size_t)split_factor(M, N, K) * (size_t)M * (size_t)N * sizeof(float) : 0;
}

// Grid of a launch of p: one-dimensional when the partitions are added inside the launch (p.plan.fused), else
// tiles x partitions with the reduction kernel behind it.
inline dim3 launch_grid(Params& p) {
    const long long ntiles = (long long)p.tiles_m * p.tiles_n;
    const unsigned fused = SPLITK > 1 ? helix_splitk::plan_launch(p.plan, ntiles, p.splits, p.M, p.N) : 0u;
    if (SPLITK <= 1) p.plan = helix_splitk::Plan{0, 0u, nullptr};
    return fused ? dim3(fused, 1, 1) : dim3((unsigned)ntiles, (unsigned)p.splits, 1);
}

inline void bench_layout(int M, int N, int K, size_t* ae, size_t* be, size_t* ce, int* lda, int* ldb, int* ldc) {
    *ae = (size_t)M * K; *be = (size_t)N * K; *ce = (size_t)M * N;
    *lda = K; *ldb = K; *ldc = N;
}

}  // namespace tpl
