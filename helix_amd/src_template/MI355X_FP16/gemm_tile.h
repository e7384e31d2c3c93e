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

#include "helix_abi.h"
#include "helix_fastdiv.h"

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
    // SPLIT_K > 1, partitions summed inside the launch: the grid is one-dimensional, workgroup id L runs partition
    // (L / 8) % splits of tile number (L / 8) / splits of XCD L % 8
    int fused;
    unsigned xcc_map;  // XCC_ID the hardware reports for workgroup ids 0 .. 7 (ids are dealt round-robin), 4 bits each
    unsigned* arrive;  // one arrival counter per output tile, zero between launches
    ConvGeom g;
};


// ---- workgroup id -> output tile and K range --------------------------------------------------------------
struct TileRange {
    int m0, n0, k_begin, k_end;
    int tile, split;   // output tile number and K partition of this workgroup
    bool idle;         // a workgroup id beyond the tiles of its XCD (grids are padded to whole rounds of 8 ids)
};

__device__ __forceinline__ TileRange tile_range_of_workgroup(const Params& p) {
    // workgroup id -> (tile_m, tile_n), XCD-aware: ids are dealt round-robin to the 8 XCDs, so XCD x is given the
    // compact run of tiles [x * per + min(x, rem), ...) and walks it slot by slot
    const int ntiles = p.tiles_m * p.tiles_n;
    const int per = ntiles / 8, rem = ntiles % 8;
    int pid, split = 0;
    bool idle = false;
    if (SPLITK > 1 && p.fused) {
        const int xcd = (int)blockIdx.x % 8, j = (int)blockIdx.x / 8;
        const int slot = j / p.splits;
        split = j - slot * p.splits;
        idle = slot >= per + (xcd < rem ? 1 : 0);
        pid = xcd * per + (xcd < rem ? xcd : rem) + slot;
    } else {
        const int xcd = (int)blockIdx.x % 8, slot = (int)blockIdx.x / 8;
        pid = xcd * per + (xcd < rem ? xcd : rem) + slot;
        split = (int)blockIdx.y;
    }
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
        k_begin = split * per_k * BK;
        k_end = k_begin + per_k * BK;
        if (k_end > p.K) k_end = p.K;
        if (k_begin > p.K) k_begin = p.K;
    }
    return TileRange{tile_m * BM, tile_n * BN, k_begin, k_end, pid, split, idle};
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

// ---- K partitions summed inside the launch --------------------------------------------------------------------
// The eight L2 caches of the part are not coherent with each other: a workgroup that reads another one's partial
// sums across XCDs needs the writer to write its whole L2 back and the reader to invalidate its own (the
// device-scope release / acquire), which costs more than a second kernel.  Inside one XCD there is nothing to do:
// stores go through the compute unit's write-through vector cache to the shared L2, and a load that bypasses the
// vector cache finds them there.  So the host numbers the workgroups such that all partitions of a tile fall on
// one XCD (ids are dealt round-robin), every workgroup checks the XCC_ID the hardware reports against the one
// expected for its id, and
//   * writes its partial tile, waits until the L2 has acknowledged the stores, and counts itself in on the tile's
//     arrival counter (one device-scope atomic per workgroup, no spinning: nobody waits for anybody);
//   * the workgroup whose arrival completes the tile adds the partials in partition order (the same order and the
//     same FP32 additions as helix_splitk_reduce_kernel, so both paths give identical bits), resets the counter and
//     stores the FP16 result (straight from the sums: the partial tiles are read row by row, not in the MFMA layout);
//   * a workgroup that finds itself on another XCD than expected adds the device-scope release, and tells the
//     tile's last workgroup through the counter's upper half to add the acquire: correct on any placement, fast on
//     the expected one.
// Measured on 196 x 512 x 4608 (64 x 64 tiles, 8 partitions): 3.3 us from the last partial store to the end of the
// launch (arrival 1.8 us, sum 1.5 us) against 5.0 us for the second kernel and the gap in front of it.  Fetching the
// counter's cache line ahead of the arrival (an atomic add of zero at the start of the kernel, or next to the partial
// stores) was measured as well and is 0.5 - 0.7 us slower: it holds up the loads behind it.
__device__ __forceinline__ unsigned xcc_id() {   // HW_REG_XCC_ID (register 20), XCC_ID = bits 3:0
    return (unsigned)__builtin_amdgcn_s_getreg((4 - 1) << 11 | 0 << 6 | 20) & 15u;
}

typedef __attribute__((address_space(3))) unsigned char* lds_bytes_t;

// The threads of a workgroup walk the tile linearly (thread t takes the four-column chunks t, t + NTHREADS, ...), add
// the first PARTS partitions of each chunk in order (partitions beyond p.splits read as zeros through the buffer
// bounds check and add nothing) and store four halves.  BATCH chunks x PARTS partitions of loads are in flight per
// thread.
template <int PARTS, int BATCH>
__device__ __forceinline__ void sum_partitions(const Params& p, const TileRange& tr, int tid) {
    constexpr int CH_PER_ROW = BN / 4, PER_THREAD = BM * CH_PER_ROW / NTHREADS;
    static_assert((BM * CH_PER_ROW) % NTHREADS == 0, "the tile divides over the threads");
    const int slice_bytes = p.M * p.N * 4;                // one partition; the host keeps splits * slice below 2^31
    // cache policy sc0 | sc1: past this compute unit's vector cache, to the L2 the partials were written to
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(p.ws, (unsigned)p.splits * (unsigned)slice_bytes);
    const bool wide = (((uintptr_t)p.C & 7) == 0) && (p.ldc % 4 == 0);
    for (int c0 = 0; c0 < PER_THREAD; c0 += BATCH) {
        floatx4 v[BATCH][PARTS];
        int row[BATCH], col[BATCH];
#pragma unroll
        for (int b = 0; b < BATCH; b++) {
            const int chunk = tid + (c0 + b) * NTHREADS;
            // a last batch that is not full: its surplus chunks lie beyond the tile and are masked out by row
            row[b] = (c0 + b < PER_THREAD) ? tr.m0 + chunk / CH_PER_ROW : p.M;
            col[b] = tr.n0 + (chunk % CH_PER_ROW) * 4;
            const int voff = (row[b] < p.M && col[b] < p.N) ? (row[b] * p.N + col[b]) * 4 : OOB_OFFSET;
            // the partition's offset goes into the per-lane offset, the one the bounds check looks at
#pragma unroll
            for (int k = 0; k < PARTS; k++) {
                const int off = (k < p.splits && voff != OOB_OFFSET) ? voff + k * slice_bytes : OOB_OFFSET;
                v[b][k] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rs, off, 0, 17));
            }
        }
#pragma unroll
        for (int b = 0; b < BATCH; b++) {
            floatx4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int k = 0; k < PARTS; k++) {
                sum[0] += v[b][k][0]; sum[1] += v[b][k][1]; sum[2] += v[b][k][2]; sum[3] += v[b][k][3];
            }
            if (row[b] < p.M && col[b] < p.N) {           // N is a multiple of 4 on this path: whole chunks
                half_t* dst = p.C + (size_t)row[b] * p.ldc + col[b];
                const half4 h = {(half_t)sum[0], (half_t)sum[1], (half_t)sum[2], (half_t)sum[3]};
                if (wide) {
                    *(half4*)dst = h;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++) dst[e] = h[e];
                }
            }
        }
    }
}

// Called by every thread of the workgroup behind store_partial: counts the workgroup in and, in the one workgroup
// whose arrival completes the tile, adds the partitions and stores the result.
__device__ __forceinline__ void sum_partitions_if_last(const Params& p, const TileRange& tr, int tid, unsigned char* smem) {
    const bool placed = xcc_id() == ((p.xcc_map >> (4 * ((unsigned)blockIdx.x % 8u))) & 15u);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // this wave's partial sums have reached the L2
    if (!placed) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    __syncthreads();                                      // ... and every other wave's; the LDS ring is free
    volatile __attribute__((address_space(3))) unsigned* flag =
        (volatile __attribute__((address_space(3))) unsigned*)(lds_bytes_t)smem;
    if (tid == 0) {
        *flag = __hip_atomic_fetch_add(p.arrive + tr.tile, placed ? 1u : 0x10001u, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    const unsigned old = *flag;
    if ((int)(old & 0xffffu) + 1 != p.splits) return;
    if ((old >> 16) != 0 || !placed) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    if (tid == 0) __hip_atomic_store(p.arrive + tr.tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    // sixteen 16-byte loads in flight per thread: four chunks of up to four partitions, or two chunks of up to eight
    if (p.splits <= 4) sum_partitions<4, 4>(p, tr, tid);
    else sum_partitions<SPLITK, 2>(p, tr, tid);
}

// The epilogue of a tile kernel: accumulators -> C, through the workspace when K is partitioned.
__device__ __forceinline__ void store_tile(floatx4 (&acc)[TM][TN], const Params& p, const TileRange& tr, int tid, int wave,
                                           int wave_m, int wave_n, int lane, unsigned char* smem) {
    if (SPLITK > 1) {
        store_partial(acc, p, tr.m0, tr.n0, tr.split, wave_m, wave_n, lane);
        if (p.fused) sum_partitions_if_last(p, tr, tid, smem);   // else helix_splitk_reduce_kernel adds the partials
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

}  // namespace tpl

#if SPLIT_K > 1
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <mutex>

namespace {

// Arrival counters of the in-launch partition sum: FUSED_MAX_TILES per launch, ARRIVE_SETS sets used in turn so that
// up to ARRIVE_SETS launches of this library may be in flight on one GPU at a time (different streams).  They live
// in the library's device image, are zero when the code object is loaded, and every launch leaves them zero.
constexpr int FUSED_MAX_TILES = 1024, ARRIVE_SETS = 8;
static __device__ unsigned helix_arrive[ARRIVE_SETS * FUSED_MAX_TILES];

// Workgroup id -> XCC_ID as the hardware deals a one-dimensional grid, recorded once per device.
__global__ void helix_xcc_probe_kernel(unsigned* out) {
    if (threadIdx.x == 0) out[blockIdx.x] = xcc_id();
}

}  // namespace

namespace tpl {

struct FusedSplitK {
    int state = 0;              // 0: not looked at yet; 1: usable; -1: not usable on this device (second kernel instead)
    unsigned* arrive = nullptr; // device address of helix_arrive on this device
    unsigned xcc_map = 0;
};

// Per device, on first use: where the counters live and which XCC_ID the round-robin deal gives workgroup ids
// 0 .. 7 (probed with a 64-workgroup launch; an irregular deal, any HIP error, or HELIX_SPLITK_REDUCE=kernel in the
// environment leaves the second-kernel path in charge).  The probe synchronises the device once; it must not
// happen under stream capture, like any first launch of a library.
inline const FusedSplitK& fused_splitk() {
    static FusedSplitK per_device[64];
    static std::mutex lock;
    static const FusedSplitK none{-1, nullptr, 0};
    int d = -1;
    if (hipGetDevice(&d) != hipSuccess || d < 0 || d >= 64) return none;
    std::lock_guard<std::mutex> hold(lock);
    FusedSplitK& f = per_device[d];
    if (f.state != 0) return f;
    f.state = -1;
    const char* how = getenv("HELIX_SPLITK_REDUCE");
    if (how && strcmp(how, "kernel") == 0) return f;
    unsigned* base = nullptr;
    unsigned seen[64];
    constexpr int PROBE = 64;
    bool ok = hipGetSymbolAddress((void**)&base, HIP_SYMBOL(helix_arrive)) == hipSuccess && base != nullptr;
    if (ok) {
        hipLaunchKernelGGL(helix_xcc_probe_kernel, dim3(PROBE), dim3(64), 0, nullptr, base);
        ok = hipGetLastError() == hipSuccess && hipMemcpy(seen, base, sizeof(seen), hipMemcpyDeviceToHost) == hipSuccess &&
             hipMemset(base, 0, sizeof(seen)) == hipSuccess && hipDeviceSynchronize() == hipSuccess;
    }
    if (!ok) {
        (void)hipGetLastError();
        return f;
    }
    unsigned map = 0;
    for (int i = 0; i < PROBE; i++)
        if (seen[i] > 15u || seen[i] != seen[i % 8]) return f;
    for (int i = 0; i < 8; i++) map |= seen[i] << (4 * i);
    f.arrive = base;
    f.xcc_map = map;
    f.state = 1;
    if (getenv("HELIX_DEBUG")) fprintf(stderr, "helix: device %d deals workgroup ids 0..7 to XCC_IDs 0x%08x (nibble per id)\n", d, map);
    return f;
}

// Sets up p for a launch whose K partitions are summed inside it and returns the one-dimensional grid size, or
// returns 0 when this launch takes the second-kernel path.
inline unsigned fused_grid(Params& p) {
    static std::atomic<unsigned> launches{0};
    p.fused = 0;
    const long long ntiles = (long long)p.tiles_m * p.tiles_n;
    // byte offsets into the partials are 32-bit; chunks of four columns must not straddle the edge of C
    if (p.splits < 2 || ntiles > FUSED_MAX_TILES || (long long)p.splits * p.M * p.N * 4 >= 0x7fffffffLL || p.N % 4 != 0)
        return 0;
    const FusedSplitK& f = fused_splitk();
    if (f.state != 1) return 0;
    p.fused = 1;
    p.xcc_map = f.xcc_map;
    p.arrive = f.arrive + (launches.fetch_add(1) % ARRIVE_SETS) * FUSED_MAX_TILES;
    const long long slots = (ntiles + 7) / 8;            // most tiles any XCD is given
    return (unsigned)(8 * slots * p.splits);
}

}  // namespace tpl
#else
namespace tpl {
inline unsigned fused_grid(Params& p) {
    p.fused = 0;
    return 0;
}
}  // namespace tpl
#endif

namespace tpl {

inline void bench_layout(int M, int N, int K, size_t* ae, size_t* be, size_t* ce, int* lda, int* ldb, int* ldc) {
    *ae = (size_t)M * K; *be = (size_t)N * K; *ce = (size_t)M * N;
    *lda = K; *ldb = K; *ldc = N;
}

}  // namespace tpl
