// MI355X (gfx950 / CDNA4) FP32 GEMM + implicit-GEMM convolution template on the FP32 matrix cores.
//
//   GEMM : C[M x N] = A^T * B with A stored K x M and B stored K x N (row-major FP32), the operand
//          convention of the reference FP32 kernel (src_template/Ampere_FP32/sgemm.cu:138,378-382).
//   CONV : y[B,OH,OW,OC] = conv2d(x[B,H,W,IC], w[OC,kH,kW,IC]), FP32, == GEMM with M = B*OH*OW, N = OC,
//          K = kH*kW*IC; both operands are then K-contiguous and are transposed on their way into LDS.
//
// Role in the reference: src_template/Ampere_FP32/sgemm.cu:97-350 (`mySgemmCPAsyncTemplate`, a CUDA-core
// register-tiled SGEMM with macros BM, BN, BK, TM, TN, :60-93).  Here the contraction runs on
// v_mfma_f32_32x32x2_f32: one wave64 owns a WAVE_M x WAVE_N tile made of 32x32 MFMA tiles, each MFMA
// consuming two k values; products are accumulated in ascending k within a K partition, the order the CPU
// path uses.
//
// Compile-time parameters: BM x BN workgroup tile, BK (K extent of one LDS stage), WAVE_M x WAVE_N, K_GROUPS
// (waves per wave tile, each taking BK / K_GROUPS of every K tile; 1 unless the configuration is a K-group one).
//
// K partitions: a problem is split along K, up to 8 ways, when that shortens the launch: few tiles and a long K
// (compute units idle), or a tile count that leaves the last round of workgroups mostly empty (split_factor
// below); partial sums go to the caller's workspace (helix_workspace_bytes) and are added in partition order by
// the last workgroup of a tile to finish (all partitions of a tile run on one XCD, common/helix_splitk.h) or,
// where that is not available (K-group configurations among them), by a second kernel; same bits either way.
// Without the workspace the problem runs unpartitioned.  The reference's FP32 template has no K partition.
//
// LDS layout: A stage is [BK][BM + 32] floats, B stage [BK][BN + 32]; a fragment read takes lanes 0-31
// from row k and lanes 32-63 from row k+1, and the 32-float row padding puts the two half-waves on
// different halves of the 64 banks.  In CONV mode operands arrive K-contiguous and are written
// transposed into the same layout.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "helix_abi.h"
#include "helix_im2col.h"
#include "helix_fastdiv.h"
#include "helix_splitk.h"

#ifndef BM
#define BM 128
#endif
#ifndef BN
#define BN 128
#endif
#ifndef BK
#define BK 16
#endif
#ifndef WAVE_M
#define WAVE_M 64
#endif
#ifndef WAVE_N
#define WAVE_N 64
#endif
#ifndef K_GROUPS
#define K_GROUPS 1   // groups of waves that share one output tile and each take a slice of every K tile
#endif
#ifndef GROUP_ROWS
#define GROUP_ROWS 8
#endif
#ifndef SPLITK_TARGET_BLOCKS
#define SPLITK_TARGET_BLOCKS 768   // workgroups a K-partitioned launch aims for: three per compute unit
#endif

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef int intx4 __attribute__((ext_vector_type(4)));

// K_GROUPS > 1: the workgroup holds K_GROUPS waves per wave tile.  An accumulator is a chain of dependent MFMAs,
// K / 2 of them at 64 cycles each, whatever the tile shape: a problem of few tiles and long K is bound by that
// chain (and by the few bytes its workgroups keep in flight), so the waves of a group each multiply BK / K_GROUPS
// of every K tile and the partial tiles are added through LDS at the end -- the K partitioning of a split-K
// launch, inside the workgroup and without the second kernel.
constexpr int KG = K_GROUPS;
constexpr int WAVES_M = BM / WAVE_M, WAVES_N = BN / WAVE_N, WAVES_MN = WAVES_M * WAVES_N, NWAVES = WAVES_MN * KG,
              NTHREADS = 64 * NWAVES;
constexpr int TM = WAVE_M / 32, TN = WAVE_N / 32;
constexpr int KSTEPS = BK / 2 / KG;   // MFMA k steps (2 of K each) of one wave per K tile
// LDS row strides in floats.  GEMM mode: +32, which puts the two half-waves of a fragment read on different bank
// halves and keeps rows 16-byte aligned for the 128-bit tile writes.  CONV mode writes scalars, BK/4 lanes per
// tile row along k: the extra 16 / (BK/4) floats make the rows those lanes write fall on different banks
// (4 * stride = 64 / (BK/4) mod 64) instead of all on one; from BK = 64 on one extra float (an odd stride: 16
// distinct banks for the 16 or 32 lanes of a row, where an even one put them all on the same bank).
constexpr int CONV_PAD = 32 + (BK >= 64 ? 1 : BK >= 8 ? 64 / BK : 0);
template <bool CONV> struct Lds {
    static constexpr int LDA = BM + (CONV ? CONV_PAD : 32), LDB = BN + (CONV ? CONV_PAD : 32);
    static constexpr int A_STAGE = BK * LDA, B_STAGE = BK * LDB;    // floats
    static constexpr int STAGE = A_STAGE + B_STAGE;
    static constexpr int BYTES = 2 * STAGE * 4;
};
constexpr int REDUCE_BYTES = (KG - 1) * BM * BN * 4;   // partial tiles of the wave groups beyond the first
constexpr int STAGES_BYTES = Lds<true>::BYTES > Lds<false>::BYTES ? Lds<true>::BYTES : Lds<false>::BYTES;
constexpr int LDS_BYTES = STAGES_BYTES > REDUCE_BYTES ? STAGES_BYTES : REDUCE_BYTES;
// GEMM mode: tile rows are k, 16-byte chunks run along m / n
constexpr int A_CPR = BM / 4, B_CPR = BN / 4;                // chunks per tile row
constexpr int A_ITERS = BK * A_CPR / NTHREADS, B_ITERS = BK * B_CPR / NTHREADS;
// CONV mode: tile rows are m / n, 16-byte chunks run along k
constexpr int K_CPR = BK / 4;
constexpr int AC_ITERS = BM * K_CPR / NTHREADS, BC_ITERS = BN * K_CPR / NTHREADS;

static_assert(BM % WAVE_M == 0 && BN % WAVE_N == 0, "block tile must be a multiple of the wave tile");
static_assert(WAVE_M % 32 == 0 && WAVE_N % 32 == 0, "wave tile is built from 32x32 MFMA tiles");
static_assert(BK % 4 == 0 && BK >= 4, "BK must be a multiple of 4");
static_assert(KG >= 1 && (BK / 2) % KG == 0, "the k steps of a K tile must divide among the wave groups");
static_assert(NTHREADS <= 1024, "too many waves");
static_assert((BK * A_CPR) % NTHREADS == 0 && (BK * B_CPR) % NTHREADS == 0, "tile copy must divide evenly");
static_assert((BM * K_CPR) % NTHREADS == 0 && (BN * K_CPR) % NTHREADS == 0, "conv tile copy must divide evenly");
static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of a gfx950 CU exceeded");

using helix_fastdiv::FastDiv;   // division by a run-time constant as multiply and shift

struct ConvGeom {
    int H, W, IC, OH, OW, kW, stride, pad, M;
    FastDiv by_OW, by_OH, by_IC, by_kW;
};

struct Params {
    const float* A;  // GEMM: K x M (lda).  CONV: x, NHWC
    const float* B;  // GEMM: K x N (ldb).  CONV: w, [OC][kH][kW][IC]
    float* C;        // M x N (ldc)
    int M, N, K, lda, ldb, ldc;
    int tiles_m, tiles_n;
    unsigned a_bytes;
    float* ws;       // splits > 1: [splits][M][N] partial sums
    int splits;      // K partitions of this launch
    int k_per;       // K extent of one partition, a multiple of BK
    helix_splitk::Plan plan;   // how the partitions of a tile are added
    ConvGeom g;
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

__device__ __forceinline__ floatx4 buf_load16(__amdgpu_buffer_rsrc_t r, int voff) {
    return __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, 0, 0));
}

constexpr int OOB = 0x7fffffff;  // byte offset beyond any buffer: the load returns zeros

// The tile parameters appear as (otherwise unused) template arguments so that every configuration's
// kernel has its own symbol name and a profiler lists configurations separately.
template <bool CONV, int T_BM = BM, int T_BN = BN, int T_BK = BK, int T_WM = WAVE_M, int T_WN = WAVE_N, int T_KG = KG>
__global__ __launch_bounds__(NTHREADS) void helix_sgemm_f32_kernel(const Params p) {
    constexpr int LDA_S = Lds<CONV>::LDA, LDB_S = Lds<CONV>::LDB, A_STAGE = Lds<CONV>::A_STAGE, STAGE = Lds<CONV>::STAGE;
    extern __shared__ __attribute__((aligned(16))) float smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wave_kg = wave / WAVES_MN, wave_mn = wave % WAVES_MN;
    const int wave_m = wave_mn / WAVES_N, wave_n = wave_mn % WAVES_N;

    // workgroup id -> tile number (the round-robin deal over the 8 XCDs undone: each XCD is given a compact run of
    // tile numbers) and K partition, then walk groups of tile rows
    const helix_splitk::Unit unit = helix_splitk::unit_of_workgroup(p.plan, p.tiles_m * p.tiles_n, p.splits);
    if (unit.idle) return;
    const int pid = unit.tile;
    const int group_tiles = GROUP_ROWS * p.tiles_n;
    const int first_m = (pid / group_tiles) * GROUP_ROWS;
    const int gsize = (p.tiles_m - first_m) < GROUP_ROWS ? (p.tiles_m - first_m) : GROUP_ROWS;
    const int tile_m = first_m + (pid % group_tiles) % gsize;
    const int tile_n = (pid % group_tiles) / gsize;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    // K range of this workgroup
    const int k_lo = unit.split * p.k_per;
    const int k_hi = (k_lo + p.k_per) < p.K ? (k_lo + p.k_per) : p.K;

    constexpr int NA = CONV ? AC_ITERS : A_ITERS;
    constexpr int NB = CONV ? BC_ITERS : B_ITERS;
    // two sets of staging registers: a K tile is requested two tiles ahead of its use, so that its loads have
    // a whole tile of MFMAs plus the previous tile's LDS writes to land
    floatx4 stage_a[2][NA], stage_b[2][NB];

    // CONV: per-row gather state
    int cv_img[NA], cv_ih[NA], cv_iw[NA];
    if (CONV) {
#pragma unroll
        for (int i = 0; i < NA; i++) {
            const int m = m0 + (tid + i * NTHREADS) / K_CPR;
            const int t = p.g.by_OW.div(m);
            const int ow = m - t * p.g.OW;
            const int b = p.g.by_OH.div(t);
            const int oh = t - b * p.g.OH;
            cv_img[i] = (m < p.g.M) ? b * p.g.H * p.g.W : -1;
            cv_ih[i] = oh * p.g.stride - p.g.pad;
            cv_iw[i] = ow * p.g.stride - p.g.pad;
        }
    }

    // CONV: buffer descriptors of the whole input and of this tile's weight rows (N x K row-major; rows >= N fall
    // outside), and the byte offsets of the next K tile to request: conv_offsets(k0) fills them for the tile at k0
    // (index arithmetic only), load_global then issues the loads from them.
    const int rows_b = (p.N - n0) < BN ? (p.N - n0) : BN;
    const __amdgpu_buffer_rsrc_t conv_ra = make_rsrc(p.A, CONV ? p.a_bytes : 0u);
    const __amdgpu_buffer_rsrc_t conv_rb =
        make_rsrc(p.B + (CONV ? (size_t)n0 * p.K : 0), CONV ? (unsigned)((size_t)rows_b * p.K * 4) : 0u);
    int off_a[NA], off_b[NB];
    auto conv_offsets = [&](int k0) {
        const int k = k0 + (tid % K_CPR) * 4;
        const bool dead = k >= k_hi;
        const int t = p.g.by_IC.div(k);
        const int c = k - t * p.g.IC;
        const int kh = p.g.by_kW.div(t);
        const int kw = t - kh * p.g.kW;
#pragma unroll
        for (int i = 0; i < NA; i++) {
            const int ih = cv_ih[i] + kh, iw = cv_iw[i] + kw;
            // no short-circuit evaluation and the offset computed either way: branches or predicated blocks here
            // would cut the tile's MFMA block into pieces
            const bool ok = (!dead) & (cv_img[i] >= 0) & ((unsigned)ih < (unsigned)p.g.H) & ((unsigned)iw < (unsigned)p.g.W);
            const int off = ((cv_img[i] + ih * p.g.W + iw) * p.g.IC + c) * 4;
            off_a[i] = ok ? off : OOB;
        }
#pragma unroll
        for (int i = 0; i < NB; i++) {
            const int n = (tid + i * NTHREADS) / K_CPR;
            const int off = (n * p.K + k) * 4;
            off_b[i] = dead ? OOB : off;
        }
    };

    auto load_global = [&](int k0, auto set_c) {
        constexpr int SET = decltype(set_c)::value;
        if (!CONV) {
            // rows k0.. of A^T (K x M) starting at column m0; whole rows are inside the buffer, rows >= K are not
            // past the end of the K range the descriptors are empty: the loads still issue (the wait counts in
            // front of the LDS writes then never depend on a branch) and return zeros
            const bool live = k0 < k_hi;
            __amdgpu_buffer_rsrc_t ra = make_rsrc(p.A + (size_t)(live ? k0 : 0) * p.lda + m0,
                                                  live ? (unsigned)(((size_t)(k_hi - k0) * p.lda - m0) * 4) : 0u);
            __amdgpu_buffer_rsrc_t rb = make_rsrc(p.B + (size_t)(live ? k0 : 0) * p.ldb + n0,
                                                  live ? (unsigned)(((size_t)(k_hi - k0) * p.ldb - n0) * 4) : 0u);
#pragma unroll
            for (int i = 0; i < NA; i++) {
                const int c = tid + i * NTHREADS;
                stage_a[SET][i] = buf_load16(ra, ((c / A_CPR) * p.lda + (c % A_CPR) * 4) * 4);
            }
#pragma unroll
            for (int i = 0; i < NB; i++) {
                const int c = tid + i * NTHREADS;
                stage_b[SET][i] = buf_load16(rb, ((c / B_CPR) * p.ldb + (c % B_CPR) * 4) * 4);
            }
        } else {
            // the offsets were computed a tile earlier (conv_offsets), among that tile's MFMAs
#pragma unroll
            for (int i = 0; i < NA; i++) stage_a[SET][i] = buf_load16(conv_ra, off_a[i]);
#pragma unroll
            for (int i = 0; i < NB; i++) stage_b[SET][i] = buf_load16(conv_rb, off_b[i]);
        }
    };

    auto store_lds = [&](int stage, auto set_c) {
        constexpr int SET = decltype(set_c)::value;
        float* sa = smem + stage * STAGE;
        float* sb = sa + A_STAGE;
        if (!CONV) {
#pragma unroll
            for (int i = 0; i < NA; i++) {
                const int c = tid + i * NTHREADS;
                *(floatx4*)(sa + (c / A_CPR) * LDA_S + (c % A_CPR) * 4) = stage_a[SET][i];
            }
#pragma unroll
            for (int i = 0; i < NB; i++) {
                const int c = tid + i * NTHREADS;
                *(floatx4*)(sb + (c / B_CPR) * LDB_S + (c % B_CPR) * 4) = stage_b[SET][i];
            }
        } else {
            const int kc = (tid % K_CPR) * 4;
#pragma unroll
            for (int i = 0; i < NA; i++) {
                const int m = (tid + i * NTHREADS) / K_CPR;
#pragma unroll
                for (int e = 0; e < 4; e++) sa[(kc + e) * LDA_S + m] = stage_a[SET][i][e];
            }
#pragma unroll
            for (int i = 0; i < NB; i++) {
                const int n = (tid + i * NTHREADS) / K_CPR;
#pragma unroll
                for (int e = 0; e < 4; e++) sb[(kc + e) * LDB_S + n] = stage_b[SET][i][e];
            }
        }
    };

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    // MFMA 32x32x2: lane l supplies A[l % 32][l / 32] and B[l / 32][l % 32]
    const int frow = lane & 31, fk = lane >> 5;
    const int a_rd = (wave_kg * (BK / KG) + fk) * LDA_S + wave_m * WAVE_M + frow;
    const int b_rd = A_STAGE + (wave_kg * (BK / KG) + fk) * LDB_S + wave_n * WAVE_N + frow;

    const int ktiles = (k_hi - k_lo + BK - 1) / BK;
    constexpr std::integral_constant<int, 0> set0{};
    constexpr std::integral_constant<int, 1> set1{};
    if (ktiles > 0) {
        if (CONV) conv_offsets(k_lo);
        load_global(k_lo, set0);
        if (CONV) conv_offsets(k_lo + BK);
        load_global(k_lo + BK, set1);
        if (CONV) conv_offsets(k_lo + 2 * BK);
        store_lds(0, set0);
    }
    __syncthreads();

    // Tile kt is multiplied from LDS stage kt % 2.  Its staging set (kt % 2) is free again -- the tile went to
    // LDS during tile kt - 1 -- and is refilled with tile kt + 2 before the MFMAs; tile kt + 1, requested a
    // whole tile earlier, goes from the other set to the other LDS stage after them.
    auto tile = [&](int kt, auto set_c) {
        constexpr int SET = decltype(set_c)::value;
        constexpr std::integral_constant<int, SET ^ 1> other{};
        load_global(k_lo + (kt + 2) * BK, set_c);       // empty past the end of the K range
        // the loads stay in front of the MFMAs and of the LDS writes below: sunk behind the writes, their
        // wait counts would drain the whole queue every tile
        __builtin_amdgcn_sched_barrier(0);
        // CONV: the gather offsets of tile kt + 3, free to be scheduled among the MFMAs below (computed in front
        // of their own loads they ran while the matrix pipe sat idle: all waves leave the barrier together)
        if (CONV) {
            int k_next = k_lo + (kt + 3) * BK;
            asm volatile("" : "+s"(k_next));   // keeps the arithmetic that follows on this side of the fence above
            conv_offsets(k_next);
        }

        const float* sb = smem + SET * STAGE;
#pragma unroll
        for (int s = 0; s < KSTEPS; s++) {
            float af[TM], bf[TN];
#pragma unroll
            for (int i = 0; i < TM; i++) af[i] = sb[a_rd + s * 2 * LDA_S + i * 32];
#pragma unroll
            for (int j = 0; j < TN; j++) bf[j] = sb[b_rd + s * 2 * LDB_S + j * 32];
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        if (CONV) {
            // issue order of the block above: the index arithmetic of conv_offsets dealt out behind the MFMAs, a
            // few instructions each (fragment reads are left to the scheduler, which keeps them a k step ahead)
            // (the first 16 MFMAs take all of it; asking for more groups only costs compile time, minutes for the
            // 128 x 128 wave tile)
            constexpr int MFMA = 0x008, VALU = 0x002, VALU_PER_MFMA = 3;
            constexpr int GROUPS = KSTEPS * TM * TN < 16 ? KSTEPS * TM * TN : 16;
#pragma unroll
            for (int q = 0; q < GROUPS; q++) {
                __builtin_amdgcn_sched_group_barrier(MFMA, 1, SET);
                __builtin_amdgcn_sched_group_barrier(VALU, VALU_PER_MFMA, SET);
            }
        }

        __builtin_amdgcn_sched_barrier(0);
        store_lds(SET ^ 1, other);                       // zeros past the end: the stage is not read again
        __syncthreads();
    };
    int kt = 0;
    for (; kt + 1 < ktiles; kt += 2) {
        tile(kt, set0);
        tile(kt + 1, set1);
    }
    if (kt < ktiles) tile(kt, set0);

    if (KG > 1) {
        // every wave is past the last tile's barrier: the stages are free.  Groups 1.. leave their partial tiles
        // in LDS ([group][wave tile][32x32 tile][register][lane]), group 0 adds them in group order and stores.
        float* red = smem;
        constexpr int TILE = TM * TN * 16 * 64;
        if (wave_kg > 0) {
            float* mine = red + ((wave_kg - 1) * WAVES_MN + wave_mn) * TILE + lane;
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
#pragma unroll
                    for (int v = 0; v < 16; v++) mine[((i * TN + j) * 16 + v) * 64] = acc[i][j][v];
        }
        __syncthreads();
        if (wave_kg > 0) return;
        for (int g = 1; g < KG; g++) {
            const float* theirs = red + ((g - 1) * WAVES_MN + wave_mn) * TILE + lane;
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
#pragma unroll
                    for (int v = 0; v < 16; v++) acc[i][j][v] += theirs[((i * TN + j) * 16 + v) * 64];
        }
    }

    // lane l holds column (l % 32); rows 8*(v/4) + 4*(l/32) + (v%4)
    const int col_l = lane & 31, row_l = (lane >> 5) * 4;
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int col = n0 + wave_n * WAVE_N + j * 32 + col_l;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = m0 + wave_m * WAVE_M + i * 32 + (v / 4) * 8 + row_l + (v % 4);
                if (row < p.M && col < p.N) {
                    if (p.splits > 1) p.ws[((size_t)unit.split * p.M + row) * p.N + col] = acc[i][j][v];
                    else __builtin_nontemporal_store(acc[i][j][v], &p.C[(size_t)row * p.ldc + col]);   // not read again by this launch
                }
            }
        }
    }
    if (KG == 1 && p.splits > 1 && p.plan.fused) {           // else helix_sgemm_splitk_reduce_kernel adds the partials
        // loads in flight while adding: what the main loop's registers already allow (32 where LDS keeps the kernel to
        // two waves per SIMD, 16 from 64 accumulator registers per lane on, else 8)
        constexpr bool ROOMY = ((160 * 1024) / LDS_BYTES) * NWAVES <= 8;
        constexpr int LOADS = ROOMY ? 32 : (TM * TN * 16 >= 64 ? 16 : 8);
        helix_splitk::sum_partitions_if_last<float, BM, BN, NTHREADS, 8, LOADS>(
            p.plan, p.ws, p.C, p.M, p.N, p.ldc, p.splits, pid, m0, n0, tid, (unsigned char*)smem);
    }
}

// Sums the K partitions in a fixed order (deterministic).
__global__ void helix_sgemm_splitk_reduce_kernel(const float* ws, float* C, int M, int N, int ldc, int splits) {
    const size_t total = (size_t)M * N;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        float s = 0.f;
        for (int k = 0; k < splits; k++) s += ws[(size_t)k * total + idx];
        C[(idx / N) * ldc + idx % N] = s;
    }
}

}  // namespace

#include <stdio.h>

namespace tpl {

constexpr int kElemBytes = 4;

inline const char* info_json() {
    static char buf[1024];
    static bool done = false;
    if (!done) {
        snprintf(buf, sizeof(buf),
                 "{\"family\": \"sgemm_f32\", \"arch\": \"gfx950\", \"mfma\": \"v_mfma_f32_32x32x2_f32\", "
                 "\"lds_stages\": 2, \"block_rows\": %d, \"block_cols\": %d, \"wave_rows\": %d, \"wave_cols\": %d, "
                 "\"block_k\": %d, \"k_groups\": %d, \"split_k\": \"up to 8 K partitions when the tiles leave compute units idle and the caller passes the workspace\", \"threads\": %d, \"lds_bytes\": %d, "
                 "\"layout_a\": \"K x M row-major f32 (A transposed)\", \"layout_b\": \"K x N row-major f32\", "
                 "\"layout_c\": \"M x N row-major f32\", \"accumulate\": \"f32\", "
                 "\"k_multiple\": 1, \"ld_multiple\": 4, \"conv\": \"NHWC x [OC][kH][kW][IC]; implicit GEMM when IC %% 4 == 0, else channel-padded copies or a column buffer in the workspace\"}",
                 BM, BN, WAVE_M, WAVE_N, BK, KG, NTHREADS, LDS_BYTES);
        done = true;
    }
    return buf;
}

// K partitions for an M x N x K problem.  At most SPLITK_FEW_TILES tiles (they do not even cover half of the
// compute units): towards SPLITK_TARGET workgroups, three per compute unit -- this kernel hides its LDS and
// global latencies across workgroups that share a compute unit --, at most SPLITK_MAX, and never so many that a
// partition walks less than SPLITK_MIN_K_FEW of K (SPLITK_MIN_K_TINY when there are at most 32 tiles: a
// 14 x 14 x 480 -> 192 1x1 convolution went 18 -> 10 us).  The reference's FP32 template has no K partition
// (src_template/Ampere_FP32/sgemm.cu); its FP16 one is 2-way (gemm_splitK.cu:124-129).
constexpr int SPLITK_MAX = 8, SPLITK_TARGET = SPLITK_TARGET_BLOCKS, SPLITK_MIN_K_FEW = 256, SPLITK_FEW_TILES = 128,
              SPLITK_MIN_K_TINY = 64, SPLITK_TINY_TILES = 32;

// More than SPLITK_FEW_TILES tiles: workgroups beyond one per compute unit queue up behind each other, so a launch
// takes ceil(workgroups / 256) rounds of one partition's K walk, and the partition count is the one that makes
// rounds x walk (plus a fixed cost per workgroup and the reduction pass) smallest -- 196 tiles of K = 4608 take four
// rounds of 1152 four ways and four rounds of 922 five ways (measured 305 -> 262 us), 784 tiles four rounds of 4608
// unpartitioned and thirteen of 1152 four ways (1060 -> 938 us).  Times in seconds, matrix pipes at
// SPLITK_MFMA_FRACTION of their peak; scripts/MI355X_FP32/MI355X_FP32_gemm.py evaluates the same expression.
constexpr double SPLITK_MFMA_FRACTION = 0.8, SPLITK_FP32_MFMA_FLOPS = 157.3e12, SPLITK_REDUCE_BYTES_PER_S = 5e12,
                 SPLITK_REDUCE_LAUNCH_S = 4e-6, SPLITK_MIN_GAIN = 0.98;
constexpr int SPLITK_MIN_K_BALANCE = 128, SPLITK_COMPUTE_UNITS = 256;

inline int split_factor(long long M, long long N, long long K) {
    const long long tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
    if (tiles <= 0) return 1;
    if (tiles <= SPLITK_FEW_TILES) {
        long long s = (SPLITK_TARGET + tiles - 1) / tiles;
        if (s > SPLITK_MAX) s = SPLITK_MAX;
        const long long min_k = tiles <= SPLITK_TINY_TILES ? SPLITK_MIN_K_TINY : SPLITK_MIN_K_FEW;
        if (s > K / min_k) s = K / min_k;
        return s < 1 ? 1 : (int)s;
    }
    const double per_k = 2.0 * BM * BN * SPLITK_COMPUTE_UNITS / (SPLITK_MFMA_FRACTION * SPLITK_FP32_MFMA_FLOPS);
    const double fixed = 1e-6 + 1.5e-6 * (BM * BN) / (128.0 * 128.0);
    const long long ktiles = (K + BK - 1) / BK;
    int best = 1;
    double best_t = 0.0;
    for (int s = 1; s <= SPLITK_MAX && (s == 1 || K / s >= SPLITK_MIN_K_BALANCE); s++) {
        const double walk = (double)(((ktiles + s - 1) / s) * BK);
        const double rounds = (double)((tiles * s + SPLITK_COMPUTE_UNITS - 1) / SPLITK_COMPUTE_UNITS);
        const double reduce = s > 1 ? SPLITK_REDUCE_LAUNCH_S + (s + 1.0) * (double)M * (double)N * 4.0 / SPLITK_REDUCE_BYTES_PER_S : 0.0;
        const double t = rounds * (walk * per_k + fixed) + reduce;
        if (s == 1 || t < best_t * SPLITK_MIN_GAIN) {   // a further partition has to pay for itself
            best_t = t;
            best = s;
        }
    }
    return best;
}

// Partial sums of the K partitions; a caller that passes less runs the problem unpartitioned.
inline size_t workspace_bytes(int M, int N, int K) {
    const int s = split_factor(M, N, K);
    return s > 1 ? (size_t)s * (size_t)M * (size_t)N * sizeof(float) : 0;
}

inline void bench_layout(int M, int N, int K, size_t* ae, size_t* be, size_t* ce, int* lda, int* ldb, int* ldc) {
    const int Mp = (M + 3) / 4 * 4, Np = (N + 3) / 4 * 4;
    *ae = (size_t)K * Mp; *be = (size_t)K * Np; *ce = (size_t)M * Np;
    *lda = Mp; *ldb = Np; *ldc = Np;
}

template <bool CONV>
inline int launch(Params& p, void* ws, size_t ws_bytes, hipStream_t s) {
    static int rc = (int)hipFuncSetAttribute((const void*)helix_sgemm_f32_kernel<CONV>,
                                             hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
    if (rc) return rc;
    const long long ntiles = (long long)p.tiles_m * p.tiles_n;
    if (ntiles > 0x7fffffffLL) return HELIX_ERR_INVALID_VALUE;
    p.splits = split_factor(p.M, p.N, p.K);
    if (p.splits > 1 && (!ws || ((uintptr_t)ws & 3) || ws_bytes < workspace_bytes(p.M, p.N, p.K))) p.splits = 1;
    const int ktiles = (p.K + BK - 1) / BK;
    p.k_per = ((ktiles + p.splits - 1) / p.splits) * BK;
    p.ws = (float*)ws;
    // partitions added inside the launch where that is available (one-dimensional grid), else by the second kernel
    p.plan = helix_splitk::Plan{0, 0u, nullptr};
    const unsigned fused = KG == 1 ? helix_splitk::plan_launch(p.plan, ntiles, p.splits, p.M, p.N) : 0u;
    const dim3 grid = fused ? dim3(fused, 1, 1) : dim3((unsigned)ntiles, (unsigned)p.splits, 1);
    hipLaunchKernelGGL(helix_sgemm_f32_kernel<CONV>, grid, dim3(NTHREADS), LDS_BYTES, s, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    if (p.splits > 1 && !fused) {
        const size_t total = (size_t)p.M * p.N;
        int blocks = (int)((total + 255) / 256);
        if (blocks > 8192) blocks = 8192;
        hipLaunchKernelGGL(helix_sgemm_splitk_reduce_kernel, dim3(blocks), dim3(256), 0, s, (const float*)ws, p.C, p.M,
                           p.N, p.ldc, p.splits);
        e = hipGetLastError();
    }
    return (int)e;
}

inline int gemm(const void* A, const void* B, void* C, int M, int N, int K, int lda, int ldb, int ldc, void* ws,
                size_t ws_bytes, hipStream_t s) {
    if (lda % 4 != 0 || ldb % 4 != 0) return HELIX_ERR_INVALID_VALUE;  // 16-byte loads along M and N
    if (lda < M || ldb < N || ldc < N) return HELIX_ERR_INVALID_VALUE;
    if (((uintptr_t)A & 15) || ((uintptr_t)B & 15) || ((uintptr_t)C & 3)) return HELIX_ERR_INVALID_VALUE;
    // byte offsets inside one K tile are 32-bit, and a buffer descriptor spans at most 4 GiB
    if ((long long)K * lda * 4 >= 0xffffffffLL || (long long)K * ldb * 4 >= 0xffffffffLL)
        return HELIX_ERR_INVALID_VALUE;
    if ((long long)BK * lda * 4 >= 0x7fffffffLL || (long long)BK * ldb * 4 >= 0x7fffffffLL)
        return HELIX_ERR_INVALID_VALUE;
    Params p{};
    p.A = (const float*)A; p.B = (const float*)B; p.C = (float*)C;
    p.M = M; p.N = N; p.K = K; p.lda = lda; p.ldb = ldb; p.ldc = ldc;
    p.tiles_m = (M + BM - 1) / BM; p.tiles_n = (N + BN - 1) / BN;
    return launch<false>(p, ws, ws_bytes, s);
}

// Convolutions whose channel count is not a multiple of 4 run on channel-padded copies of activations and
// weights in the workspace, or (IC = 1, where padding would quadruple the work) through a column buffer (K x M,
// the A layout of this template) and transposed weights (K x N) there, then through the GEMM above.
inline size_t conv_workspace_bytes(int batch, int H, int W, int IC, int OC, int kH, int kW, int stride, int pad) {
    const int OH = (H + 2 * pad - kH) / stride + 1, OW = (W + 2 * pad - kW) / stride + 1;
    const long long M = (long long)batch * OH * OW, K = (long long)kH * kW * IC;
    if (M > 0x7fffffffLL || K > 0x7fffffffLL) return 0;
    if (IC % 4 == 0) return workspace_bytes((int)M, OC, (int)K);
    if (helix_im2col::pads_channels(batch, H, W, IC, 4, 4)) {
        const int ICp = helix_im2col::padded_channels(IC, 4);
        return helix_im2col::align256((size_t)batch * H * W * ICp * 4) +
               helix_im2col::align256((size_t)OC * kH * kW * ICp * 4) + workspace_bytes((int)M, OC, ICp * kH * kW);
    }
    const long long Mp = (M + 3) / 4 * 4, Np = (OC + 3) / 4 * 4;
    return helix_im2col::align256((size_t)K * Mp * 4) + helix_im2col::align256((size_t)K * Np * 4) +
           workspace_bytes((int)M, OC, (int)K);
}

inline int conv2d(const void* x, const void* w, void* y, int batch, int H, int W, int IC, int OC, int kH, int kW,
                  int stride, int pad, void* ws, size_t ws_bytes, hipStream_t s);

inline int conv2d_padded_channels(const void* x, const void* w, void* y, int batch, int H, int W, int IC, int OC,
                                  int kH, int kW, int stride, int pad, void* ws, size_t ws_bytes, hipStream_t s) {
    const int ICp = helix_im2col::padded_channels(IC, 4);
    const long long pixels = (long long)batch * H * W, taps = (long long)OC * kH * kW;
    if (taps * (ICp / 4) > 0x7fffffffLL) return HELIX_ERR_INVALID_VALUE;
    const size_t xp_bytes = helix_im2col::align256((size_t)pixels * ICp * 4);
    const size_t wp_bytes = helix_im2col::align256((size_t)taps * ICp * 4);
    if (!ws || ws_bytes < conv_workspace_bytes(batch, H, W, IC, OC, kH, kW, stride, pad)) return HELIX_ERR_WORKSPACE;
    if ((uintptr_t)ws & 15) return HELIX_ERR_INVALID_VALUE;
    float* xp = (float*)ws;
    float* wp = (float*)((unsigned char*)ws + xp_bytes);
    const helix_fastdiv::FastDiv by_chunks = helix_fastdiv::make(ICp / 4);
    hipLaunchKernelGGL((helix_im2col::pad_channels_kernel<float, 4>),
                       dim3(helix_im2col::grid_for((size_t)pixels * (ICp / 4))), dim3(256), 0, s, (const float*)x, xp,
                       (int)pixels, IC, ICp, by_chunks);
    hipLaunchKernelGGL((helix_im2col::pad_channels_kernel<float, 4>),
                       dim3(helix_im2col::grid_for((size_t)taps * (ICp / 4))), dim3(256), 0, s, (const float*)w, wp,
                       (int)taps, IC, ICp, by_chunks);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    return conv2d(xp, wp, y, batch, H, W, ICp, OC, kH, kW, stride, pad, (unsigned char*)ws + xp_bytes + wp_bytes,
                  ws_bytes - xp_bytes - wp_bytes, s);
}

inline int conv2d_explicit(const void* x, const void* w, void* y, int batch, int H, int W, int IC, int OC, int kH,
                           int kW, int stride, int pad, void* ws, size_t ws_bytes, hipStream_t s) {
    const int OH = (H + 2 * pad - kH) / stride + 1, OW = (W + 2 * pad - kW) / stride + 1;
    const long long M = (long long)batch * OH * OW, K = (long long)kH * kW * IC;
    if (M > 0x7fffffffLL - 4 || K > 0x7fffffffLL) return HELIX_ERR_INVALID_VALUE;
    const int Mp = (int)((M + 3) / 4 * 4), Np = (OC + 3) / 4 * 4;
    const size_t col_bytes = helix_im2col::align256((size_t)K * Mp * 4);
    if (!ws || ws_bytes < conv_workspace_bytes(batch, H, W, IC, OC, kH, kW, stride, pad)) return HELIX_ERR_WORKSPACE;
    float* col = (float*)ws;
    float* wt = (float*)((unsigned char*)ws + col_bytes);
    const helix_im2col::Geom g = helix_im2col::make_geom(H, W, IC, OH, OW, kW, stride, pad, (int)M, (int)K);
    hipLaunchKernelGGL((helix_im2col::im2col_cols_kernel<float>),
                       dim3(helix_im2col::grid_for((size_t)Mp), (unsigned)(K < 65535 ? K : 65535)), dim3(256), 0, s,
                       (const float*)x, col, g, Mp);
    hipLaunchKernelGGL((helix_im2col::pack_weights_cols_kernel<float>), dim3(helix_im2col::grid_for((size_t)K * Np)),
                       dim3(256), 0, s, (const float*)w, wt, OC, (int)K, Np);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    const size_t used = col_bytes + helix_im2col::align256((size_t)K * Np * 4);
    return gemm(col, wt, y, (int)M, OC, (int)K, Mp, Np, OC, (unsigned char*)ws + used, ws_bytes - used, s);
}

inline int conv2d(const void* x, const void* w, void* y, int batch, int H, int W, int IC, int OC, int kH, int kW,
                  int stride, int pad, void* ws, size_t ws_bytes, hipStream_t s) {
    if (((uintptr_t)x & 15) || ((uintptr_t)w & 15) || ((uintptr_t)y & 3)) return HELIX_ERR_INVALID_VALUE;
    if (IC % 4 != 0) {   // a 16-byte chunk of the implicit gather must stay inside one filter tap
        if (helix_im2col::pads_channels(batch, H, W, IC, 4, 4))
            return conv2d_padded_channels(x, w, y, batch, H, W, IC, OC, kH, kW, stride, pad, ws, ws_bytes, s);
        return conv2d_explicit(x, w, y, batch, H, W, IC, OC, kH, kW, stride, pad, ws, ws_bytes, s);
    }
    const int OH = (H + 2 * pad - kH) / stride + 1, OW = (W + 2 * pad - kW) / stride + 1;
    const long long M = (long long)batch * OH * OW, K = (long long)kH * kW * IC;
    const long long xbytes = (long long)batch * H * W * IC * 4;
    if (M > 0x7fffffffLL || K > 0x7fffffffLL || xbytes >= 0x7fffffffLL) return HELIX_ERR_INVALID_VALUE;
    if ((long long)BN * K * 4 >= 0x7fffffffLL) return HELIX_ERR_INVALID_VALUE;
    Params p{};
    p.A = (const float*)x; p.B = (const float*)w; p.C = (float*)y;
    p.M = (int)M; p.N = OC; p.K = (int)K; p.lda = 0; p.ldb = (int)K; p.ldc = OC;
    p.tiles_m = (int)((M + BM - 1) / BM); p.tiles_n = (OC + BN - 1) / BN;
    p.a_bytes = (unsigned)xbytes;
    p.g = ConvGeom{H, W, IC, OH, OW, kW, stride, pad, (int)M,
                   helix_fastdiv::make(OW), helix_fastdiv::make(OH), helix_fastdiv::make(IC), helix_fastdiv::make(kW)};
    return launch<true>(p, ws, ws_bytes, s);
}

}  // namespace tpl

#include "helix_host.h"
