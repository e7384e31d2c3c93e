// MI355X (gfx950 / CDNA4) FP16 GEMM template with direct-to-LDS copies and a two-group wave schedule.
//
//   C[M x N] = A[M x K] * B[N x K]^T          FP16 in, FP32 accumulate (MFMA), FP16 out
//
// Role in the reference: the deeper-pipelined points of src_template/Ampere_FP16/gemm.cu (K_STAGE = 3 .. 5: a ring
// of cp.async stages, :156-198, :239-394).  Same operand layouts, tile parameters, workgroup -> tile mapping,
// epilogue and split-K as gemm.hip (shared through gemm_tile.h); what differs is how a K tile travels and how the
// waves divide the work:
//   * global memory -> LDS without passing through registers (buffer_load ... lds: one wave-wide instruction
//     writes 1 KiB of consecutive LDS), into a ring of K_STAGES stages of BLOCK_K (32, 64 or 128) columns;
//   * a workgroup is eight waves, normally two on each SIMD.  On arrival each wave takes a ticket per SIMD: the first
//     wave of a SIMD joins group 0, the second group 1 (if the waves are not spread two per SIMD, groups and copy
//     quarters are dealt by wave index instead).  A wave alternates between two phases per K tile,
//       M(t): read its fragments of tile t (the whole tile: KSTEPS x (TM + TN) ds_read_b128) into registers,
//       C(t): KSTEPS x TM x TN MFMAs on those registers, nothing else,
//     with a workgroup barrier behind every phase, and group 1 runs one phase behind group 0.  So on every SIMD
//     one wave issues an unbroken run of MFMAs on operands that are already in registers while the other one
//     absorbs the latency of LDS and of global memory; the matrix pipe idles only across the barriers.
//   * group 0 also feeds the ring: in M(t), before its reads, each of its four waves issues the copies of its
//     quarter of tile t + K_STAGES - 1 into the stage tile t - 1 occupied (every wave was done reading that one
//     at the barrier two phases earlier), and at the end of C(t) it waits until tile t + 1 has landed, so the
//     barrier behind C(t) publishes tile t + 1 to both groups.  A copy has K_STAGES - 1 K tiles to land.
// Measured on 8192^3 (256 x 256 tile): with nothing to copy the two-group schedule runs a 64-column K tile in 2190
// cycles where the MFMAs alone need 2048; a burst of 64 KiB of copies per compute unit takes 1.4 us to land.  Two
// 64-column stages measure fastest for that tile; rings of three or four 32-column stages (two or three tiles in
// flight, but twice the barriers per K) are about 10 % slower there and are built for the smaller tiles.
//
// LDS layout: rows of 128 bytes (256 for BLOCK_K = 128); 16-byte chunk c of LDS row r sits at chunk position
// c ^ key(r), key(r) = (r / rows_per_256B) mod chunks_per_row, the layout gemm.hip reads without bank conflicts.
// With BLOCK_K = 32 a matrix row fills only half an LDS row, so matrix rows r and r + 8 of every block of 16 rows
// share LDS row (r / 16) * 8 + r % 8 -- chunks 0..3 hold the first, 4..7 the second: the 16 rows of an MFMA
// fragment then spread over the 16 bank groups exactly as they do with 64-column tiles.
//
// No convolution entry: helix_conv2d of such a library returns HELIX_ERR_UNSUPPORTED (the gather of an implicit
// GEMM lives in gemm.hip).
#include "gemm_tile.h"

namespace {

constexpr bool PAIRED = (BK == 32);                 // two matrix rows per LDS row
constexpr int LROW_BYTES = BK == 128 ? 256 : 128;   // LDS row
constexpr int LCH = LROW_BYTES / 16;                // chunk positions per LDS row (8 or 16)
constexpr int LRP = 256 / LROW_BYTES;               // LDS rows per 256 bytes (2 or 1)
constexpr int MPL = PAIRED ? 2 : 1;                 // matrix rows per LDS row
constexpr int RING = STAGES;                        // stages of the ring
constexpr int RING_BYTES = RING * STAGE_BYTES;
constexpr int ROLE_BYTES = 64;                      // four ticket counters behind the ring (one per SIMD)
constexpr int LDS_BYTES = (RING_BYTES > NWAVES * STRIP_BYTES ? RING_BYTES : NWAVES * STRIP_BYTES) + ROLE_BYTES;
constexpr int DMA_BYTES = 1024;                     // one wave-wide 16-byte-per-lane copy fills 1 KiB of LDS
constexpr int LRPI = DMA_BYTES / LROW_BYTES;        // LDS rows per copy instruction (8 or 4)
constexpr int MRPI = LRPI * MPL;                    // matrix rows per copy instruction (16, 8 or 4)
constexpr int DMA_A = (BM / 4) / MRPI, DMA_B = (BN / 4) / MRPI;   // copy instructions per K tile of a copying wave
constexpr int NDMA = DMA_A + DMA_B;
constexpr int KEY_PERIOD = LRP * LCH;               // LDS rows after which the swizzle key repeats (16)
constexpr int NVOFF = KEY_PERIOD / LRPI;            // distinct per-lane offsets among a wave's copies (2 or 4)
constexpr int PERIOD_MROWS = KEY_PERIOD * MPL;      // matrix rows per key period

static_assert(BK == 32 || BK == 64 || BK == 128, "BLOCK_K: 32, 64 or 128");
static_assert(RING >= 2 && RING <= 5, "K_STAGES: a ring of 2 to 5 stages");
static_assert(NWAVES == 8, "eight waves: two per SIMD, one of each group");
static_assert((BM / 4) % MRPI == 0 && (BN / 4) % MRPI == 0 && DMA_A >= 1 && DMA_B >= 1,
              "each of the four copying waves fills whole 1 KiB pieces of a stage");
static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of a gfx950 CU exceeded");
static_assert(KSTEPS * (TM + TN) * 4 + TM * TN * 4 <= 236,
              "accumulators and a whole K tile of fragments live in 256 registers");
static_assert((RING - 2) * NDMA <= 63, "copies in flight are counted in a 6-bit counter");

__device__ __forceinline__ int lds_key(int lrow) { return (lrow / LRP) & (LCH - 1); }

// 128-bit buffer descriptor as four dwords: base address (48 bits), stride 0, byte count, raw-buffer flags
__device__ __forceinline__ intx4 raw_rsrc(const void* base, unsigned bytes) {
    const unsigned long long a = (unsigned long long)base;
    intx4 r = {(int)(unsigned)a, (int)((a >> 32) & 0xffffu), (int)bytes, 0x00020000};
    return r;
}

// One 16-byte-per-lane direct-to-LDS buffer load: lane l's data lands at LDS byte lds_addr + 16 * l (lds_addr is
// wave-uniform and goes through M0); voff is the lane's byte offset into the buffer, out-of-range lanes store
// zeros.  Issued from inline assembly so that the compiler neither orders LDS reads behind it nor counts it in its
// own s_waitcnt bookkeeping: completion is tracked by hand (wait_vmcnt) in front of the barrier that publishes it.
// sc1: a tile is read once per compute unit, so the copy goes past the CU's vector cache to L2 (measured: +2 %).
__device__ __forceinline__ void dma16(intx4 rsrc, unsigned lds_addr, int voff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen sc1 lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(rsrc)
                 : "memory", "m0");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {   // s_waitcnt vmcnt(N), other counters untouched
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}
// at most `tiles` K tiles' worth of this wave's copies still in flight
__device__ __forceinline__ void wait_copies(int tiles) {
    if (RING >= 5 && tiles >= 3) wait_vmcnt<(RING >= 5 ? 3 : 0) * NDMA>();
    else if (RING >= 4 && tiles == 2) wait_vmcnt<(RING >= 4 ? 2 : 0) * NDMA>();
    else if (RING >= 3 && tiles == 1) wait_vmcnt<(RING >= 3 ? 1 : 0) * NDMA>();
    else wait_vmcnt<0>();
}
__device__ __forceinline__ void wait_lgkmcnt0() { __builtin_amdgcn_s_waitcnt(15 | (7 << 4) | (0 << 8) | (3 << 14)); }

__device__ __forceinline__ void phase_barrier() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
}

typedef __attribute__((address_space(3))) unsigned char* lds_ptr_t;

// The tile parameters appear as (otherwise unused) template arguments so that every configuration's kernel has
// its own symbol name and a profiler lists configurations separately.
template <int T_STAGES = STAGES, int T_BM = BM, int T_BN = BN, int T_WM = WM, int T_WN = WN, int T_BK = BK,
          int T_SPLITK = SPLITK>
__global__ __launch_bounds__(NTHREADS) void helix_gemm_f16_dtl_kernel(const Params p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
    const TileRange tr = tile_range_of_workgroup(p);
    const int m0 = tr.m0, n0 = tr.n0, k_begin = tr.k_begin, k_end = tr.k_end;

    // ---- groups: one ticket counter per SIMD ------------------------------------------------------------------
    int* role = (int*)(smem + LDS_BYTES - ROLE_BYTES);
    if (tid < 4) role[tid] = 0;
    __syncthreads();
    // HW_REG_HW_ID (register 4), SIMD_ID = bits 5:4
    const int hw_simd = __builtin_amdgcn_s_getreg((2 - 1) << 11 | 4 << 6 | 4) & 3;
    int ticket = 0;
    if (lane == 0) ticket = atomicAdd(&role[hw_simd], 1);
    __syncthreads();
    // The dispatcher usually places two of the eight waves on each SIMD, and then the tickets give every SIMD one
    // wave of each group.  Nothing guarantees that placement (small tiles share a compute unit with other
    // workgroups): when the counts are not 2 / 2 / 2 / 2 the groups and the copy quarters are dealt by wave index
    // instead, which is correct under any placement (the two waves of a SIMD may then be in the same phase).
    const bool two_per_simd = role[0] == 2 && role[1] == 2 && role[2] == 2 && role[3] == 2;
    // wave-uniform values, kept in scalar registers (lane 0 holds the ticket)
    const int grp = __builtin_amdgcn_readfirstlane(two_per_simd ? (ticket & 1) : (wave & 1));
    // the quarter of every stage a group-0 wave copies
    const int simd = __builtin_amdgcn_readfirstlane(two_per_simd ? hw_simd : (wave >> 1));

    // ---- copy geometry of a group-0 wave: quarter `simd` of the A rows and of the B rows of every stage ----------
    // Copy instruction j fills LRPI consecutive LDS rows (1 KiB) from LDS row q / MPL + j * LRPI on; lane l lands at
    // byte 16 * l of that piece: LDS row + l / LCH, chunk position l % LCH, which holds chunk
    // (l % LCH) ^ key(LDS row) -- with paired rows, chunk = 4 * (second row of the pair) + the row's own 16-byte
    // chunk.  The key repeats every KEY_PERIOD LDS rows, so NVOFF per-lane offsets serve all j.
    const int qa0 = simd * (BM / 4), qb0 = simd * (BN / 4);
    const int rows_a = (p.M - m0) < BM ? (p.M - m0) : BM;
    const int rows_b = (p.N - n0) < BN ? (p.N - n0) : BN;
    const half_t* baseA = p.A + (size_t)m0 * p.lda;
    const half_t* baseB = p.B + (size_t)n0 * p.ldb;
    const unsigned bytesA = (unsigned)(((size_t)(rows_a - 1) * p.lda + p.K) * 2);
    const unsigned bytesB = (unsigned)(((size_t)(rows_b - 1) * p.ldb + p.K) * 2);
    int voff_a[NVOFF], voff_b[NVOFF], gch_a[NVOFF], gch_b[NVOFF];
    auto lane_source = [&](int q0, int jj, int ld, int* gch) -> int {
        const int lrow = q0 / MPL + jj * LRPI + lane / LCH;
        const int chunk = (lane % LCH) ^ lds_key(lrow);
        int mrow = lrow, kch = chunk;
        if (PAIRED) {
            mrow = (lrow / 8) * 16 + (chunk >> 2) * 8 + (lrow & 7);
            kch = chunk & 3;
        }
        *gch = kch;
        return (mrow * ld + kch * 8) * 2;
    };
#pragma unroll
    for (int jj = 0; jj < NVOFF; jj++) {
        voff_a[jj] = lane_source(qa0, jj, p.lda, &gch_a[jj]);
        voff_b[jj] = lane_source(qb0, jj, p.ldb, &gch_b[jj]);
    }
    const int period_a = PERIOD_MROWS * p.lda * 2, period_b = PERIOD_MROWS * p.ldb * 2;   // bytes per key period
    const unsigned lds_base = (unsigned)(uintptr_t)(lds_ptr_t)smem;
    const unsigned lds_a = lds_base + (unsigned)(qa0 * BK * 2);
    const unsigned lds_b = lds_base + (unsigned)(A_STAGE_BYTES + qb0 * BK * 2);

    // K tiles: when the K range is not a multiple of BLOCK_K the narrow tile comes first (tile 0 covers `first_w`
    // columns, every later tile BLOCK_K), so that only the prologue's copies need a column mask
    const int ktiles = (k_end - k_begin + BK - 1) / BK;
    const int first_w = ((k_end - k_begin) % BK) ? ((k_end - k_begin) % BK) : BK;
    auto tile_k0 = [&](int t) -> int { return t == 0 ? k_begin : k_begin + first_w + (t - 1) * BK; };

    auto copy_tile = [&](int t, int stage, bool narrow) {
        const int k0 = tile_k0(t);
        const intx4 ra = raw_rsrc(baseA + k0, bytesA - (unsigned)k0 * 2u);
        const intx4 rb = raw_rsrc(baseB + k0, bytesB - (unsigned)k0 * 2u);
        const unsigned sa = lds_a + (unsigned)(stage * STAGE_BYTES), sb = lds_b + (unsigned)(stage * STAGE_BYTES);
#pragma unroll
        for (int j = 0; j < (DMA_A > DMA_B ? DMA_A : DMA_B); j++) {
            if (j < DMA_A) {
                int off = voff_a[j % NVOFF] + (j / NVOFF) * period_a;
                if (narrow && gch_a[j % NVOFF] * 8 >= first_w) off = OOB_OFFSET;
                dma16(ra, sa + (unsigned)(j * DMA_BYTES), off);
            }
            if (j < DMA_B) {
                int off = voff_b[j % NVOFF] + (j / NVOFF) * period_b;
                if (narrow && gch_b[j % NVOFF] * 8 >= first_w) off = OOB_OFFSET;
                dma16(rb, sb + (unsigned)(j * DMA_BYTES), off);
            }
        }
    };

    // ---- fragment read geometry -----------------------------------------------------------------
    // MFMA 16x16x32: lane l supplies row (l % 16), k = 8 * (l / 16) .. +7 of both operands, i.e. 16-byte chunk
    // 4 * s + l / 16 of its row for k-step s.
    const int frow = lane & 15, fq = lane >> 4;
    auto frag_addr = [&](int row0, int s) -> int {     // row0: first matrix row of the 16-row fragment
        int lrow, chunk;
        if (PAIRED) {
            lrow = row0 / 2 + (frow & 7);
            chunk = (frow >> 3) * 4 + fq;
        } else {
            lrow = row0 + frow;
            chunk = s * 4 + fq;
        }
        return lrow * LROW_BYTES + ((chunk ^ lds_key(lrow)) << 4);
    };
    auto read_a = [&](const unsigned char* sb, int s, int i) -> half8 {
        return *(const half8*)(sb + frag_addr(wave_m * WM + i * 16, s));
    };
    auto read_b = [&](const unsigned char* sb, int s, int j) -> half8 {
        return *(const half8*)(sb + A_STAGE_BYTES + frag_addr(wave_n * WN + j * 16, s));
    };

    floatx4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
    half8 fa[KSTEPS][TM], fb[KSTEPS][TN];

    // ---- prologue: tiles 0 .. RING-2 on their way, tile 0 landed and published -----------------------------------
    if (grp == 0) {
#pragma unroll
        for (int h = 0; h < RING - 1; h++)
            if (h < ktiles) copy_tile(h, h, h == 0);
        const int after = ktiles - 1 < RING - 2 ? ktiles - 1 : RING - 2;   // tiles issued behind tile 0
        wait_copies(after);
    }
    phase_barrier();
    if (grp == 1) phase_barrier();   // group 1 runs one phase behind

    int stage = 0;                   // ring stage of tile t
    for (int t = 0; t < ktiles; t++) {
        // ---- M(t) ----
        int stage_in = stage + RING - 1;
        if (stage_in >= RING) stage_in -= RING;
        if (grp == 0 && t + RING - 1 < ktiles) copy_tile(t + RING - 1, stage_in, false);
        const unsigned char* sb = smem + stage * STAGE_BYTES;
#pragma unroll
        for (int s = 0; s < KSTEPS; s++) {
#pragma unroll
            for (int i = 0; i < TM; i++) fa[s][i] = read_a(sb, s, i);
#pragma unroll
            for (int j = 0; j < TN; j++) fb[s][j] = read_b(sb, s, j);
        }
        wait_lgkmcnt0();             // this wave is done with the stage before it arrives at the barrier
        phase_barrier();
        // ---- C(t) ----
        // the B fragment goes first, which leaves the transposed 16 x 16 block in the accumulator (see store_tile)
#pragma unroll
        for (int s = 0; s < KSTEPS; s++)
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[s][j], fa[s][i], acc[i][j], 0, 0, 0);
        if (grp == 0) {              // tile t + 1 must have landed; the tiles issued behind it may still be in flight
            int after = ktiles - 2 - t;
            if (after > RING - 2) after = RING - 2;
            wait_copies(after < 0 ? 0 : after);
        }
        phase_barrier();
        stage = stage + 1 == RING ? 0 : stage + 1;
    }
    if (grp == 0) phase_barrier();   // the barrier group 1 passes behind its last phase

    store_tile<LDS_BYTES>(acc, p, tr, tid, wave, wave_m, wave_n, lane, smem);
}

}  // namespace

// -------------------------------------------------------------------------------------------------
// host side
// -------------------------------------------------------------------------------------------------
#include <stdio.h>

namespace tpl {

inline const char* info_json() {
    static char buf[1024];
    static bool done = false;
    if (!done) {
        snprintf(buf, sizeof(buf),
                 "{\"family\": \"gemm_f16\", \"arch\": \"gfx950\", \"mfma\": \"v_mfma_f32_16x16x32_f16\", "
                 "\"k_stages\": %d, \"block_rows\": %d, \"block_cols\": %d, \"wave_rows\": %d, \"wave_cols\": %d, "
                 "\"block_k\": %d, \"split_k\": %d, \"direct_to_lds\": %d, \"threads\": %d, \"lds_bytes\": %d, "
                 "\"layout_a\": \"M x K row-major f16\", \"layout_b\": \"N x K row-major f16\", "
                 "\"layout_c\": \"M x N row-major f16\", \"accumulate\": \"f32\", "
                 "\"k_multiple\": 8, \"ld_multiple\": 8, \"conv\": \"unsupported\"}",
                 STAGES, BM, BN, WM, WN, BK, SPLITK, 1, NTHREADS, LDS_BYTES);
        done = true;
    }
    return buf;
}

inline int set_lds_attr() {
    static int rc = (int)hipFuncSetAttribute((const void*)helix_gemm_f16_dtl_kernel<>,
                                             hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
    return rc;
}

inline int gemm(const void* A, const void* B, void* C, int M, int N, int K, int lda, int ldb, int ldc, void* ws,
                size_t ws_bytes, hipStream_t s) {
    if (K % 8 != 0 || lda % 8 != 0 || ldb % 8 != 0) return HELIX_ERR_INVALID_VALUE;
    if (lda < K || ldb < K || ldc < N) return HELIX_ERR_INVALID_VALUE;
    if (((uintptr_t)A & 15) || ((uintptr_t)B & 15) || ((uintptr_t)C & 1)) return HELIX_ERR_INVALID_VALUE;
    // per-tile byte offsets are 32-bit
    if ((long long)BM * lda * 2 >= 0x7fffffffLL || (long long)BN * ldb * 2 >= 0x7fffffffLL)
        return HELIX_ERR_INVALID_VALUE;
    Params p{};
    p.A = (const half_t*)A; p.B = (const half_t*)B; p.C = (half_t*)C; p.ws = (float*)ws;
    p.M = M; p.N = N; p.K = K; p.lda = lda; p.ldb = ldb; p.ldc = ldc;
    p.tiles_m = (M + BM - 1) / BM; p.tiles_n = (N + BN - 1) / BN;
    p.splits = split_factor(M, N, K);
    if (SPLITK > 1) {
        if (!ws || ws_bytes < workspace_bytes(M, N, K)) return HELIX_ERR_WORKSPACE;
    }
    int rc = set_lds_attr();
    if (rc) return rc;
    const long long ntiles = (long long)p.tiles_m * p.tiles_n;
    if (ntiles > 0x7fffffffLL) return HELIX_ERR_INVALID_VALUE;
    const dim3 grid = launch_grid(p), block(NTHREADS, 1, 1);   // K partitions added inside the launch where available
    hipLaunchKernelGGL(helix_gemm_f16_dtl_kernel<>, grid, block, LDS_BYTES, s, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    if (SPLITK > 1 && !p.plan.fused) {
        size_t total = (size_t)M * N;
        int blocks = (int)((total + 255) / 256);
        if (blocks > 8192) blocks = 8192;
        hipLaunchKernelGGL(helix_splitk_reduce_kernel, dim3(blocks), dim3(256), 0, s, (const float*)ws, p.C, M, N, ldc,
                           p.splits);
        e = hipGetLastError();
        if (e != hipSuccess) return (int)e;
    }
    return 0;
}

inline size_t conv_workspace_bytes(int, int, int, int, int, int, int, int, int) { return 0; }

inline int conv2d(const void*, const void*, void*, int, int, int, int, int, int, int, int, int, void*, size_t,
                  hipStream_t) {
    return HELIX_ERR_UNSUPPORTED;
}

}  // namespace tpl

#if SPLIT_K == 1
#define HELIX_TPL_SCRATCH_BYTES 256   // no K partition: this library never asks for a workspace
#endif
#include "helix_host.h"
