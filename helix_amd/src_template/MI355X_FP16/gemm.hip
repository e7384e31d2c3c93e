// MI355X (gfx950 / CDNA4) FP16 GEMM + implicit-GEMM convolution template.
//
//   GEMM : C[M x N] = A[M x K] * B[N x K]^T          FP16 in, FP32 accumulate (MFMA), FP16 out
//   CONV : y[B,OH,OW,OC] = conv2d(x[B,H,W,IC], w[OC,kH,kW,IC])  == the same GEMM with
//          M = B*OH*OW, N = OC, K = kH*kW*IC, where the A tile is gathered from x on the fly.
//
// Role in the reference: this file stands where src_template/Ampere_FP16/gemm.cu (tensor-core HGEMM,
// :120-534), gemm_splitK.cu (:120-509) and the im2col.cu + GEMM pair (im2col.cu:38-97) stand.  The
// operand layout (B stored N x K) follows gemm.cu:144,597-601; unlike the reference's
// `mma...f16.f16.f16.f16` (gemm.cu:54-57) accumulation is FP32.
//
// Compile-time parameters (set with -D by the build script, one shared library per combination):
//   BLOCK_ROWS x BLOCK_COLS   workgroup tile of C           (reference BLOCK_ROWS / BLOCK_COLS)
//   WAVE_ROWS  x WAVE_COLS    tile of C owned by one wave64 (reference WARP_ROWS / WARP_COLS)
//   BLOCK_K                   K extent of one LDS stage
//   LDS_STAGES                LDS ring depth                (reference K_STAGE)
//   SPLIT_K                   1: each workgroup walks all of K.  > 1: K is partitioned over blockIdx.y into
//                             2 .. SPLIT_K ranges, as many as it takes to give every compute unit a
//                             workgroup (FP32 workspace + fixed-order reduction kernel)
//
// Kernel structure
//   * one wave64 computes (WAVE_ROWS/32) x (WAVE_COLS/32) v_mfma_f32_32x32x16_f16 tiles; per 16-wide
//     k step it reads one 16-byte fragment per 32 rows of A and of B from LDS (ds_read_b128).
//   * global -> LDS uses gfx950's 128-bit direct-to-LDS buffer loads (DIRECT_TO_LDS=1, default): no
//     staging registers, no ds_write; hardware bounds checking zero-fills rows beyond M / N and the K
//     tail.  The copy of tile t+1 is issued after tile t's fragments are read and lands while tile t's
//     MFMAs run; one wait + barrier per tile.  DIRECT_TO_LDS=0 keeps the register-staged variant
//     (buffer_load -> VGPR -> ds_write_b128).
//   * LDS rows are BLOCK_K halves; 16-byte chunk c of row r is stored at chunk (c ^ key(r)), with
//     key(r) = (r / rows_per_256B) mod chunks_per_row, so that 16 consecutive rows of one chunk column
//     land in 16 different 16-byte bank groups (64 banks x 4 B): fragment reads and tile writes are
//     both conflict-free.
//   * workgroup id -> tile: ids are dealt round-robin to the 8 XCDs by the hardware, so id is first
//     remapped to (xcd, slot) -> xcd * ids_per_xcd + slot, then walked in column-major groups of
//     GROUP_ROWS tile rows; each XCD's L2 then sees a compact patch of tiles sharing A and B panels.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "helix_abi.h"

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
#ifndef LDS_STAGES
#define LDS_STAGES 2
#endif
#ifndef SPLIT_K
#define SPLIT_K 1
#endif
#ifndef GROUP_ROWS
#define GROUP_ROWS 8
#endif
#ifndef DIRECT_TO_LDS
#define DIRECT_TO_LDS 1
#endif

namespace {

typedef _Float16 half_t;
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef int intx4 __attribute__((ext_vector_type(4)));
typedef int intx2 __attribute__((ext_vector_type(2)));

constexpr int BM = BLOCK_ROWS, BN = BLOCK_COLS, WM = WAVE_ROWS, WN = WAVE_COLS, BK = BLOCK_K;
constexpr int STAGES = LDS_STAGES, SPLITK = SPLIT_K;
constexpr int WAVES_M = BM / WM, WAVES_N = BN / WN, NWAVES = WAVES_M * WAVES_N, NTHREADS = 64 * NWAVES;
constexpr int TM = WM / 32, TN = WN / 32;      // MFMA tiles per wave
constexpr int KCH = BK / 8;                    // 16-byte chunks per LDS row
constexpr int ROW_BYTES = BK * 2;
constexpr int RP = ROW_BYTES >= 256 ? 1 : 256 / ROW_BYTES;  // rows per 256 bytes of LDS
constexpr int A_ITERS = BM * KCH / NTHREADS, B_ITERS = BN * KCH / NTHREADS;
constexpr int ROWS_PER_ITER = NTHREADS / KCH;
constexpr int A_STAGE_BYTES = BM * ROW_BYTES, B_STAGE_BYTES = BN * ROW_BYTES;
constexpr int STAGE_BYTES = A_STAGE_BYTES + B_STAGE_BYTES;
constexpr int RING_BYTES = STAGES * STAGE_BYTES;
// epilogue staging: one 32 x WAVE_COLS strip of halves per wave, rows padded by 16 bytes
constexpr int STRIP_LD = WN * 2 + 16;
constexpr int STRIP_BYTES = 32 * STRIP_LD;
constexpr int LDS_BYTES = RING_BYTES > NWAVES * STRIP_BYTES ? RING_BYTES : NWAVES * STRIP_BYTES;

static_assert(BM % WM == 0 && BN % WN == 0, "block tile must be a multiple of the wave tile");
static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile is built from 32x32 MFMA tiles");
static_assert(BK % 16 == 0 && (KCH & (KCH - 1)) == 0 && KCH >= 2, "BLOCK_K must be 16 * 2^n");
static_assert(NTHREADS <= 1024 && NTHREADS % KCH == 0, "bad thread count");
static_assert((BM * KCH) % NTHREADS == 0 && (BN * KCH) % NTHREADS == 0, "tile copy must divide evenly");
#if DIRECT_TO_LDS
static_assert(STAGES >= 2 && STAGES <= 4, "LDS ring depth must be 2..4");
static_assert((BK / 16) % 2 == 0, "BLOCK_K must hold an even number of 16-wide MFMA k-steps");
static_assert((STAGES - 1) * (A_ITERS + B_ITERS) <= 63, "too many copy instructions in flight for vmcnt");
#else
static_assert(STAGES == 2, "the register-staged variant implements the two-stage ring only");
#endif
static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of a gfx950 CU exceeded");
static_assert(SPLITK >= 1 && SPLITK <= 8, "SPLIT_K out of range");

struct ConvGeom {
    int H, W, IC, OH, OW, kW, stride, pad, M;  // M = batch*OH*OW
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
    ConvGeom g;
};

__device__ __forceinline__ int swz_key(int row) { return (row / RP) & (KCH - 1); }

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

constexpr int OOB_OFFSET = 0x7fffffff;  // byte offset beyond any buffer: the load returns zeros
constexpr int KSTEPS = BK / 16;         // MFMA k-steps per K tile
typedef __attribute__((address_space(3))) unsigned char* lds_ptr_t;

// s_waitcnt vmcnt(N): at most N buffer loads of this wave (also the direct-to-LDS ones) are still in flight
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N <= 63, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// 128-bit buffer descriptor as four dwords: base address (48 bits), stride 0, byte count, raw-buffer flags
__device__ __forceinline__ intx4 raw_rsrc(const void* base, unsigned bytes) {
    const unsigned long long a = (unsigned long long)base;
    intx4 r = {(int)(unsigned)a, (int)((a >> 32) & 0xffffu), (int)bytes, 0x00020000};
    return r;
}

// One 16-byte-per-lane direct-to-LDS buffer load: lane l's data lands at LDS byte (lds_addr + 16*l).
// lds_addr must be wave-uniform (it is moved into M0); voff is the per-lane byte offset into the buffer.
__device__ __forceinline__ void dma16(intx4 rsrc, unsigned lds_addr, int voff) {
    asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(rsrc)
                 : "memory", "m0");
}

__device__ __forceinline__ intx4 buf_load16(__amdgpu_buffer_rsrc_t r, int voff) {
    return __builtin_bit_cast(intx4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, 0, 0));
}

// The tile parameters appear as (otherwise unused) template arguments so that every configuration's
// kernel has its own symbol name and a profiler lists configurations separately.
// MODE: 0 = GEMM; 1 = convolution, general gather (tap and channel of every 16-byte chunk computed per K
// tile); 2 = convolution with IC a multiple of BLOCK_K and at most 32 filter taps: a K tile then lies inside
// one filter tap, so the tap offset is one scalar per tile and each copy slot only tests its tap-validity bit.
template <int MODE, int T_STAGES = STAGES, int T_BM = BM, int T_BN = BN, int T_WM = WM, int T_WN = WN, int T_BK = BK,
          int T_SPLITK = SPLITK>
__global__ __launch_bounds__(NTHREADS) void helix_gemm_f16_kernel(const Params p) {
    constexpr bool CONV = (MODE != 0);
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: lives in a scalar register
    const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;

    // ---- workgroup id -> (tile_m, tile_n), XCD-aware ------------------------------------------
    const int ntiles = p.tiles_m * p.tiles_n;
    int pid = blockIdx.x;
    {
        const int per = ntiles / 8, rem = ntiles % 8;
        const int xcd = pid % 8, slot = pid / 8;
        pid = xcd * per + (xcd < rem ? xcd : rem) + slot;
    }
    const int group_tiles = GROUP_ROWS * p.tiles_n;
    const int grp = pid / group_tiles;
    const int first_m = grp * GROUP_ROWS;
    const int gsize = (p.tiles_m - first_m) < GROUP_ROWS ? (p.tiles_m - first_m) : GROUP_ROWS;
    const int in_grp = pid % group_tiles;
    const int tile_m = first_m + in_grp % gsize;
    const int tile_n = in_grp / gsize;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    // ---- K range of this workgroup (split-K partitions are multiples of BLOCK_K) -----------------
    int k_begin = 0, k_end = p.K;
    if (SPLITK > 1) {
        const int ktiles = (p.K + BK - 1) / BK;
        const int per = (ktiles + p.splits - 1) / p.splits;
        k_begin = (int)blockIdx.y * per * BK;
        k_end = k_begin + per * BK;
        if (k_end > p.K) k_end = p.K;
        if (k_begin > p.K) k_begin = p.K;
    }

    // ---- per-thread copy geometry ---------------------------------------------------------------
    // Copy slot c = tid + i*NTHREADS of a tile lands at LDS byte c*16 (so one wave-wide copy instruction
    // fills 1 KiB of consecutive LDS, which is what a direct-to-LDS load requires); it holds row r = c / KCH
    // and, because of the swizzle, global chunk g = (c % KCH) ^ key(r) of that row.
    const int cpos = tid % KCH;
    const int r0 = tid / KCH;
    int gch_a[A_ITERS], gch_b[B_ITERS];    // global 16-byte chunk index within the K tile
#pragma unroll
    for (int i = 0; i < A_ITERS; i++) gch_a[i] = cpos ^ swz_key(r0 + i * ROWS_PER_ITER);
#pragma unroll
    for (int i = 0; i < B_ITERS; i++) gch_b[i] = cpos ^ swz_key(r0 + i * ROWS_PER_ITER);

    // B operand: rows n0.. of an N x K matrix
    const int rows_b = (p.N - n0) < BN ? (p.N - n0) : BN;
    const half_t* baseB = p.B + (size_t)n0 * p.ldb;
    const unsigned bytesB = (unsigned)(((size_t)(rows_b - 1) * p.ldb + p.K) * 2);
    int voff_b[B_ITERS];
#pragma unroll
    for (int i = 0; i < B_ITERS; i++) voff_b[i] = ((r0 + i * ROWS_PER_ITER) * p.ldb + gch_b[i] * 8) * 2;

    // A operand
    const half_t* baseA = nullptr;
    unsigned bytesA = 0;
    int voff_a[A_ITERS];
    int cv_img[A_ITERS], cv_ih[A_ITERS], cv_iw[A_ITERS];  // CONV: image base offset, top-left tap coords
    int cv_base[A_ITERS];                                 // MODE 2: byte offset of the row's top-left tap + chunk
    unsigned cv_taps[A_ITERS];                            // MODE 2: bit t set = filter tap t reads inside the image
    if (!CONV) {
        const int rows_a = (p.M - m0) < BM ? (p.M - m0) : BM;
        baseA = p.A + (size_t)m0 * p.lda;
        bytesA = (unsigned)(((size_t)(rows_a - 1) * p.lda + p.K) * 2);
#pragma unroll
        for (int i = 0; i < A_ITERS; i++) voff_a[i] = ((r0 + i * ROWS_PER_ITER) * p.lda + gch_a[i] * 8) * 2;
    } else {
        baseA = p.A;
        bytesA = p.a_bytes;
#pragma unroll
        for (int i = 0; i < A_ITERS; i++) {
            const int m = m0 + r0 + i * ROWS_PER_ITER;
            const int ow = m % p.g.OW;
            const int t = m / p.g.OW;
            const int oh = t % p.g.OH;
            const int b = t / p.g.OH;
            cv_img[i] = (m < p.g.M) ? b * p.g.H * p.g.W : -1;
            cv_ih[i] = oh * p.g.stride - p.g.pad;
            cv_iw[i] = ow * p.g.stride - p.g.pad;
            if (MODE == 2) {
                cv_base[i] = ((cv_img[i] + cv_ih[i] * p.g.W + cv_iw[i]) * p.g.IC + gch_a[i] * 8) * 2;
                unsigned taps = 0;
                const int ntaps = p.K / p.g.IC;
                for (int t = 0; t < ntaps; t++) {
                    const int ih = cv_ih[i] + t / p.g.kW, iw = cv_iw[i] + t % p.g.kW;
                    if (cv_img[i] >= 0 && ih >= 0 && ih < p.g.H && iw >= 0 && iw < p.g.W) taps |= 1u << t;
                }
                cv_taps[i] = taps;
            }
        }
    }

    // MODE 2: scalar state of the K tile at k0: byte offset of its filter tap and channel block, and its tap bit
    struct ConvTile { int soff; unsigned tapbit; };
    auto conv_tile = [&](int k0) -> ConvTile {
        ConvTile ct{0, 0u};
        if (MODE == 2 && k0 < p.K) {
            const int tap = k0 / p.g.IC, c0 = k0 % p.g.IC;
            ct.soff = (((tap / p.g.kW) * p.g.W + tap % p.g.kW) * p.g.IC + c0) * 2;
            ct.tapbit = 1u << tap;
        }
        return ct;
    };

    // Byte offset (relative to the operand's buffer descriptor) of copy slot i for the K tile at k0, or
    // OOB_OFFSET when the slot must read zeros (beyond K, conv padding, rows beyond M).
    auto a_offset = [&](int i, int k0, bool tail, ConvTile ct) -> int {
        if (!CONV) {
            return (tail && k0 + gch_a[i] * 8 >= p.K) ? OOB_OFFSET : voff_a[i];
        } else if (MODE == 2) {
            return (cv_taps[i] & ct.tapbit) ? cv_base[i] + ct.soff : OOB_OFFSET;
        } else {
            const int k = k0 + gch_a[i] * 8;  // k = (kh*kW + kw)*IC + c, 8 consecutive c per chunk
            const int c = k % p.g.IC;
            const int t = k / p.g.IC;
            const int kw = t % p.g.kW;
            const int kh = t / p.g.kW;
            const int ih = cv_ih[i] + kh, iw = cv_iw[i] + kw;
            const bool ok = k < p.K && cv_img[i] >= 0 && ih >= 0 && ih < p.g.H && iw >= 0 && iw < p.g.W;
            return ok ? ((cv_img[i] + ih * p.g.W + iw) * p.g.IC + c) * 2 : OOB_OFFSET;
        }
    };
    auto b_offset = [&](int i, int k0, bool tail) -> int {
        return (tail && k0 + gch_b[i] * 8 >= p.K) ? OOB_OFFSET : voff_b[i];
    };

#if DIRECT_TO_LDS
    // global -> LDS without passing through registers: each wave-wide load deposits 64 x 16 bytes at a
    // wave-uniform LDS address (M0) in lane order.  The loads are issued from inline assembly so that
    // the compiler does not serialise later LDS reads behind them; completion is tracked by hand with
    // s_waitcnt vmcnt(n) before the workgroup barrier that publishes a stage.
    const unsigned lds_base = (unsigned)(uintptr_t)(lds_ptr_t)smem;
    const unsigned lds_wave = lds_base + (unsigned)wave * 1024u;
    // copy slot `idx` (A slots first, then B slots) of the K tile at k0 into LDS stage `stage`
    auto copy_slot = [&](int idx, int stage, int k0, bool tail, intx4 ra, intx4 rb, ConvTile ct) {
        if (idx < A_ITERS) {
            const int off = a_offset(idx, k0, tail, ct);
            dma16(ra, lds_wave + (unsigned)(stage * STAGE_BYTES + idx * NTHREADS * 16), off);
        } else {
            const int i = idx - A_ITERS;
            const int off = b_offset(i, k0, tail);
            dma16(rb, lds_wave + (unsigned)(stage * STAGE_BYTES + A_STAGE_BYTES + i * NTHREADS * 16), off);
        }
    };
    auto rsrc_a = [&](int k0) -> intx4 {
        return CONV ? raw_rsrc(baseA, bytesA) : raw_rsrc(baseA + k0, bytesA - (unsigned)k0 * 2u);
    };
    auto rsrc_b = [&](int k0) -> intx4 { return raw_rsrc(baseB + k0, bytesB - (unsigned)k0 * 2u); };
#else
    intx4 stage_a[A_ITERS], stage_b[B_ITERS];
    auto load_global = [&](int k0) {
        const bool tail = (k0 + BK > p.K);
        __amdgpu_buffer_rsrc_t rb = make_rsrc(baseB + k0, bytesB - (unsigned)k0 * 2u);
        __amdgpu_buffer_rsrc_t ra = CONV ? make_rsrc(baseA, bytesA) : make_rsrc(baseA + k0, bytesA - (unsigned)k0 * 2u);
#pragma unroll
        for (int i = 0; i < B_ITERS; i++) stage_b[i] = buf_load16(rb, b_offset(i, k0, tail));
        const ConvTile ct = conv_tile(k0);
#pragma unroll
        for (int i = 0; i < A_ITERS; i++) stage_a[i] = buf_load16(ra, a_offset(i, k0, tail, ct));
    };
    auto store_lds = [&](int stage) {
        unsigned char* base = smem + stage * STAGE_BYTES + tid * 16;
#pragma unroll
        for (int i = 0; i < A_ITERS; i++) *(intx4*)(base + i * NTHREADS * 16) = stage_a[i];
#pragma unroll
        for (int i = 0; i < B_ITERS; i++) *(intx4*)(base + A_STAGE_BYTES + i * NTHREADS * 16) = stage_b[i];
    };
#endif

    // ---- fragment read geometry -----------------------------------------------------------------
    // MFMA 32x32x16: lane l supplies row (l % 32), k = 8*(l/32) .. +7 of both operands.
    const int frow = lane & 31, fhalf = lane >> 5;
    const int a_row = wave_m * WM + frow;
    const int b_row = wave_n * WN + frow;
    const int a_rd = a_row * ROW_BYTES, b_rd = A_STAGE_BYTES + b_row * ROW_BYTES;
    auto read_a = [&](const unsigned char* sb, int s, int i) -> half8 {
        return *(const half8*)(sb + a_rd + i * 32 * ROW_BYTES + (((s * 2 + fhalf) ^ swz_key(a_row + i * 32)) << 4));
    };
    auto read_b = [&](const unsigned char* sb, int s, int j) -> half8 {
        return *(const half8*)(sb + b_rd + j * 32 * ROW_BYTES + (((s * 2 + fhalf) ^ swz_key(b_row + j * 32)) << 4));
    };

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    const int ktiles = (k_end - k_begin + BK - 1) / BK;

#if DIRECT_TO_LDS
    // Software pipeline over K tiles with an LDS ring of STAGES stages (tile t lives in stage t % STAGES):
    //   * during the MFMAs of k-step s the fragments of k-step s+1 are read from LDS (two register sets);
    //   * before the last k-step of tile t the wave waits for its own copies of tile t+1 and the workgroup
    //     barrier publishes that stage; at that point tile t's stage has been read completely (its last
    //     fragments sit in registers), so the copy of tile t+STAGES is issued into it during the last
    //     k-step, next to the reads of tile t+1's first fragments.  A copy therefore has a whole K tile
    //     (STAGES-1 of them for deeper rings) to land before anyone waits for it.
    // Every MFMA is followed by its share of the LDS reads / copy instructions and a scheduling fence, so
    // the matrix pipe always has the next MFMA queued while the memory instructions issue in its shadow.
    constexpr int NM = TM * TN;                    // MFMAs per k-step
    constexpr int NR = TM + TN;                    // fragment reads per k-step
    constexpr int NV = A_ITERS + B_ITERS;          // copy instructions per K tile
    constexpr int RPM = (NR + NM - 1) / NM;        // reads issued behind each MFMA
    constexpr int VPM = (NV + NM - 1) / NM;        // copies issued behind each MFMA (last k-step only)
    half8 fa[2][TM], fb[2][TN];

    // fragment read order: a[0], b[0..TN-1], a[1..TM-1] -- the order the MFMAs below first need them
    auto read_frag = [&](int idx, int set, const unsigned char* sb, int step) {
        if (idx == 0) fa[set][0] = read_a(sb, step, 0);
        else if (idx <= TN) fb[set][idx - 1] = read_b(sb, step, idx - 1);
        else fa[set][idx - TN] = read_a(sb, step, idx - TN);
    };

    if (ktiles > 0) {
        // prologue: tiles 0 .. STAGES-1 in flight, tile 0 complete and published
#pragma unroll
        for (int t = 0; t < STAGES; t++) {
            if (t < ktiles) {
                const int k0 = k_begin + t * BK;
                const bool tail = (k0 + BK > p.K);
                const intx4 ra = rsrc_a(k0), rb = rsrc_b(k0);
                const ConvTile ct = conv_tile(k0);
#pragma unroll
                for (int idx = 0; idx < NV; idx++) copy_slot(idx, t, k0, tail, ra, rb, ct);
            }
        }
        // the copies complete in issue order: allow the later tiles' copies to stay in flight
        if (ktiles >= STAGES) wait_vmcnt<(STAGES - 1) * NV>(); else wait_vmcnt<0>();
        __syncthreads();
#pragma unroll
        for (int idx = 0; idx < NR; idx++) read_frag(idx, 0, smem, 0);
    }

    int stage_cur = 0;
    for (int kt = 0; kt < ktiles; kt++) {
        const unsigned char* sb = smem + stage_cur * STAGE_BYTES;
        const int stage_nxt = (stage_cur + 1 == STAGES) ? 0 : stage_cur + 1;
        const int kt_cpy = kt + STAGES;            // tile copied into stage_cur once tile kt has been read
        const int k0c = k_begin + kt_cpy * BK;
        const bool tailc = (k0c + BK > p.K);
        // past the last tile the copy still issues, with empty descriptors: it writes zeros into a stage
        // nobody reads again, which keeps the loop body free of branches
        intx4 ra = rsrc_a(k0c), rb = rsrc_b(k0c);
        if (kt_cpy >= ktiles) { ra[2] = 0; rb[2] = 0; }
        const ConvTile ctc = conv_tile(k0c);

#pragma unroll
        for (int s = 0; s < KSTEPS; s++) {
            const int cur = s & 1, nxt = cur ^ 1;
            const bool last = (s == KSTEPS - 1);
            if (last) {
                // tile kt+1 must be complete in LDS before its first fragments are read; the copies of
                // tiles kt+2 .. kt+STAGES-1 (issued later) may stay in flight
                __builtin_amdgcn_sched_barrier(0);
                if (STAGES > 2 && kt + STAGES - 1 < ktiles) wait_vmcnt<(STAGES - 2) * NV>(); else wait_vmcnt<0>();
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
            }
            const unsigned char* rd_base = last ? smem + stage_nxt * STAGE_BYTES : sb;
            const int rd_step = last ? 0 : s + 1;
#pragma unroll
            for (int m = 0; m < NM; m++) {
                const int i = m / TN, j = m % TN;
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[cur][j], fa[cur][i], acc[i][j], 0, 0, 0);
                // (after the last tile these reads fetch an unused stage; their values are never consumed)
#pragma unroll
                for (int r = 0; r < RPM; r++)
                    if (m * RPM + r < NR) read_frag(m * RPM + r, nxt, rd_base, rd_step);
                if (last) {
#pragma unroll
                    for (int v = 0; v < VPM; v++)
                        if (m * VPM + v < NV) copy_slot(m * VPM + v, stage_cur, k0c, tailc, ra, rb, ctc);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        stage_cur = stage_nxt;
    }
#else
    if (ktiles > 0) {
        load_global(k_begin);
        store_lds(0);
    }
    __syncthreads();

    for (int kt = 0; kt < ktiles; kt++) {
        const int cur = kt & 1;
        const bool more = (kt + 1 < ktiles);
        if (more) load_global(k_begin + (kt + 1) * BK);

        const unsigned char* sb = smem + cur * STAGE_BYTES;
#pragma unroll
        for (int s = 0; s < KSTEPS; s++) {
            half8 af[TM], bf[TN];
#pragma unroll
            for (int i = 0; i < TM; i++) af[i] = read_a(sb, s, i);
#pragma unroll
            for (int j = 0; j < TN; j++) bf[j] = read_b(sb, s, j);
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[j], af[i], acc[i][j], 0, 0, 0);
        }

        if (more) store_lds(cur ^ 1);
        __syncthreads();
    }
#endif

    // ---- epilogue ---------------------------------------------------------------------------------
    // The MFMAs were issued with the B fragment as the first operand, so accumulator tile (i, j) holds the
    // transposed 32x32 block: lane l owns tile row m = l % 32 and, in registers 4g..4g+3, the four
    // consecutive tile columns n = 8g + 4*(l/32) + {0,1,2,3}.
    const int m_l = lane & 31, n_l = (lane >> 5) * 4;
    if (SPLITK > 1) {
        // FP32 partial sums: four consecutive columns per lane, one 16-byte store where that is aligned
        const bool vec_ok = (p.N % 4 == 0);
#pragma unroll
        for (int i = 0; i < TM; i++) {
            const int row = m0 + wave_m * WM + i * 32 + m_l;
#pragma unroll
            for (int j = 0; j < TN; j++) {
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int col = n0 + wave_n * WN + j * 32 + g * 8 + n_l;
                    if (row < p.M) {
                        float* dst = p.ws + ((size_t)blockIdx.y * p.M + row) * p.N + col;
                        if (vec_ok && col + 4 <= p.N) {
                            floatx4 v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                            *(floatx4*)dst = v;
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; e++)
                                if (col + e < p.N) dst[e] = acc[i][j][4 * g + e];
                        }
                    }
                }
            }
        }
    } else {
        // FP16 result through LDS: each wave rounds a 32 x WAVE_COLS strip into its private LDS region
        // (8-byte writes), reads it back row-contiguous and stores 16 bytes per lane, so a store
        // instruction covers whole 2*WAVE_COLS-byte row segments.
#if DIRECT_TO_LDS
        wait_vmcnt<0>();   // the (empty) copies issued behind the last tiles still write zeros into the ring
#endif
        __syncthreads();   // every wave is done reading the ring; the strips reuse its memory
        unsigned char* strip = smem + wave * STRIP_BYTES;
        // widest store the row stride and base address allow: 8, 4, 2 or 1 halves at a time
        const int valign = (int)(((uintptr_t)p.C >> 1) | (unsigned)p.ldc) & 7;
        const int vec = (valign == 0) ? 8 : (valign & 3) == 0 ? 4 : (valign & 1) == 0 ? 2 : 1;
        constexpr int CPR = WN / 8;                    // 16-byte chunks per strip row
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int j = 0; j < TN; j++) {
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    half4 h = {(half_t)acc[i][j][4 * g], (half_t)acc[i][j][4 * g + 1], (half_t)acc[i][j][4 * g + 2],
                               (half_t)acc[i][j][4 * g + 3]};
                    *(half4*)(strip + m_l * STRIP_LD + (j * 32 + g * 8 + n_l) * 2) = h;
                }
            }
            __builtin_amdgcn_wave_barrier();   // same-wave LDS traffic stays in program order
#pragma unroll
            for (int t = 0; t < (32 * CPR) / 64; t++) {
                const int idx = t * 64 + lane;
                const int r = idx / CPR, ch = idx % CPR;
                const intx4 v = *(const intx4*)(strip + r * STRIP_LD + ch * 16);
                const int row = m0 + wave_m * WM + i * 32 + r;
                const int col = n0 + wave_n * WN + ch * 8;
                if (row < p.M && col < p.N) {
                    half_t* dst = p.C + (size_t)row * p.ldc + col;
                    if (vec == 8 && col + 8 <= p.N) {
                        *(intx4*)dst = v;
                    } else if (vec == 4 && col + 8 <= p.N) {
                        ((intx2*)dst)[0] = intx2{v[0], v[1]};
                        ((intx2*)dst)[1] = intx2{v[2], v[3]};
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

// -------------------------------------------------------------------------------------------------
// host side
// -------------------------------------------------------------------------------------------------
#include <stdio.h>

namespace tpl {

constexpr int kElemBytes = 2;

inline const char* info_json() {
    static char buf[1024];
    static bool done = false;
    if (!done) {
        snprintf(buf, sizeof(buf),
                 "{\"family\": \"gemm_f16\", \"arch\": \"gfx950\", \"mfma\": \"v_mfma_f32_32x32x16_f16\", "
                 "\"lds_stages\": %d, \"block_rows\": %d, \"block_cols\": %d, \"wave_rows\": %d, \"wave_cols\": %d, "
                 "\"block_k\": %d, \"split_k\": %d, \"threads\": %d, \"lds_bytes\": %d, "
                 "\"layout_a\": \"M x K row-major f16\", \"layout_b\": \"N x K row-major f16\", "
                 "\"layout_c\": \"M x N row-major f16\", \"accumulate\": \"f32\", "
                 "\"k_multiple\": 8, \"ld_multiple\": 8, \"conv\": \"NHWC x [OC][kH][kW][IC], IC %% 8 == 0\"}",
                 STAGES, BM, BN, WM, WN, BK, SPLITK, NTHREADS, LDS_BYTES);
        done = true;
    }
    return buf;
}

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

inline void bench_layout(int M, int N, int K, size_t* ae, size_t* be, size_t* ce, int* lda, int* ldb, int* ldc) {
    *ae = (size_t)M * K; *be = (size_t)N * K; *ce = (size_t)M * N;
    *lda = K; *ldb = K; *ldc = N;
}

template <int MODE>
inline int set_lds_attr() {
    static int rc = (int)hipFuncSetAttribute((const void*)helix_gemm_f16_kernel<MODE>,
                                             hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
    return rc;
}

template <int MODE>
inline int launch(const Params& p, void* ws, size_t ws_bytes, hipStream_t s) {
    if (SPLITK > 1) {
        const size_t need = workspace_bytes(p.M, p.N, p.K);
        if (!ws || ws_bytes < need) return HELIX_ERR_WORKSPACE;
    }
    int rc = set_lds_attr<MODE>();
    if (rc) return rc;
    const long long ntiles = (long long)p.tiles_m * p.tiles_n;
    if (ntiles > 0x7fffffffLL) return HELIX_ERR_INVALID_VALUE;
    dim3 grid((unsigned)ntiles, (unsigned)p.splits, 1), block(NTHREADS, 1, 1);
    hipLaunchKernelGGL(helix_gemm_f16_kernel<MODE>, grid, block, LDS_BYTES, s, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    if (SPLITK > 1) {
        size_t total = (size_t)p.M * p.N;
        int blocks = (int)((total + 255) / 256);
        if (blocks > 8192) blocks = 8192;
        hipLaunchKernelGGL(helix_splitk_reduce_kernel, dim3(blocks), dim3(256), 0, s, (const float*)ws, p.C, p.M,
                           p.N, p.ldc, p.splits);
        e = hipGetLastError();
        if (e != hipSuccess) return (int)e;
    }
    return 0;
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
    return launch<0>(p, ws, ws_bytes, s);
}

inline int conv2d(const void* x, const void* w, void* y, int batch, int H, int W, int IC, int OC, int kH, int kW,
                  int stride, int pad, void* ws, size_t ws_bytes, hipStream_t s) {
    if (IC % 8 != 0) return HELIX_ERR_INVALID_VALUE;  // a 16-byte chunk must stay inside one filter tap
    const int OH = (H + 2 * pad - kH) / stride + 1, OW = (W + 2 * pad - kW) / stride + 1;
    const long long M = (long long)batch * OH * OW, K = (long long)kH * kW * IC;
    const long long xbytes = (long long)batch * H * W * IC * 2;
    if (M > 0x7fffffffLL || K > 0x7fffffffLL || xbytes >= 0x7fffffffLL) return HELIX_ERR_INVALID_VALUE;
    if ((long long)BN * K * 2 >= 0x7fffffffLL) return HELIX_ERR_INVALID_VALUE;
    if (((uintptr_t)x & 15) || ((uintptr_t)w & 15) || ((uintptr_t)y & 1)) return HELIX_ERR_INVALID_VALUE;
    Params p{};
    p.A = (const half_t*)x; p.B = (const half_t*)w; p.C = (half_t*)y; p.ws = (float*)ws;
    p.M = (int)M; p.N = OC; p.K = (int)K; p.lda = 0; p.ldb = (int)K; p.ldc = OC;
    p.tiles_m = (int)((M + BM - 1) / BM); p.tiles_n = (OC + BN - 1) / BN;
    p.a_bytes = (unsigned)xbytes;
    p.splits = split_factor(M, OC, K);
    p.g = ConvGeom{H, W, IC, OH, OW, kW, stride, pad, (int)M};
    // a K tile inside one filter tap (and a tap mask that fits 32 bits) takes the scalar-tap gather
    if (IC % BK == 0 && kH * kW <= 32) return launch<2>(p, ws, ws_bytes, s);
    return launch<1>(p, ws, ws_bytes, s);
}

}  // namespace tpl

#include "helix_host.h"
