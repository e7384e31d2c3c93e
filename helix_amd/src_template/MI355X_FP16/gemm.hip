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
// Compile-time parameters (set with -D by the build script, one shared library per combination; gemm_tile.h holds
// their defaults and the parts shared with the direct-to-LDS template gemm_dtl.hip):
//   BLOCK_ROWS x BLOCK_COLS   workgroup tile of C           (reference BLOCK_ROWS / BLOCK_COLS)
//   WAVE_ROWS  x WAVE_COLS    tile of C owned by one wave64 (reference WARP_ROWS / WARP_COLS)
//   BLOCK_K                   K extent of one LDS stage (64 or 128)
//   K_STAGES                  K tiles in the pipeline: the tile being multiplied from LDS and K_STAGES - 1 tiles on
//                             their way through staging registers (2: one register set; 3: two, so that a load
//                             has two tiles to land -- a few percent on mid-size tiles, where the registers allow
//                             it)                                                  (reference K_STAGE)
//   SPLIT_K                   1: each workgroup walks all of K.  > 1: K is partitioned into 2 .. SPLIT_K ranges, as
//                             many as it takes to give every compute unit a workgroup (FP32 workspace; the
//                             partitions of a tile are summed in order by the last of them to finish, inside
//                             the launch, or by a reduction kernel where that is not available)
//
// Kernel structure
//   * one wave64 computes (WAVE_ROWS/16) x (WAVE_COLS/16) v_mfma_f32_16x16x32_f16 tiles.  The 16x16x32
//     shape does twice the K depth per accumulator access of the 32x32x16 one; on random data, where the
//     chip runs against its power limit, MFMA-only loops measure 1.95 PFLOP/s with it against 1.69.
//   * global -> registers (128-bit buffer loads; hardware bounds checking zero-fills rows beyond M / N and
//     the K tail) -> LDS (ds_write_b128) -> fragments (ds_read_b128).  Two LDS stages; the loads of a tile
//     are issued K_STAGES - 1 tiles ahead of its LDS writes and every memory instruction sits behind its own MFMA, evenly
//     spread over the tile, so that the four waves of a workgroup never queue bursts on the CU's single
//     address unit (a burst of 64 KiB behind a barrier costs more than the k-step it hides in).
//   * LDS rows are BLOCK_K halves; 16-byte chunk c of row r is stored at chunk (c ^ key(r)), with
//     key(r) = (r / rows_per_256B) mod chunks_per_row, so that 16 consecutive rows of one chunk column
//     land in 16 different 16-byte bank groups (64 banks x 4 B): fragment reads and tile writes are
//     both conflict-free.
//   * workgroup id -> tile: ids are dealt round-robin to the 8 XCDs by the hardware, so id is first
//     remapped to (xcd, slot) -> xcd * ids_per_xcd + slot, then walked in column-major groups of
//     GROUP_ROWS tile rows; each XCD's L2 then sees a compact patch of tiles sharing A and B panels.
#include "gemm_tile.h"
#include "helix_im2col.h"

namespace {

constexpr int KCH = BK / 8;                    // 16-byte chunks per LDS row
constexpr int ROW_BYTES = BK * 2;
constexpr int RP = ROW_BYTES >= 256 ? 1 : 256 / ROW_BYTES;  // rows per 256 bytes of LDS
constexpr int A_ITERS = BM * KCH / NTHREADS, B_ITERS = BN * KCH / NTHREADS;
constexpr int ROWS_PER_ITER = NTHREADS / KCH;
constexpr int RING_BYTES = 2 * STAGE_BYTES;
constexpr int LDS_BYTES = RING_BYTES > NWAVES * STRIP_BYTES ? RING_BYTES : NWAVES * STRIP_BYTES;

static_assert(BK == 64 || BK == 128, "BLOCK_K holds an even number of 32-wide MFMA k-steps: 64 or 128");
static_assert(NTHREADS % KCH == 0, "bad thread count");
static_assert((BM * KCH) % NTHREADS == 0 && (BN * KCH) % NTHREADS == 0, "tile copy must divide evenly");
static_assert(STAGES >= 2 && STAGES <= 4, "K_STAGES: one to three K tiles staged in registers behind the one in LDS");
constexpr int RT = STAGES - 1;                 // K tiles in flight in staging registers
static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of a gfx950 CU exceeded");

__device__ __forceinline__ int swz_key(int row) { return (row / RP) & (KCH - 1); }

__device__ __forceinline__ intx4 buf_load16(__amdgpu_buffer_rsrc_t r, int voff) {
    // cache policy sc0 | sc1 (bits 0 and 4): a tile is read once per compute unit, so the loads go past the CU's
    // vector cache to L2, where the compute units of an XCD share the panels (measured: +2 % at 8192^3)
    return __builtin_bit_cast(intx4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, 0, 17));
}

// ---- static instruction schedule of one K tile ---------------------------------------------------------
// A K tile is G = KSTEPS * TM * TN MFMAs ("slots"), and every memory instruction of the tile is issued behind
// one of them.  A 16x16x32 MFMA keeps the matrix pipe busy for 16 cycles, which leaves the wave room for
// about two other instructions per slot before the pipe runs dry, so the instructions are dealt out as
// evenly as the data dependences allow.  The operand with more fragments per k-step is "resident" (double
// buffered by k-step), the other one is "streamed" (PD fragments ahead through 2*PD registers):
//   * streamed fragment n+PD is read behind the first MFMA that uses fragment n           (slot n * T_RES);
//   * resident fragment v of the next k-step is read half way between two of those  (slot s*NM + v*T_STR +
//     T_STR/2); the next tile's first k-step is read in the PD * T_RES slots past the barrier;
//   * the LDS write of copy slot idx goes to the least loaded slot of its share of the first WSLOTS slots,
//     the global load that refills the same register follows it in the same slot.
constexpr bool RES_A = (TM > TN);              // resident operand: A if it has more fragments, else B
constexpr int T_RES = RES_A ? TM : TN, T_STR = RES_A ? TN : TM;
constexpr int NM = TM * TN;                    // MFMAs per k-step
constexpr int G = KSTEPS * NM;                 // MFMAs per K tile
constexpr int PD = T_STR < 2 ? T_STR : 2;      // read-ahead distance of the streamed operand, in fragments
constexpr int AW = 2 * PD;                     // its register window
constexpr int NSTR = KSTEPS * T_STR;           // streamed fragments per K tile
constexpr int G_BAR = (NSTR - PD) * T_RES;     // slot in front of which the workgroup barrier sits
constexpr int NV = A_ITERS + B_ITERS;          // copy slots (16 bytes per thread each) per K tile
#ifdef WRITE_SLOTS
constexpr int WSLOTS = WRITE_SLOTS;
#else
// LDS writes are kept to the first two thirds of the slots in front of the barrier, so that they have drained
// when the barrier is reached
constexpr int WSLOTS = (2 * G_BAR / 3) > 0 ? (2 * G_BAR / 3) : 1;
#endif
static_assert(NSTR % AW == 0, "streamed fragment window must divide the fragments of a tile");
static_assert(WSLOTS >= 1 && WSLOTS <= G_BAR, "LDS writes must be issued in front of the barrier");

struct Schedule {
    int wslot[NV];   // slot of the LDS write of copy slot idx
    int lslot[NV];   // slot of the global load that refills its register (the same slot)
};

constexpr int res_read_slot(int s, int v) { return s * NM + v * T_STR + T_STR / 2; }      // k-step s+1, in tile
constexpr int res_next_slot(int v) { return G_BAR + v * PD + (PD - 1); }                  // next tile, k-step 0

constexpr Schedule make_schedule() {
    Schedule sc{};
    int cnt[G] = {};
    for (int n = 0; n < NSTR; n++) cnt[n * T_RES]++;
    for (int s = 0; s + 1 < KSTEPS; s++)
        for (int v = 0; v < T_RES; v++) cnt[res_read_slot(s, v)]++;
    for (int v = 0; v < T_RES; v++) cnt[res_next_slot(v)]++;
    for (int idx = 0; idx < NV; idx++) {
        const int lo = idx * WSLOTS / NV;
        int hi = (idx + 1) * WSLOTS / NV;
        if (hi <= lo) hi = lo + 1;
        int best = lo;
        for (int g = lo; g < hi; g++)
            if (cnt[g] < cnt[best]) best = g;
        sc.wslot[idx] = best;
        cnt[best]++;
    }
    // the refill goes out right behind the write that frees its register: every load then has a whole K tile to
    // land (spreading the loads evenly over the tile instead left the last ones 60 % of a tile and measured 1 - 3 %
    // slower at 8192^3)
    for (int idx = 0; idx < NV; idx++) {
        sc.lslot[idx] = sc.wslot[idx];
        cnt[sc.lslot[idx]]++;
    }
    return sc;
}


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

    const TileRange tr = tile_range_of_workgroup(p);
    if (tr.idle) return;
    const int m0 = tr.m0, n0 = tr.n0, k_begin = tr.k_begin, k_end = tr.k_end;

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
            const int t = p.g.by_OW.div(m);
            const int ow = m - t * p.g.OW;
            const int b = p.g.by_OH.div(t);
            const int oh = t - b * p.g.OH;
            cv_img[i] = (m < p.g.M) ? b * p.g.H * p.g.W : -1;
            cv_ih[i] = oh * p.g.stride - p.g.pad;
            cv_iw[i] = ow * p.g.stride - p.g.pad;
            if (MODE == 2) {
                cv_base[i] = ((cv_img[i] + cv_ih[i] * p.g.W + cv_iw[i]) * p.g.IC + gch_a[i] * 8) * 2;
                // taps inside the image form a rectangle kh in [kh_lo, kh_hi) x kw in [kw_lo, kw_hi)
                const int kH = p.g.by_kW.div(p.g.by_IC.div(p.K));
                const int kw_lo = cv_iw[i] < 0 ? -cv_iw[i] : 0;
                const int kw_hi = (p.g.W - cv_iw[i]) < p.g.kW ? (p.g.W - cv_iw[i]) : p.g.kW;
                const int kh_lo = cv_ih[i] < 0 ? -cv_ih[i] : 0;
                const int kh_hi = (p.g.H - cv_ih[i]) < kH ? (p.g.H - cv_ih[i]) : kH;
                const unsigned row_bits = (kw_hi > kw_lo && cv_img[i] >= 0) ? ((1u << kw_hi) - (1u << kw_lo)) : 0u;
                unsigned taps = 0;
                for (int kh = 0; kh < kH; kh++)
                    if (kh >= kh_lo && kh < kh_hi) taps |= row_bits << (kh * p.g.kW);
                cv_taps[i] = taps;
            }
        }
    }

    // MODE 2: scalar state of a K tile: byte offset of its filter tap and channel block, and its tap bit.
    // K tiles are visited in order, so the state is stepped from tile to tile (a tile never straddles a tap:
    // IC is a multiple of BLOCK_K) instead of being derived from k0 with integer divisions every tile.
    struct ConvTile { int soff; unsigned tapbit; };
    struct ConvWalk {
        int k0, c0, kw, tap, tap_off;   // tile start, channel within the tap, tap column, tap index, tap byte offset
    };
    ConvWalk walk{0, 0, 0, 0, 0};
    if (MODE == 2) {
        const int tap = p.g.by_IC.div(k_begin), kh = p.g.by_kW.div(tap);
        walk.k0 = k_begin;
        walk.c0 = k_begin - tap * p.g.IC;
        walk.kw = tap - kh * p.g.kW;
        walk.tap = tap;
        walk.tap_off = (kh * p.g.W + walk.kw) * p.g.IC * 2;
    }
    // state of the tile the walk stands on (empty past the end of K), then one tile forward
    auto conv_next = [&]() -> ConvTile {
        ConvTile ct{0, 0u};
        if (MODE == 2) {
            if (walk.k0 < p.K) {
                ct.soff = walk.tap_off + walk.c0 * 2;
                ct.tapbit = 1u << walk.tap;
            }
            walk.k0 += BK;
            walk.c0 += BK;
            if (walk.c0 >= p.g.IC) {
                walk.c0 = 0;
                walk.tap += 1;
                walk.kw += 1;
                walk.tap_off += p.g.IC * 2;
                if (walk.kw == p.g.kW) {
                    walk.kw = 0;
                    walk.tap_off += (p.g.W - p.g.kW) * p.g.IC * 2;
                }
            }
        }
        return ct;
    };

    // Byte offset (relative to the operand's buffer descriptor) of copy slot i for the K tile at k0, or
    // OOB_OFFSET when the slot must read zeros (conv padding, rows beyond M, and -- only for the first tile
    // of the K range, which is the one that may be narrower than BLOCK_K -- columns beyond its width).
    auto a_offset = [&](int i, int k0, bool narrow, int width, ConvTile ct) -> int {
        if (!CONV) {
            return (narrow && gch_a[i] * 8 >= width) ? OOB_OFFSET : voff_a[i];
        } else if (MODE == 2) {
            return (cv_taps[i] & ct.tapbit) ? cv_base[i] + ct.soff : OOB_OFFSET;
        } else {
            const int k = k0 + gch_a[i] * 8;  // k = (kh*kW + kw)*IC + c, 8 consecutive c per chunk
            const int t = p.g.by_IC.div(k);
            const int c = k - t * p.g.IC;
            const int kh = p.g.by_kW.div(t);
            const int kw = t - kh * p.g.kW;
            const int ih = cv_ih[i] + kh, iw = cv_iw[i] + kw;
            const bool ok = !(narrow && gch_a[i] * 8 >= width) && cv_img[i] >= 0 && ih >= 0 && ih < p.g.H && iw >= 0 &&
                            iw < p.g.W;
            return ok ? ((cv_img[i] + ih * p.g.W + iw) * p.g.IC + c) * 2 : OOB_OFFSET;
        }
    };
    auto b_offset = [&](int i, bool narrow, int width) -> int {
        return (narrow && gch_b[i] * 8 >= width) ? OOB_OFFSET : voff_b[i];
    };

    // global -> registers -> LDS.  Copy slot idx (A slots first, then B slots) of a K tile is one 16-byte
    // buffer load per lane; hardware bounds checking zero-fills rows beyond M / N.
    auto load_slot = [&](int idx, int k0, bool narrow, int width, __amdgpu_buffer_rsrc_t ra,
                         __amdgpu_buffer_rsrc_t rb, ConvTile ct) -> intx4 {
        if (idx < A_ITERS) return buf_load16(ra, a_offset(idx, k0, narrow, width, ct));
        return buf_load16(rb, b_offset(idx - A_ITERS, narrow, width));
    };
    auto store_slot = [&](int idx, int stage, intx4 v) {
        const int off = idx < A_ITERS ? idx * NTHREADS * 16 : A_STAGE_BYTES + (idx - A_ITERS) * NTHREADS * 16;
        *(intx4*)(smem + stage * STAGE_BYTES + off + tid * 16) = v;
    };
    // descriptors of the K tile at k0; `live` false gives empty ones (every load returns zeros)
    auto rsrc_a = [&](int k0, bool live) -> __amdgpu_buffer_rsrc_t {
        const unsigned n = !live ? 0u : CONV ? bytesA : bytesA - (unsigned)k0 * 2u;
        return make_rsrc(CONV ? baseA : baseA + k0, n);
    };
    auto rsrc_b = [&](int k0, bool live) -> __amdgpu_buffer_rsrc_t {
        return make_rsrc(baseB + k0, live ? bytesB - (unsigned)k0 * 2u : 0u);
    };

    // ---- fragment read geometry -----------------------------------------------------------------
    // MFMA 16x16x32: lane l supplies row (l % 16), k = 8*(l/16) .. +7 of both operands, i.e. 16-byte chunk
    // (4*s + l/16) of its row for k-step s.
    const int frow = lane & 15, fq = lane >> 4;
    const int a_row = wave_m * WM + frow;
    const int b_row = wave_n * WN + frow;
    const int a_rd = a_row * ROW_BYTES, b_rd = A_STAGE_BYTES + b_row * ROW_BYTES;
    auto read_a = [&](const unsigned char* sb, int s, int i) -> half8 {
        return *(const half8*)(sb + a_rd + i * 16 * ROW_BYTES + (((s * 4 + fq) ^ swz_key(a_row + i * 16)) << 4));
    };
    auto read_b = [&](const unsigned char* sb, int s, int j) -> half8 {
        return *(const half8*)(sb + b_rd + j * 16 * ROW_BYTES + (((s * 4 + fq) ^ swz_key(b_row + j * 16)) << 4));
    };

    floatx4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    const int ktiles = (k_end - k_begin + BK - 1) / BK;

    // Software pipeline over K tiles.  Tile t is multiplied from LDS stage t % 2 while
    //   * the staging registers that hold tile t+1 (loaded a tile ago) are written to the other stage with
    //     ds_write_b128 and each register is refilled with the same slot of tile t+2, so a global load has
    //     a whole K tile to land;
    //   * fragments are read ahead of the MFMAs that use them: the operand with more fragments per k-step
    //     (the "resident" one) is double-buffered by k-step and read one k-step ahead, the other one is
    //     streamed through a small rotating set of registers, PD fragments ahead;
    //   * one workgroup barrier per tile, placed between the last fragment read of tile t and the first one
    //     of tile t+1 (PD streamed fragments before the end of the tile).  It publishes tile t+1, whose LDS
    //     writes were all issued -- and had time to drain -- earlier in the tile, and it frees stage t % 2.
    // Every MFMA is followed by its share of the memory instructions and a scheduling fence: the matrix pipe
    // always has the next MFMA queued while the memory instructions issue in its shadow.
    constexpr Schedule sched = make_schedule();
    half8 fr[2][T_RES], fs[AW];
    intx4 st[RT][NV];

    auto read_res = [&](const unsigned char* sb, int s, int v) -> half8 {
        return RES_A ? read_a(sb, s, v) : read_b(sb, s, v);
    };
    auto read_str = [&](const unsigned char* sb, int s, int u) -> half8 {
        return RES_A ? read_b(sb, s, u) : read_a(sb, s, u);
    };

    // K tiles: when the K range is not a multiple of BLOCK_K the narrow tile comes first (tile 0 covers
    // `first_w` columns, every later tile BLOCK_K), so that only the prologue's loads need a column mask
    const int first_w = ((k_end - k_begin) % BK) ? ((k_end - k_begin) % BK) : BK;
    auto tile_k0 = [&](int t) -> int { return t == 0 ? k_begin : k_begin + first_w + (t - 1) * BK; };

    if (ktiles > 0) {
        // prologue: tiles 0 .. RT-1 into the staging register sets (tile j in set j), tile 0 on to LDS and its set
        // refilled with tile RT
#pragma unroll
        for (int j = 0; j < RT; j++) {
            const int k0 = tile_k0(j);
            const __amdgpu_buffer_rsrc_t ra = rsrc_a(k0, j < ktiles), rb = rsrc_b(k0, j < ktiles);
            const ConvTile ct = conv_next();
#pragma unroll
            for (int idx = 0; idx < NV; idx++) st[j][idx] = load_slot(idx, k0, j == 0, j == 0 ? first_w : BK, ra, rb, ct);
        }
        {
            const int k0 = tile_k0(RT);
            const __amdgpu_buffer_rsrc_t ra = rsrc_a(k0, RT < ktiles), rb = rsrc_b(k0, RT < ktiles);
            const ConvTile ct = conv_next();
#pragma unroll
            for (int idx = 0; idx < NV; idx++) {
                store_slot(idx, 0, st[0][idx]);
                st[0][idx] = load_slot(idx, k0, false, BK, ra, rb, ct);
            }
        }
        __syncthreads();
        // first fragments of tile 0, in the order in which the loop reads those of the next tile past its
        // barrier: the compiler's wait counts at the loop head are the merge of both paths
#pragma unroll
        for (int g = G_BAR; g < G; g++) {
            if (g % T_RES == 0) {
                const int n = g / T_RES + PD - NSTR;
                fs[n % AW] = read_str(smem, n / T_STR, n % T_STR);
            }
#pragma unroll
            for (int r = 0; r < T_RES; r++)
                if (res_next_slot(r) == g) fr[0][r] = read_res(smem, 0, r);
        }
    }

    // Slots [LO, HI) of K tile kt, multiplied from LDS stage `stage`.  stv: the staging registers that hold tile
    // kt + 1.  k0c, ra, rb, ctc: start, descriptors and conv state of tile kt + 1 + RT, the one loaded into those
    // registers once they are written.
    auto tile_part = [&](auto lo_c, auto hi_c, int stage, intx4 (&stv)[NV], int k0c, __amdgpu_buffer_rsrc_t ra,
                         __amdgpu_buffer_rsrc_t rb, ConvTile ctc) {
        constexpr int LO = decltype(lo_c)::value, HI = decltype(hi_c)::value;
        const unsigned char* sb = smem + stage * STAGE_BYTES;
        const unsigned char* sb_nxt = smem + (stage ^ 1) * STAGE_BYTES;
#pragma unroll
        for (int n = LO / T_RES; n < (HI + T_RES - 1) / T_RES; n++) {   // streamed fragment n: k-step s, index u
#pragma unroll
          for (int v = 0; v < T_RES; v++) {                             // resident fragment v
            const int g = n * T_RES + v;                                // slot
            if (g < LO || g >= HI) continue;
            const int s = n / T_STR, u = n % T_STR;
            if (RES_A) acc[v][u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fs[n % AW], fr[s & 1][v], acc[v][u], 0, 0, 0);
            else acc[u][v] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fr[s & 1][v], fs[n % AW], acc[u][v], 0, 0, 0);
            // streamed fragment n+PD, behind the first MFMA of fragment n (past the barrier: the next tile's)
            if (v == 0) {
                const int n2 = n + PD;
                if (n2 < NSTR) fs[n2 % AW] = read_str(sb, n2 / T_STR, n2 % T_STR);
                else fs[n2 % AW] = read_str(sb_nxt, (n2 - NSTR) / T_STR, (n2 - NSTR) % T_STR);
            }
            // resident fragments of the next k-step, or of the next tile's first k-step past the barrier
            // (after the last tile these reads fetch an unused stage; their values are never consumed)
#pragma unroll
            for (int r = 0; r < T_RES; r++) {
                if (s + 1 < KSTEPS && res_read_slot(s, r) == g) fr[(s + 1) & 1][r] = read_res(sb, s + 1, r);
                if (res_next_slot(r) == g) fr[0][r] = read_res(sb_nxt, 0, r);
            }
            // LDS writes of the staged tile and the refills of their registers
#pragma unroll
            for (int idx = 0; idx < NV; idx++) {
                if (sched.wslot[idx] == g) store_slot(idx, stage ^ 1, stv[idx]);
                if (sched.lslot[idx] == g) stv[idx] = load_slot(idx, k0c, false, BK, ra, rb, ctc);
            }
            __builtin_amdgcn_sched_barrier(0);
          }
        }
    };
    constexpr std::integral_constant<int, 0> c_0{};
    constexpr std::integral_constant<int, G_BAR> c_bar{};
    constexpr std::integral_constant<int, G> c_end{};
    // one K tile: multiply tile kt from `stage`, move tile kt + 1 from its registers to the other stage, refill them
    // with tile kt + 1 + RT
    auto tile_step = [&](int kt, int stage, intx4 (&stv)[NV]) {
        const int kt_ld = kt + 1 + RT;
        const int k0c = tile_k0(kt_ld);
        // past the last tile the loads still issue, with empty descriptors, which keeps the body branch-free
        const __amdgpu_buffer_rsrc_t ra = rsrc_a(k0c, kt_ld < ktiles), rb = rsrc_b(k0c, kt_ld < ktiles);
        const ConvTile ctc = conv_next();
        tile_part(c_0, c_bar, stage, stv, k0c, ra, rb, ctc);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        tile_part(c_bar, c_end, stage, stv, k0c, ra, rb, ctc);
    };
    // tile kt + 1 sits in register set (kt + 1) % RT and LDS stage (kt + 1) % 2.  One register set: a plain loop
    // with the stage as a variable (unrolling it doubles the register pressure of the one-wave tiles, whose copy
    // slots already fill the file).  More sets: the loop is unrolled over the least common multiple of the two
    // periods so that the set is a compile-time constant.
    constexpr int UNROLL = (RT % 2 == 0) ? RT : 2 * RT;
    if constexpr (RT == 1) {
        int stage = 0;
        for (int kt = 0; kt < ktiles; kt++) {
            tile_step(kt, stage, st[0]);
            stage ^= 1;
        }
    } else {
        int kt = 0;
        for (; kt + UNROLL <= ktiles; kt += UNROLL) {
#pragma unroll
            for (int u = 0; u < UNROLL; u++) tile_step(kt + u, u & 1, st[(u + 1) % RT]);
        }
#pragma unroll
        for (int u = 0; u < UNROLL - 1; u++)
            if (kt + u < ktiles) tile_step(kt + u, u & 1, st[(u + 1) % RT]);
    }

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
                 "\"k_multiple\": 8, \"ld_multiple\": 8, \"conv\": \"NHWC x [OC][kH][kW][IC]; implicit GEMM when IC %% 8 == 0, else column buffer in the workspace\"}",
                 STAGES, BM, BN, WM, WN, BK, SPLITK, 0, NTHREADS, LDS_BYTES);
        done = true;
    }
    return buf;
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
    Params q = p;
    const dim3 grid = launch_grid(q), block(NTHREADS, 1, 1);   // K partitions added inside the launch where available
    hipLaunchKernelGGL(helix_gemm_f16_kernel<MODE>, grid, block, LDS_BYTES, s, q);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    if (SPLITK > 1 && !q.plan.fused) {
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

// Convolutions whose channel count is not a multiple of 8 run on channel-padded copies of activations and
// weights in the workspace, or (thin inputs, where padding would multiply the work) through a column buffer (K
// padded to a multiple of 8) and repacked weights there, then through the GEMM above.
inline int conv_padded_k(int IC, int kH, int kW) { return (IC * kH * kW + 7) / 8 * 8; }

inline size_t conv_workspace_bytes(int batch, int H, int W, int IC, int OC, int kH, int kW, int stride, int pad) {
    const int OH = (H + 2 * pad - kH) / stride + 1, OW = (W + 2 * pad - kW) / stride + 1;
    const long long M = (long long)batch * OH * OW;
    if (M > 0x7fffffffLL) return 0;
    if (IC % 8 == 0) return workspace_bytes((int)M, OC, IC * kH * kW);
    if (helix_im2col::pads_channels(batch, H, W, IC, 8, 2)) {
        const int ICp = helix_im2col::padded_channels(IC, 8);
        return helix_im2col::align256((size_t)batch * H * W * ICp * 2) +
               helix_im2col::align256((size_t)OC * kH * kW * ICp * 2) + workspace_bytes((int)M, OC, ICp * kH * kW);
    }
    const int Kp = conv_padded_k(IC, kH, kW);
    return helix_im2col::align256((size_t)M * Kp * 2) + helix_im2col::align256((size_t)OC * Kp * 2) +
           workspace_bytes((int)M, OC, Kp);
}

inline int conv2d(const void* x, const void* w, void* y, int batch, int H, int W, int IC, int OC, int kH, int kW,
                  int stride, int pad, void* ws, size_t ws_bytes, hipStream_t s);

inline int conv2d_padded_channels(const void* x, const void* w, void* y, int batch, int H, int W, int IC, int OC,
                                  int kH, int kW, int stride, int pad, void* ws, size_t ws_bytes, hipStream_t s) {
    const int ICp = helix_im2col::padded_channels(IC, 8);
    const long long pixels = (long long)batch * H * W, taps = (long long)OC * kH * kW;
    if (taps * (ICp / 8) > 0x7fffffffLL) return HELIX_ERR_INVALID_VALUE;
    const size_t xp_bytes = helix_im2col::align256((size_t)pixels * ICp * 2);
    const size_t wp_bytes = helix_im2col::align256((size_t)taps * ICp * 2);
    if (!ws || ws_bytes < conv_workspace_bytes(batch, H, W, IC, OC, kH, kW, stride, pad)) return HELIX_ERR_WORKSPACE;
    if ((uintptr_t)ws & 15) return HELIX_ERR_INVALID_VALUE;
    half_t* xp = (half_t*)ws;
    half_t* wp = (half_t*)((unsigned char*)ws + xp_bytes);
    const helix_fastdiv::FastDiv by_chunks = helix_fastdiv::make(ICp / 8);
    hipLaunchKernelGGL((helix_im2col::pad_channels_kernel<half_t, 8>),
                       dim3(helix_im2col::grid_for((size_t)pixels * (ICp / 8))), dim3(256), 0, s, (const half_t*)x, xp,
                       (int)pixels, IC, ICp, by_chunks);
    hipLaunchKernelGGL((helix_im2col::pad_channels_kernel<half_t, 8>),
                       dim3(helix_im2col::grid_for((size_t)taps * (ICp / 8))), dim3(256), 0, s, (const half_t*)w, wp,
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
    if (M > 0x7fffffffLL || K > 0x7fffffffLL) return HELIX_ERR_INVALID_VALUE;
    const int Kp = conv_padded_k(IC, kH, kW);
    const size_t col_bytes = helix_im2col::align256((size_t)M * Kp * 2);
    const size_t wp_bytes = helix_im2col::align256((size_t)OC * Kp * 2);
    if (!ws || ws_bytes < conv_workspace_bytes(batch, H, W, IC, OC, kH, kW, stride, pad)) return HELIX_ERR_WORKSPACE;
    half_t* col = (half_t*)ws;
    half_t* wp = (half_t*)((unsigned char*)ws + col_bytes);
    void* rest = (unsigned char*)ws + col_bytes + wp_bytes;
    if (M * (Kp / 8) > 0x7fffffffLL) return HELIX_ERR_INVALID_VALUE;
    const helix_im2col::Geom g = helix_im2col::make_geom(H, W, IC, OH, OW, kW, stride, pad, (int)M, (int)K);
    hipLaunchKernelGGL((helix_im2col::im2col_rows_kernel<half_t, 8>), dim3(helix_im2col::grid_for((size_t)M * (Kp / 8))),
                       dim3(256), 0, s, (const half_t*)x, col, g, Kp, helix_fastdiv::make(Kp / 8));
    hipLaunchKernelGGL((helix_im2col::pack_weights_rows_kernel<half_t>), dim3(helix_im2col::grid_for((size_t)OC * Kp)),
                       dim3(256), 0, s, (const half_t*)w, wp, OC, (int)K, Kp);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    return gemm(col, wp, y, (int)M, OC, Kp, Kp, Kp, OC, rest, ws_bytes - col_bytes - wp_bytes, s);
}

inline int conv2d(const void* x, const void* w, void* y, int batch, int H, int W, int IC, int OC, int kH, int kW,
                  int stride, int pad, void* ws, size_t ws_bytes, hipStream_t s) {
    if (((uintptr_t)x & 15) || ((uintptr_t)w & 15) || ((uintptr_t)y & 1)) return HELIX_ERR_INVALID_VALUE;
    if (IC % 8 != 0) {   // a 16-byte chunk of the implicit gather must stay inside one filter tap
        if (helix_im2col::pads_channels(batch, H, W, IC, 8, 2))
            return conv2d_padded_channels(x, w, y, batch, H, W, IC, OC, kH, kW, stride, pad, ws, ws_bytes, s);
        return conv2d_explicit(x, w, y, batch, H, W, IC, OC, kH, kW, stride, pad, ws, ws_bytes, s);
    }
    const int OH = (H + 2 * pad - kH) / stride + 1, OW = (W + 2 * pad - kW) / stride + 1;
    const long long M = (long long)batch * OH * OW, K = (long long)kH * kW * IC;
    const long long xbytes = (long long)batch * H * W * IC * 2;
    if (M > 0x7fffffffLL || K > 0x7fffffffLL || xbytes >= 0x7fffffffLL) return HELIX_ERR_INVALID_VALUE;
    if ((long long)BN * K * 2 >= 0x7fffffffLL) return HELIX_ERR_INVALID_VALUE;
    // a 1 x 1 filter walked pixel by pixel gathers nothing: the activations as they lie are the A operand (rows =
    // pixels, K = IC), so the layer is the plain GEMM and runs without the gather's index arithmetic
    if (kH == 1 && kW == 1 && stride == 1 && pad == 0)
        return gemm(x, w, y, (int)M, OC, IC, IC, IC, OC, ws, ws_bytes, s);
    Params p{};
    p.A = (const half_t*)x; p.B = (const half_t*)w; p.C = (half_t*)y; p.ws = (float*)ws;
    p.M = (int)M; p.N = OC; p.K = (int)K; p.lda = 0; p.ldb = (int)K; p.ldc = OC;
    p.tiles_m = (int)((M + BM - 1) / BM); p.tiles_n = (OC + BN - 1) / BN;
    p.a_bytes = (unsigned)xbytes;
    p.splits = split_factor(M, OC, K);
    p.g = ConvGeom{H, W, IC, OH, OW, kW, stride, pad, (int)M,
                   helix_fastdiv::make(OW), helix_fastdiv::make(OH), helix_fastdiv::make(IC), helix_fastdiv::make(kW)};
    // a K tile inside one filter tap (and a tap mask that fits 32 bits) takes the scalar-tap gather
    if (IC % BK == 0 && kH * kW <= 32 && kW < 32) return launch<2>(p, ws, ws_bytes, s);
    return launch<1>(p, ws, ws_bytes, s);
}

}  // namespace tpl

#if SPLIT_K == 1
#define HELIX_TPL_SCRATCH_BYTES 256   // no K partition: this library never asks for a workspace
#endif
#include "helix_host.h"
