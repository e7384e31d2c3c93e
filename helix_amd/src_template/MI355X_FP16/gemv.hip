// MI355X (gfx950 / CDNA4) FP16 GEMV / skinny-GEMM template: HBM-bound weight streaming.
//
//   C[M x N] = A[M x K] * B[N x K]^T,  M small (decode batch), B = the weight matrix, streamed once.
//   FP16 in, FP32 accumulate, FP16 out.  Up to MFMA_MIN_M - 1 activation rows the products are
//   v_dot2_f32_f16 with a wave reduction (no MFMA); from MFMA_MIN_M rows on, the vector units would need
//   more time for the M x K x N dot products than HBM needs for the weights (at M = 16: 48 us against 59 us
//   for 8192 x 28672, before any overhead), and the same stream feeds v_mfma_f32_16x16x32_f16 instead.
//
// Role in the reference: src_template/Ampere_FP16/gemv.cu:152-252 (`mySGemvKernel_Stage4` and its
// N_TILE dispatch) and gemv_splitK.cu:153-260.  The reference names the streamed matrix A (Mbig x K)
// and the skinny one B (Nsmall x K) and swaps M and N on the host so that M >= N (gemv.cu:384-386);
// here the streamed matrix is always the B operand of the common GEMM signature and callers with a
// tall-skinny problem swap operands themselves (C^T = B * A^T).
//
// Kernel structure
//   * a workgroup (4 waves) first stages its M_TILE activation rows for its K range in LDS, once;
//   * each wave then walks its own run of consecutive weight rows, ROWS rows at a time, from first to
//     last column: the 64 lanes are spread along K and every load instruction fetches one contiguous
//     1 KiB segment of a row (128-bit per lane, non-temporal), so a wave reads long sequential spans of
//     HBM -- the access pattern that streams fastest on this part;
//   * per 512-wide K step a lane reads the matching 16 bytes of each activation row from LDS
//     (conflict-free ds_read_b128) and issues M_TILE x ROWS x 4 v_dot2_f32_f16;
//   * the M_TILE x ROWS FP32 partial sums per lane are reduced across the wave with a transposing
//     butterfly (each exchange halves the number of live values, ~2 instructions per value instead of
//     12 for one butterfly per value) and written by the lanes that own them;
//   * activations of up to 64 KiB leave room for two workgroups per CU; between 64 and 128 KiB one workgroup of
//     twice as many waves takes the CU alone (same waves per CU, no K partition);
//   * K is partitioned over blockIdx.z when the activations of the whole K range would not fit even that
//     (M_TILE * K * 2 bytes > 128 KiB) or when SPLIT_K asks for it; partials then go to an FP32
//     workspace and a second kernel sums them in fixed order (deterministic; the reference uses half
//     atomics, gemv_splitK.cu:213-217).
//
// MFMA variant (M >= MFMA_MIN_M)
//   * a workgroup walks its K range in chunks of MFMA_KCHUNK columns and stages 16 activation rows of the
//     chunk in LDS, rows 16 bytes apart from a multiple of 256 so that 16 rows of one column sit in 16
//     different bank groups;
//   * a wave owns runs of 16 consecutive weight rows; per 256-wide K step it issues eight 16-byte loads per
//     lane, straight into registers in the operand layout of the MFMA (lane l: row l % 16, columns 8*(l/16)
//     .. +7 of a 32-wide block): 512 contiguous bytes per row and step, 64 per row and instruction; the same
//     columns of activation row l % 16 come from LDS;
//   * eight MFMAs per step accumulate the 16 x 16 block y[m][n]; steps are double-buffered; buffer bounds
//     checking zero-fills weight rows beyond N;
//   * K is partitioned over blockIdx.z only when the weight rows alone give the launch too few waves to cover
//     the latency of the stream (FP32 workspace + fixed-order reduce).
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
#define GEMV_R4 2
#define GEMV_KU4 4
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
#ifndef TARGET_WAVES
#define TARGET_WAVES 2048   // waves a launch aims for: 256 compute units x 8
#endif
#ifndef MFMA_MIN_M
#define MFMA_MIN_M 9        // activation rows from which the MFMA variant takes over (measured crossover)
#endif
#ifndef MFMA_TARGET_WAVES
#define MFMA_TARGET_WAVES 8192
#endif
#ifndef MFMA_WAVES_PER_BLOCK
#define MFMA_WAVES_PER_BLOCK 4
#endif
#ifndef MFMA_KCHUNK
#define MFMA_KCHUNK 1024    // columns of the 16 activation rows staged in LDS at a time by the MFMA variant
#endif

namespace {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef int intx4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));

constexpr int SPLITK = SPLIT_K;
constexpr int WPB = WAVES_PER_BLOCK;
constexpr int KSTEP = 64 * 8;  // halves covered by one wave-wide 128-bit load

struct Params {
    const half_t* A;  // M x K activations
    const half_t* B;  // N x K weights
    half_t* C;        // M x N
    float* ws;        // ksplit > 1: [ksplit][M][N] FP32 partial sums
    int M, N, K, lda, ldb, ldc;
    int kchunk;         // K range of one workgroup (multiple of KSTEP)
    int ksplit;         // number of K ranges (grid.z)
    int rows_per_wave;  // consecutive weight rows owned by one wave
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

// WAVES: waves per workgroup.  WAVES_PER_BLOCK when the staged activations leave room for two workgroups per
// CU, twice that when they need more than half of the LDS, so that a long K costs neither occupancy nor a
// K partition with its second kernel.
template <int MT, int ROWS, int KU, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void helix_gemv_f16_kernel(const Params p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    half_t* xs = (half_t*)smem;                      // [MT][kchunk] activations of this K range

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

    const half_t* wrow[ROWS];
    auto set_rows = [&](int n0) {
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            const int n = (n0 + r) < p.N ? (n0 + r) : (p.N - 1);   // clamp: duplicates are never stored
            wrow[r] = p.B + (size_t)n * p.ldb + lane * 8;
        }
    };
    auto load_trip = [&](half8 (&w)[KU][ROWS], int kk) {
#pragma unroll
        for (int u = 0; u < KU; u++)
#pragma unroll
            for (int r = 0; r < ROWS; r++) w[u][r] = load_stream(wrow[r] + kk + u * KSTEP);
    };

    // The first trip of the first row group is requested before the activations are staged, and the
    // first trip of every later group before the previous group is reduced: the weight stream never
    // waits for anything but HBM.
    half8 wa[KU][ROWS], wb[KU][ROWS];
    const bool has_trip = (k_begin + TRIP <= k_end);
    if (row_first < row_last) {
        set_rows(row_first);
        if (has_trip) load_trip(wa, k_begin);
    }

    // ---- stage the activations: 16-byte chunks, zero beyond M and beyond K ----------------------------
    {
        const int chunks_per_row = kchunk / 8;
        const int total = MT * chunks_per_row;
        for (int c = tid; c < total; c += 64 * WAVES) {
            const int m = c / chunks_per_row, kc = (c % chunks_per_row) * 8;
            intx4 v = {0, 0, 0, 0};
            if (m0 + m < p.M && k_begin + kc < k_end) v = *(const intx4*)(p.A + (size_t)(m0 + m) * p.lda + k_begin + kc);
            *(intx4*)(xs + (size_t)m * kchunk + kc) = v;
        }
    }
    __syncthreads();

    const half_t* xl = xs + lane * 8;                // this lane's 8 halves of every 512-wide step
    float acc[MT * ROWS];
    auto dot_trip = [&](const half8 (&w)[KU][ROWS], int kk) {
#pragma unroll
        for (int u = 0; u < KU; u++)
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const half8 xv = *(const half8*)(xl + (size_t)m * kchunk + (kk - k_begin) + u * KSTEP);
#pragma unroll
                for (int r = 0; r < ROWS; r++) acc[m * ROWS + r] = dot8(w[u][r], xv, acc[m * ROWS + r]);
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
                const bool live = kk + lane * 8 < k_end;
#pragma unroll
                for (int r = 0; r < ROWS; r++) {
                    half8 z = {0, 0, 0, 0, 0, 0, 0, 0};
                    wb[u][r] = live ? load_stream(wrow[r] + kk) : z;
                }
            }
#pragma unroll
            for (int u = 0; u < KU; u++) {
                const int kk = k + u * KSTEP;
                if (kk < k_end) {   // wave-uniform: steps past the K range have no staged activations
#pragma unroll
                    for (int m = 0; m < MT; m++) {
                        const half8 xv = *(const half8*)(xl + (size_t)m * kchunk + (kk - k_begin));
#pragma unroll
                        for (int r = 0; r < ROWS; r++) acc[m * ROWS + r] = dot8(wb[u][r], xv, acc[m * ROWS + r]);
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
                        p.C[(size_t)m * p.ldc + n] = (half_t)acc[i];
                }
            }
        }
    }
}

// ---- MFMA variant -----------------------------------------------------------------------------------------
constexpr int MSTEP = 256;                      // K extent of one step: eight 16-byte loads per lane, 512 bytes per weight row
constexpr int MCH = MSTEP / 32;                 // 16-byte chunks per lane and step = MFMAs per step
constexpr int MFMA_KCHUNK_MAX = MFMA_KCHUNK;     // staged columns: a multiple of MSTEP
constexpr int MWPB = MFMA_WAVES_PER_BLOCK;
constexpr int XROW_PAD = 16;                    // bytes between staged rows: 16 rows of one column hit 16 bank groups

#ifndef MFMA_LOAD_AUX
#define MFMA_LOAD_AUX 0   // cache policy bits of the weight loads (non-temporal, 2, measures 5-10 % slower: the two
                          // halves of a 128-byte line are fetched by consecutive instructions)
#endif
__device__ __forceinline__ half8 buf_load8(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
    return __builtin_bit_cast(half8, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, MFMA_LOAD_AUX));
}

constexpr int MGROUPS = 4;                      // most 16-row groups one wave owns

__global__ __launch_bounds__(64 * MWPB) void helix_gemv_f16_mfma_kernel(const Params p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, q = lane >> 4;
    const int m0 = blockIdx.y * 16;
    const int k_begin = (int)blockIdx.z * p.kchunk;                 // K range of this workgroup: a multiple of MSTEP
    const int k_end = (k_begin + p.kchunk) < p.K ? (k_begin + p.kchunk) : p.K;
    constexpr int XC = MFMA_KCHUNK_MAX;                              // columns staged at a time
    constexpr int xrow = XC * 2 + XROW_PAD;                          // bytes per staged activation row

    const int ngroups = (p.N + 15) / 16;
    const int group_first = (blockIdx.x * MWPB + wave) * p.rows_per_wave;      // in units of 16-row groups
    const int group_last = (group_first + p.rows_per_wave) < ngroups ? (group_first + p.rows_per_wave) : ngroups;

    // weights of 16-row group g: load c of a step reads, in lane (r, q), columns 32*c + 8*q .. +7 of row r -- one
    // instruction covers 64 contiguous bytes of each of 16 rows, the eight loads of a step 512 contiguous bytes
    // per row.  Rows beyond N read as zeros (buffer bounds).
    auto w_rsrc = [&](int g) -> __amdgpu_buffer_rsrc_t {
        const int n0 = g * 16;
        const int rows_w = (p.N - n0) < 16 ? (p.N - n0) : 16;
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(p.B + (size_t)n0 * p.ldb), 0,
                                                 (int)(((size_t)(rows_w - 1) * p.ldb + p.K) * 2), 0x00020000);
    };
    const int woff = (r * p.ldb + 8 * q) * 2;
    const unsigned char* xl = smem + r * xrow + 8 * q * 2;           // this lane's activation row and column base

    floatx4 acc[MGROUPS];
#pragma unroll
    for (int gi = 0; gi < MGROUPS; gi++) acc[gi] = floatx4{0.f, 0.f, 0.f, 0.f};

    // The K range is walked in chunks of XC columns: the workgroup stages 16 activation rows of the chunk in
    // LDS, then every wave streams the chunk's columns of each of its row groups.
    for (int kc = k_begin; kc < k_end; kc += XC) {
        const int ce = (kc + XC) < k_end ? (kc + XC) : k_end;
        __syncthreads();                                              // the previous chunk has been read
        {
            constexpr int chunks_per_row = XC / 8;
            constexpr int total = 16 * chunks_per_row;
            for (int c = tid; c < total; c += 64 * MWPB) {
                const int m = c / chunks_per_row, kk = (c % chunks_per_row) * 8;
                intx4 v = {0, 0, 0, 0};
                if (m0 + m < p.M && kc + kk < ce) v = *(const intx4*)(p.A + (size_t)(m0 + m) * p.lda + kc + kk);
                *(intx4*)(smem + m * xrow + kk * 2) = v;
            }
        }
        __syncthreads();

#pragma unroll
        for (int gi = 0; gi < MGROUPS; gi++) {
            const int g = group_first + gi;
            if (g >= group_last) break;
            const __amdgpu_buffer_rsrc_t rw = w_rsrc(g);
            half8 wa[MCH], wb[MCH];
            auto load_step = [&](half8 (&w)[MCH], int k) {
                if (k + MSTEP <= ce) {
#pragma unroll
                    for (int c = 0; c < MCH; c++) w[c] = buf_load8(rw, woff + c * 64, k * 2);
                } else {   // partial step: columns beyond the chunk read zeros
#pragma unroll
                    for (int c = 0; c < MCH; c++)
                        w[c] = buf_load8(rw, (k + 32 * c + 8 * q < ce) ? woff + c * 64 : 0x7fffffff, k * 2);
                }
            };
            auto mfma_step = [&](const half8 (&w)[MCH], int k) {
#pragma unroll
                for (int c = 0; c < MCH; c++) {
                    const half8 xv = *(const half8*)(xl + (k - kc) * 2 + c * 64);
                    acc[gi] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w[c], xv, acc[gi], 0, 0, 0);
                }
            };
            // double-buffered steps: step s+1 is requested before the MFMAs of step s
            load_step(wa, kc);
            int k = kc;
            for (; k + 2 * MSTEP < ce; k += 2 * MSTEP) {
                load_step(wb, k + MSTEP);
                mfma_step(wa, k);
                load_step(wa, k + 2 * MSTEP);
                mfma_step(wb, k + MSTEP);
            }
            if (k + MSTEP < ce) {
                load_step(wb, k + MSTEP);
                mfma_step(wa, k);
                mfma_step(wb, k + MSTEP);
            } else {
                mfma_step(wa, k);
            }
        }
    }

    // lane l holds y[m0 + l % 16][n0 + 4*(l/16) + {0..3}] of each of its groups
#pragma unroll
    for (int gi = 0; gi < MGROUPS; gi++) {
        const int g = group_first + gi;
        if (g >= group_last) break;
        const int m = m0 + r, n = g * 16 + 4 * q;
        if (m < p.M && n < p.N) {
            if (p.ksplit > 1) {
                float* dst = p.ws + ((size_t)blockIdx.z * p.M + m) * p.N + n;
                if ((p.N & 3) == 0) *(floatx4*)dst = acc[gi];
                else
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (n + e < p.N) dst[e] = acc[gi][e];
            } else {
                half_t* dst = p.C + (size_t)m * p.ldc + n;
                if ((p.ldc & 3) == 0 && (((uintptr_t)p.C) & 7) == 0 && n + 4 <= p.N) {
                    half4 h = {(half_t)acc[gi][0], (half_t)acc[gi][1], (half_t)acc[gi][2], (half_t)acc[gi][3]};
                    *(half4*)dst = h;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (n + e < p.N) dst[e] = (half_t)acc[gi][e];
                }
            }
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
    static char buf[1024];
    static bool done = false;
    if (!done) {
        snprintf(buf, sizeof(buf),
                 "{\"family\": \"gemv_f16\", \"arch\": \"gfx950\", \"mfma\": \"none below %d activation rows, v_mfma_f32_16x16x32_f16 from there\", \"lds_stages\": 0, "
                 "\"block_rows\": 1, \"block_cols\": 128, \"wave_rows\": 0, \"wave_cols\": 0, \"split_k\": %d, "
                 "\"threads\": %d, \"lds_bytes\": %d, \"k_step\": %d, "
                 "\"layout_a\": \"M x K row-major f16 (activations)\", "
                 "\"layout_b\": \"N x K row-major f16 (streamed weights)\", \"layout_c\": \"M x N row-major f16\", "
                 "\"accumulate\": \"f32\", \"k_multiple\": 8, \"ld_multiple\": 8}",
                 MFMA_MIN_M, SPLITK, 64 * WPB, X_LDS_BYTES, KSTEP);
        done = true;
    }
    return buf;
}

constexpr int mtile_of(int M) { return M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : M <= 8 ? 8 : 16; }

// K partitioning: enough ranges that M_TILE activation rows of one range fit X_LDS_BYTES_WIDE, at least SPLIT_K
// MFMA variant: K is partitioned only to give the launch enough waves (one wave owns up to MGROUPS groups of
// 16 weight rows): ranges are multiples of 256, at least 1024 wide, at least SPLIT_K of them
inline void k_partition_mfma(int N, int K, int* kchunk, int* ksplit) {
    const int steps = (K + MSTEP - 1) / MSTEP;
    const long long groups = (N + 15) / 16;
    long long split = (MFMA_TARGET_WAVES / 2 + groups - 1) / groups;     // aim for half the target before splitting
    const long long max_split = steps / 4 > 1 ? steps / 4 : 1;
    if (split > max_split) split = max_split;
    if (split < SPLITK) split = SPLITK;
    if (split > steps) split = steps;
    if (split < 1) split = 1;
    const int per = (int)((steps + split - 1) / split);
    *kchunk = per * MSTEP;
    *ksplit = (steps + per - 1) / per;
}

inline void k_partition(int M, int N, int K, int* kchunk, int* ksplit) {
    if (M >= MFMA_MIN_M) return k_partition_mfma(N, K, kchunk, ksplit);
    const int mt = mtile_of(M);
    const int steps = (K + KSTEP - 1) / KSTEP;
    int max_steps = X_LDS_BYTES_WIDE / (mt * KSTEP * 2);
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
    k_partition(M, N, K, &kchunk, &ksplit);
    return ksplit > 1 ? (size_t)ksplit * (size_t)M * (size_t)N * sizeof(float) : 0;
}

inline void bench_layout(int M, int N, int K, size_t* ae, size_t* be, size_t* ce, int* lda, int* ldb, int* ldc) {
    *ae = (size_t)M * K; *be = (size_t)N * K; *ce = (size_t)M * N;
    *lda = K; *ldb = K; *ldc = N;
}

template <int MT, int ROWS, int KU, int WAVES>
inline int launch_waves(Params p, int lds, hipStream_t s) {
    const int waves = (p.N + p.rows_per_wave - 1) / p.rows_per_wave;
    static int attr_rc = (int)hipFuncSetAttribute((const void*)helix_gemv_f16_kernel<MT, ROWS, KU, WAVES>,
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (attr_rc) return attr_rc;
    dim3 grid((waves + WAVES - 1) / WAVES, (p.M + MT - 1) / MT, p.ksplit), block(64 * WAVES);
    hipLaunchKernelGGL((helix_gemv_f16_kernel<MT, ROWS, KU, WAVES>), grid, block, lds, s, p);
    return (int)hipGetLastError();
}

template <int MT, int ROWS, int KU>
inline int launch_cfg(Params p, hipStream_t s) {
    // consecutive rows per wave: a multiple of ROWS that brings the launch near TARGET_WAVES waves
    long long want = ((long long)p.N * p.ksplit + TARGET_WAVES - 1) / TARGET_WAVES;
    if (want < 1) want = 1;
    p.rows_per_wave = (int)((want + ROWS - 1) / ROWS) * ROWS;
    const int lds = MT * p.kchunk * 2;
    if (lds > X_LDS_BYTES) return launch_waves<MT, ROWS, KU, 2 * WPB>(p, lds, s);
    return launch_waves<MT, ROWS, KU, WPB>(p, lds, s);
}

inline int launch_mfma(Params p, hipStream_t s) {
    if ((long long)16 * p.ldb * 2 >= 0x7fffffffLL) return HELIX_ERR_INVALID_VALUE;
    const long long groups = (p.N + 15) / 16;
    // 16-row groups per wave: as many (up to MGROUPS) as keep the launch near MFMA_TARGET_WAVES waves; the
    // staged activations are shared by all groups a workgroup walks
    long long gpw = (groups * p.ksplit + MFMA_TARGET_WAVES - 1) / MFMA_TARGET_WAVES;
    if (gpw < 1) gpw = 1;
    if (gpw > MGROUPS) gpw = MGROUPS;
    p.rows_per_wave = (int)gpw;
    const long long waves = (groups + gpw - 1) / gpw;
    const int lds = 16 * (MFMA_KCHUNK_MAX * 2 + XROW_PAD);
    dim3 grid((unsigned)((waves + MWPB - 1) / MWPB), (p.M + 15) / 16, p.ksplit), block(64 * MWPB);
    hipLaunchKernelGGL(helix_gemv_f16_mfma_kernel, grid, block, lds, s, p);
    return (int)hipGetLastError();
}

inline int gemm(const void* A, const void* B, void* C, int M, int N, int K, int lda, int ldb, int ldc, void* ws,
                size_t ws_bytes, hipStream_t s) {
    if (K % 8 != 0 || lda % 8 != 0 || ldb % 8 != 0) return HELIX_ERR_INVALID_VALUE;
    if (lda < K || ldb < K || ldc < N) return HELIX_ERR_INVALID_VALUE;
    if (((uintptr_t)A & 15) || ((uintptr_t)B & 15) || ((uintptr_t)C & 1)) return HELIX_ERR_INVALID_VALUE;
    if ((M + 15) / 16 > 65535) return HELIX_ERR_INVALID_VALUE;
    Params p{(const half_t*)A, (const half_t*)B, (half_t*)C, (float*)ws, M, N, K, lda, ldb, ldc, 0, 1, 1};
    k_partition(M, N, K, &p.kchunk, &p.ksplit);
    if (p.ksplit > 65535) return HELIX_ERR_INVALID_VALUE;
    if (p.ksplit > 1) {
        if (!ws || ws_bytes < workspace_bytes(M, N, K)) return HELIX_ERR_WORKSPACE;
    }
    int rc;
    // activation-row tile, like the reference's N_TILE pick from the skinny extent (gemv.cu:232-250); wider
    // tiles take more weight rows per pass so that one LDS read of the activations feeds several rows
    if (M >= MFMA_MIN_M) rc = launch_mfma(p, s);
    else switch (mtile_of(M)) {
        case 1: rc = launch_cfg<1, GEMV_R1, GEMV_KU1>(p, s); break;
        case 2: rc = launch_cfg<2, GEMV_R2, GEMV_KU2>(p, s); break;
        case 4: rc = launch_cfg<4, GEMV_R4, GEMV_KU4>(p, s); break;
        case 8: rc = launch_cfg<8, GEMV_R8, GEMV_KU8>(p, s); break;
        default: rc = launch_cfg<16, GEMV_R16, GEMV_KU16>(p, s); break;
    }
    if (rc) return rc;
    if (p.ksplit > 1) {
        size_t total = (size_t)M * N;
        int blocks = (int)((total + 255) / 256);
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL(helix_gemv_splitk_reduce_kernel, dim3(blocks), dim3(256), 0, s, (const float*)ws,
                           (half_t*)C, M, N, ldc, p.ksplit);
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
