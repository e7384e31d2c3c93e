// K partitions summed inside the launch: the part of split-K that the FP16 and FP32 tile templates share.
//
// A problem of few output tiles and a long K is partitioned along K so that every compute unit gets a workgroup; the
// partitions of a tile leave FP32 partial tiles in the workspace, which have to be added in partition order
// (deterministic: the reference's split-K adds FP16 atomics into C instead, src_template/Ampere_FP16/gemm_splitK.cu:495-506).
//
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
//     same FP32 additions as the reduction kernel, so both paths give identical bits), resets the counter and stores
//     the result (straight from the sums: the partial tiles are read row by row, not in the MFMA layout);
//   * a workgroup that finds itself on another XCD than expected adds the device-scope release, and tells the
//     tile's last workgroup through the counter's upper half to add the acquire: correct on any placement, fast on
//     the expected one.
// Measured on FP16 196 x 512 x 4608 (64 x 64 tiles, 8 partitions): 3.3 us from the last partial store to the end of
// the launch (arrival 1.8 us, sum 1.5 us) against 5.0 us for the second kernel and the gap in front of it.  Fetching
// the counter's cache line ahead of the arrival (an atomic add of zero at the start of the kernel, or next to the
// partial stores) was measured as well and is 0.5 - 0.7 us slower: it holds up the loads behind it.
//
// The second kernel stays as the fallback: N not a multiple of 4, more than MAX_TILES tiles, partials beyond 2 GiB, a
// device whose workgroup deal is irregular, or HELIX_SPLITK_REDUCE=kernel in the environment.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <mutex>

namespace helix_splitk {

constexpr int MAX_TILES = 1024;   // arrival counters per launch
constexpr int ARRIVE_SETS = 8;    // sets used in turn: that many launches of one library may be in flight on a GPU
constexpr int OOB_OFFSET = 0x7fffffff;

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));

// The kernel-side description of a launch (part of the kernel's parameter block).
struct Plan {
    int fused;          // 0: partitions over blockIdx.y, a second kernel adds them.  1: one-dimensional grid, workgroup
                        // id L runs partition (L / 8) % splits of tile number (L / 8) / splits of XCD L % 8
    unsigned xcc_map;   // XCC_ID the hardware reports for workgroup ids 0 .. 7 (ids are dealt round-robin), 4 bits each
    unsigned* arrive;   // one arrival counter per output tile, zero between launches
};

// Which tile (numbered XCD by XCD: XCD x is given the compact run [x * per + min(x, rem), ...) of the ntiles tiles)
// and which K partition a workgroup works on; idle: an id beyond the tiles of its XCD (grids are whole rounds of 8).
struct Unit {
    int tile, split;
    bool idle;
};

__device__ __forceinline__ Unit unit_of_workgroup(const Plan& plan, int ntiles, int splits) {
    const int per = ntiles / 8, rem = ntiles % 8;
    const int xcd = (int)blockIdx.x % 8, j = (int)blockIdx.x / 8;
    if (plan.fused) {
        const int slot = j / splits;
        return Unit{xcd * per + (xcd < rem ? xcd : rem) + slot, j - slot * splits, slot >= per + (xcd < rem ? 1 : 0)};
    }
    return Unit{xcd * per + (xcd < rem ? xcd : rem) + j, (int)blockIdx.y, false};
}

__device__ __forceinline__ unsigned xcc_id() {   // HW_REG_XCC_ID (register 20), XCC_ID = bits 3:0
    return (unsigned)__builtin_amdgcn_s_getreg((4 - 1) << 11 | 0 << 6 | 20) & 15u;
}

__device__ __forceinline__ void store_chunk(_Float16* dst, floatx4 v, bool wide) {
    const half4 h = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
    if (wide) {
        *(half4*)dst = h;
    } else {
#pragma unroll
        for (int e = 0; e < 4; e++) dst[e] = h[e];
    }
}
__device__ __forceinline__ void store_chunk(float* dst, floatx4 v, bool wide) {
    if (wide) {
        *(floatx4*)dst = v;
    } else {
#pragma unroll
        for (int e = 0; e < 4; e++) dst[e] = v[e];
    }
}

// The threads of a workgroup walk a TILE_ROWS x TILE_COLS tile linearly (thread t takes the four-column chunks t,
// t + THREADS, ...),
// add the first PARTS partitions of each chunk in order (partitions beyond `splits` read as zeros through the buffer
// bounds check and add nothing) and store four results.  BATCH chunks x PARTS partitions of loads are in flight per
// thread.
template <typename OutT, int TILE_ROWS, int TILE_COLS, int THREADS, int PARTS, int BATCH>
__device__ __forceinline__ void sum_partitions(const float* ws, OutT* C, int M, int N, int ldc, int splits, int m0, int n0,
                                               int tid) {
    constexpr int CH_PER_ROW = TILE_COLS / 4, PER_THREAD = (TILE_ROWS * CH_PER_ROW + THREADS - 1) / THREADS;
    const int slice_bytes = M * N * 4;                    // one partition; the host keeps splits * slice below 2^31
    // cache policy sc0 | sc1: past this compute unit's vector cache, to the L2 the partials were written to
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(ws), 0,
                                                                        (int)((unsigned)splits * (unsigned)slice_bytes), 0x00020000);
    const bool wide = (((uintptr_t)C % (4 * sizeof(OutT))) == 0) && (ldc % 4 == 0);
    for (int c0 = 0; c0 < PER_THREAD; c0 += BATCH) {
        floatx4 v[BATCH][PARTS];
        int row[BATCH], col[BATCH];
#pragma unroll
        for (int b = 0; b < BATCH; b++) {
            const int chunk = tid + (c0 + b) * THREADS;
            // chunks beyond the tile (a last batch that is not full, a tile that does not divide over the threads)
            // are masked out by row
            row[b] = (chunk < TILE_ROWS * CH_PER_ROW) ? m0 + chunk / CH_PER_ROW : M;
            col[b] = n0 + (chunk % CH_PER_ROW) * 4;
            const int voff = (row[b] < M && col[b] < N) ? (row[b] * N + col[b]) * 4 : OOB_OFFSET;
            // the partition's offset goes into the per-lane offset, the one the bounds check looks at
#pragma unroll
            for (int k = 0; k < PARTS; k++) {
                const int off = (k < splits && voff != OOB_OFFSET) ? voff + k * slice_bytes : OOB_OFFSET;
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
            if (row[b] < M && col[b] < N)                 // N is a multiple of 4 on this path: whole chunks
                store_chunk(C + (size_t)row[b] * ldc + col[b], sum, wide);
        }
    }
}

typedef __attribute__((address_space(3))) unsigned char* lds_bytes_t;

// Called by every thread of the workgroup once its partial tile is stored (smem: four bytes of LDS that no wave of
// the workgroup still reads): counts the workgroup in and, in the one workgroup whose arrival completes the tile, adds
// the partitions and stores the result.  MAX_PARTS: the most partitions a launch of this library uses (at most 8).
// LOADS: 16-byte loads a thread keeps in flight while adding (8, 16 or 32: chunks of up to four or up to eight
// partitions); their registers count towards the kernel's allocation, so a template picks what its main loop already
// uses -- 32 where LDS keeps the kernel to two waves per SIMD anyway.
template <typename OutT, int TILE_ROWS, int TILE_COLS, int THREADS, int MAX_PARTS, int LOADS>
__device__ __forceinline__ void sum_partitions_if_last(const Plan& plan, const float* ws, OutT* C, int M, int N, int ldc,
                                                       int splits, int tile, int m0, int n0, int tid, unsigned char* smem) {
    static_assert(LOADS == 8 || LOADS == 16 || LOADS == 32, "8, 16 or 32 loads in flight");
    const bool placed = xcc_id() == ((plan.xcc_map >> (4 * ((unsigned)blockIdx.x % 8u))) & 15u);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // this wave's partial sums have reached the L2
    if (!placed) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    __syncthreads();                                      // ... and every other wave's
    volatile __attribute__((address_space(3))) unsigned* flag =
        (volatile __attribute__((address_space(3))) unsigned*)(lds_bytes_t)smem;
    if (tid == 0) {
        *flag = __hip_atomic_fetch_add(plan.arrive + tile, placed ? 1u : 0x10001u, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    const unsigned old = *flag;
    if ((int)(old & 0xffffu) + 1 != splits) return;
    if ((old >> 16) != 0 || !placed) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    if (tid == 0) __hip_atomic_store(plan.arrive + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    constexpr int FEW = MAX_PARTS < 4 ? MAX_PARTS : 4;    // launches of up to four partitions read no further ones
    if (MAX_PARTS <= 4 || splits <= 4)
        sum_partitions<OutT, TILE_ROWS, TILE_COLS, THREADS, FEW, (LOADS / 2 / FEW > 0 ? LOADS / 2 / FEW * 2 : 1)>(ws, C, M, N, ldc, splits, m0, n0, tid);
    else
        sum_partitions<OutT, TILE_ROWS, TILE_COLS, THREADS, MAX_PARTS, (LOADS / MAX_PARTS > 0 ? LOADS / MAX_PARTS : 1)>(ws, C, M, N, ldc, splits, m0, n0, tid);
}

// ---- host side --------------------------------------------------------------------------------------------------
// HELIX_SPLITK_ENABLED = 0 (a library that never partitions K) leaves the counters, the probe and the per-device state
// out of the library; plan_launch then always answers "second-kernel path".
#ifndef HELIX_SPLITK_ENABLED
#define HELIX_SPLITK_ENABLED 1
#endif
#if HELIX_SPLITK_ENABLED
namespace {

// Arrival counters: they live in the library's device image, are zero when the code object is loaded, and every
// launch leaves them zero.
static __device__ unsigned arrive_cells[ARRIVE_SETS * MAX_TILES];

// Workgroup id -> XCC_ID as the hardware deals a one-dimensional grid, recorded once per device.
__global__ void helix_xcc_probe_kernel(unsigned* out) {
    if (threadIdx.x == 0) out[blockIdx.x] = xcc_id();
}

}  // namespace

struct DeviceState {
    int state = 0;               // 0: not looked at yet; 1: usable; -1: not usable on this device (second kernel instead)
    unsigned* arrive = nullptr;  // device address of arrive_cells on this device
    unsigned xcc_map = 0;
};

// Per device, on first use: where the counters live and which XCC_ID the round-robin deal gives workgroup ids
// 0 .. 7 (probed with a 64-workgroup launch; an irregular deal, any HIP error, or HELIX_SPLITK_REDUCE=kernel in the
// environment leaves the second-kernel path in charge).  The probe synchronises the device once; it must not
// happen under stream capture, like any first launch of a library.
inline const DeviceState& device_state() {
    static DeviceState per_device[64];
    static std::mutex lock;
    static const DeviceState none{-1, nullptr, 0};
    int d = -1;
    if (hipGetDevice(&d) != hipSuccess || d < 0 || d >= 64) return none;
    std::lock_guard<std::mutex> hold(lock);
    DeviceState& f = per_device[d];
    if (f.state != 0) return f;
    f.state = -1;
    const char* how = getenv("HELIX_SPLITK_REDUCE");
    if (how && strcmp(how, "kernel") == 0) return f;
    unsigned* base = nullptr;
    constexpr int PROBE = 64;
    unsigned seen[PROBE];
    bool ok = hipGetSymbolAddress((void**)&base, HIP_SYMBOL(arrive_cells)) == hipSuccess && base != nullptr;
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
    if (getenv("HELIX_DEBUG"))
        fprintf(stderr, "helix: device %d deals workgroup ids 0..7 to XCC_IDs 0x%08x (nibble per id)\n", d, map);
    return f;
}

// Fills `plan` for a launch of ntiles tiles x splits partitions of an M x N result and returns the one-dimensional
// grid size of a launch that adds its partitions itself, or returns 0 (plan.fused = 0) when the launch takes the
// second-kernel path.
inline unsigned plan_launch(Plan& plan, long long ntiles, int splits, long long M, long long N) {
    static std::atomic<unsigned> launches{0};
    plan.fused = 0;
    // byte offsets into the partials are 32-bit; chunks of four columns must not straddle the edge of C
    if (splits < 2 || ntiles > MAX_TILES || (long long)splits * M * N * 4 >= 0x7fffffffLL || N % 4 != 0) return 0;
    const DeviceState& f = device_state();
    if (f.state != 1) return 0;
    plan.fused = 1;
    plan.xcc_map = f.xcc_map;
    plan.arrive = f.arrive + (launches.fetch_add(1) % ARRIVE_SETS) * MAX_TILES;
    const long long slots = (ntiles + 7) / 8;            // most tiles any XCD is given
    return (unsigned)(8 * slots * splits);
}
#else
inline unsigned plan_launch(Plan& plan, long long, int, long long, long long) {
    plan.fused = 0;
    return 0;
}
#endif

}  // namespace helix_splitk
