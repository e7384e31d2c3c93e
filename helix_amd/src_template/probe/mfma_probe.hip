// MFMA-only loop for MI355X (gfx950): the rate the matrix pipes sustain when nothing else runs, on seeded and on
// all-zero operands.  On seeded operands the part runs against its power limit (the engine clock settles well below
// the 2.4 GHz of the datasheet peak), which bounds every GEMM kernel, the vendor's included; this probe measures
// that bound.  Same instruction (v_mfma_f32_16x16x32_f16), same accumulator and fragment counts per wave and same
// waves per compute unit as the 256 x 256 x 64 tile of src_template/MI355X_FP16/gemm.hip with 64 x 128 wave tiles.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "helix_probe.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int TM = 4, TN = 8, KSTEPS = 2, WAVES = 8, NTHREADS = 64 * WAVES, NWG = 256;
constexpr int FRAGS = KSTEPS * (TM + TN);          // half8 fragments per lane

__global__ void fill_kernel(_Float16* p, size_t n, float scale) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        uint32_t h = (uint32_t)i * 2654435761u + 12345u;
        h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
        p[i] = (_Float16)(((float)(h & 0xffffu) * (1.0f / 32768.0f) - 1.0f) * scale);
    }
}

__global__ __launch_bounds__(NTHREADS) void helix_mfma_probe_kernel(const half8* operands, float* sink, int loops) {
    const size_t t = (size_t)blockIdx.x * NTHREADS + threadIdx.x;
    half8 a[KSTEPS][TM], b[KSTEPS][TN];
#pragma unroll
    for (int s = 0; s < KSTEPS; s++) {
#pragma unroll
        for (int i = 0; i < TM; i++) a[s][i] = operands[t * FRAGS + s * (TM + TN) + i];
#pragma unroll
        for (int j = 0; j < TN; j++) b[s][j] = operands[t * FRAGS + s * (TM + TN) + TM + j];
    }
    floatx4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < loops; it++) {
#pragma unroll
        for (int s = 0; s < KSTEPS; s++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int i = 0; i < TM; i++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b[s][j], a[s][i], acc[i][j], 0, 0, 0);
    }
    float total = 0.f;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) total += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
    sink[t] = total;
}

}  // namespace

extern "C" int helix_mfma_probe(int zero_operands, int warmup, int launches, int loops, double* seconds_per_launch,
                                double* flop_per_launch) {
    if (launches <= 0 || loops <= 0 || warmup < 0 || !seconds_per_launch || !flop_per_launch) return (int)hipErrorInvalidValue;
    const size_t threads = (size_t)NWG * NTHREADS, halves = threads * FRAGS * 8;
    _Float16* operands = nullptr;
    float* sink = nullptr;
    hipError_t e = hipMalloc((void**)&operands, halves * 2);
    if (e != hipSuccess) return (int)e;
    e = hipMalloc((void**)&sink, threads * 4);
    if (e != hipSuccess) { (void)hipFree(operands); return (int)e; }
    // uniform in [-0.1732, 0.1732): standard deviation 0.1, like the seeded GEMM operands
    hipLaunchKernelGGL(fill_kernel, dim3(4096), dim3(256), 0, nullptr, operands, halves, zero_operands ? 0.0f : 0.17320508f);
    hipEvent_t start = nullptr, stop = nullptr;
    float ms = 0.f;
    e = hipGetLastError();
    if (e == hipSuccess) e = hipEventCreate(&start);
    if (e == hipSuccess) e = hipEventCreate(&stop);
    if (e == hipSuccess) {
        for (int i = 0; i < warmup; i++)
            hipLaunchKernelGGL(helix_mfma_probe_kernel, dim3(NWG), dim3(NTHREADS), 0, nullptr, (const half8*)operands, sink, loops);
        e = hipEventRecord(start, nullptr);
        for (int i = 0; i < launches; i++)
            hipLaunchKernelGGL(helix_mfma_probe_kernel, dim3(NWG), dim3(NTHREADS), 0, nullptr, (const half8*)operands, sink, loops);
        if (e == hipSuccess) e = hipGetLastError();
        if (e == hipSuccess) e = hipEventRecord(stop, nullptr);
        if (e == hipSuccess) e = hipEventSynchronize(stop);
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, start, stop);
    }
    if (start) (void)hipEventDestroy(start);
    if (stop) (void)hipEventDestroy(stop);
    (void)hipFree(operands);
    (void)hipFree(sink);
    if (e != hipSuccess) return (int)e;
    *seconds_per_launch = (double)ms / 1000.0 / launches;
    *flop_per_launch = (double)NWG * WAVES * (double)loops * KSTEPS * TM * TN * (2.0 * 16 * 16 * 32);
    return 0;
}
