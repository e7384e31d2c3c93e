/*
 * helix_abi.h -- C ABI exported by every MI355X (gfx950) Helix kernel-template library.
 *
 * One shared library == one instantiated kernel template, the way one executable is one
 * instantiated template in the reference (scripts/Ampere_FP16/build_Ampere_FP16.py:7-28 builds
 * `gemm_{K_STAGE}_{BLOCK_ROWS}_{BLOCK_COLS}_{WARP_ROWS}_{WARP_COLS}`; here the same parameters give
 * `libgemm_{K_STAGES}_{BLOCK_ROWS}_{BLOCK_COLS}_{WAVE_ROWS}_{WAVE_COLS}_{BLOCK_K}.so`).  Every library exports
 * every symbol below, so the host side binds one ctypes signature set and swaps libraries per
 * configuration.  An entry point a template does not implement returns HELIX_ERR_UNSUPPORTED.
 *
 * Conventions
 *   - plain pointers and sizes only; device pointers come from hipMalloc (or any allocator layered
 *     on it); the library allocates no device memory.  Its state is a one-time function-attribute
 *     initialisation and what its device image holds: the scratch array of helix_gemm_static_scratch and, in
 *     split-K libraries, 32 KiB of tile arrival counters (zero between launches) with the workgroup-id ->
 *     XCD deal of the device, probed by the first split-K launch (one device synchronisation, so that first
 *     launch must not happen under stream capture).  At most eight launches of one split-K library may be
 *     in flight on one GPU at a time (they take turns on eight counter sets).
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *   - return value: 0 on success, a positive hipError_t value if the HIP runtime failed, or one of
 *     the HELIX_ERR_* codes.  Nothing throws, exits or prints.
 *   - a shape the template cannot run (alignment, pipeline depth) is reported as
 *     HELIX_ERR_INVALID_VALUE; nothing is launched.  (The reference launches anyway and reads out
 *     of bounds.)
 *
 * Operand layouts (fixed per template family; `helix_info` reports them)
 *   gemm_f16 / gemv_f16 : C[M x N] = A[M x K] * B[N x K]^T, row-major, FP16 in, FP32 accumulate,
 *                         FP16 out.  B is stored N x K like the reference FP16 kernels
 *                         (src_template/Ampere_FP16/gemm.cu:144,597-601).
 *   sgemm_f32           : C[M x N] = A^T * B with A stored K x M and B stored K x N, row-major FP32,
 *                         like the reference FP32 kernel (src_template/Ampere_FP32/sgemm.cu:138,378-382).
 *   gemv_f32            : as gemv_f16 with FP32 everywhere
 *                         (src_template/Ampere_FP32/gemv_template_fp32.cu:153-217).
 *   conv2d              : y[B,OH,OW,OC] = conv(x[B,H,W,IC], w[OC,kH,kW,IC]), zero padding, as an
 *                         implicit GEMM with M=B*OH*OW, N=OC, K=kH*kW*IC
 *                         (shape algebra scripts/Ampere_FP16/Ampere_FP16_conv.py:432-434; replaces the
 *                         explicit src_template/Ampere_FP16/im2col.cu:38-97 pass plus GEMM).
 */
#ifndef HELIX_ABI_H
#define HELIX_ABI_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Only the entry points below are exported; everything else in a template library has hidden visibility
 * (the libraries are built with -fvisibility=hidden -Wl,-Bsymbolic), so two configurations can live in one
 * process, however they are opened, without binding to each other's tile code. */
#define HELIX_API __attribute__((visibility("default")))

#define HELIX_OK 0
#define HELIX_ERR_INVALID_VALUE 1 /* same value as hipErrorInvalidValue */
#define HELIX_ERR_UNSUPPORTED 801 /* same value as hipErrorNotSupported */
#define HELIX_ERR_WORKSPACE 2001  /* workspace pointer NULL or too small */

/* Writes a NUL-terminated JSON object describing the instantiated template (family, tile / wave /
 * LDS parameters, threads per workgroup, LDS bytes, operand layouts, shape constraints) into `json`.
 * Returns the number of bytes needed including the NUL; if that exceeds `cap` nothing is written.
 * Replaces: the configuration encoded in the reference's executable names
 * (scripts/Ampere_FP16/build_Ampere_FP16.py:13-27, scripts/Ampere_FP32/build_Ampere_FP32.py:18). */
HELIX_API int helix_info(char* json, int cap);

/* Bytes of device scratch `helix_gemm` needs for this shape (0 unless the template splits K).
 * Replaces: nothing -- the reference's split-K accumulates with FP16 atomics into C
 * (src_template/Ampere_FP16/gemm_splitK.cu:495-506); here partial sums go through an FP32 workspace and are
 * added in partition order, inside the launch by the last workgroup of a tile to finish or (environment
 * HELIX_SPLITK_REDUCE=kernel, N not a multiple of 4, more than 1024 tiles, an irregular XCD deal) by a second
 * kernel; both give the same bits. */
HELIX_API size_t helix_workspace_bytes(int M, int N, int K);

/* One GEMM / GEMV launch on `stream`.  lda/ldb/ldc are row strides in elements.
 * Replaces: the launchers `void f(half*, half*, half*, int M, int N, int K)`
 * (src_template/Ampere_FP16/gemm.cu:551-565, gemv.cu:218-252, gemv_splitK.cu:224-260) and
 * `mySgemmCPAsyncTemplate<<<>>>(a, b, c, M, N, K)` (src_template/Ampere_FP32/sgemm.cu:97,634). */
HELIX_API int helix_gemm(const void* A, const void* B, void* C, int M, int N, int K, int lda, int ldb, int ldc,
               void* workspace, size_t workspace_bytes, void* stream);

/* `helix_gemm` for callers that cannot allocate device memory or pass a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): the K-partition partial sums go to a
 * fixed array of HELIX_STATIC_SCRATCH_BYTES inside the library's device image, so the call allocates
 * nothing and needs no workspace argument.  Same kernels, same results as `helix_gemm` with the workspace
 * `helix_workspace_bytes` asks for.  A shape that needs more than HELIX_STATIC_SCRATCH_BYTES returns
 * HELIX_ERR_WORKSPACE and launches nothing; the vendor comparator libraries return HELIX_ERR_UNSUPPORTED.
 * All calls on one GPU share that GPU's array: calls that overlap on one GPU (different streams or host
 * threads) race on it; calls on one stream are ordered and safe.  The array keeps the last call's
 * contents; nothing needs clearing because a launch writes every partial sum it later reads.  The first
 * launch of a library on a device loads its code object like any first launch: warm up before capturing.
 * No counterpart in the reference: it exists for the callers named above, those that cannot allocate. */
#define HELIX_STATIC_SCRATCH_BYTES (16u << 20)
HELIX_API int helix_gemm_static_scratch(const void* A, const void* B, void* C, int M, int N, int K, int lda, int ldb,
                                        int ldc, void* stream);

/* Bytes of device scratch `helix_conv2d` needs for this problem: the split-K partial sums of the implicit
 * GEMM, plus -- when IC is not a multiple of the 16-byte gather chunk (8 halves / 4 floats) -- the
 * channel-padded copies of activations and weights, or (IC = 1; 2 in FP16) the column buffer and repacked
 * weights of the explicit im2col path.
 * Replaces: the `col` buffer the reference's im2col executable allocates for itself
 * (src_template/Ampere_FP16/im2col.cu:140-150). */
HELIX_API size_t helix_conv_workspace_bytes(int batch, int H, int W, int IC, int OC, int kH, int kW, int stride, int pad);

/* One NHWC convolution on `stream`: implicit GEMM (no column buffer) when IC is a multiple of the gather
 * chunk; else the same on copies with the channels zero-padded to the chunk, or (IC = 1; 2 in FP16) im2col
 * into the workspace followed by the GEMM, as the reference does for every layer.
 * Replaces: `im2col batch IC H W OC kH kW stride pad` followed by the GEMM executable
 * (scripts/Ampere_FP16/Ampere_FP16_conv.py:431-446, src_template/Ampere_FP16/im2col.cu:38-97). */
HELIX_API int helix_conv2d(const void* x, const void* w, void* y, int batch, int H, int W, int IC, int OC, int kH,
                 int kW, int stride, int pad, void* workspace, size_t workspace_bytes, void* stream);

/* Times caller-owned buffers: `warmup` untimed launches, then `iters` launches between two HIP
 * events recorded on `stream`; *avg_s = elapsed / iters in seconds.
 * Replaces: the event-timed loop of testF16F16GemmPerformance
 * (src_template/Ampere_FP16/gemm.cu:636-652) for callers that bring their own data. */
HELIX_API int helix_gemm_timed(const void* A, const void* B, void* C, int M, int N, int K, int lda, int ldb, int ldc,
                     void* workspace, size_t workspace_bytes, void* stream, int warmup, int iters,
                     double* avg_s);

HELIX_API int helix_conv2d_timed(const void* x, const void* w, void* y, int batch, int H, int W, int IC, int OC, int kH,
                       int kW, int stride, int pad, void* workspace, size_t workspace_bytes, void* stream,
                       int warmup, int iters, double* avg_s);

/* Self-contained measurement: allocates and initialises A, B, C (and the workspace), runs `warmup`
 * launches, then `outer` groups of `iters` event-timed launches; reports min / mean / max seconds
 * per launch over the groups.  If `rotate_bytes` > 0 the streamed operand (B) is replicated until the
 * copies total at least that many bytes and launches cycle through them, so a working set that fits
 * the 256 MB last-level cache is still measured against HBM.
 * Replaces: `main` + testF16F16GemmPerformance of every reference template, i.e. the process
 * `gemm_... M N K` whose stdout the profiler parses (src_template/Ampere_FP16/gemm.cu:622-692,
 * gemv.cu:320-435, src_template/Ampere_FP32/sgemm.cu:427-466,568-657;
 * scripts/Ampere_FP16/profile_Ampere_FP16.py:36-38). */
HELIX_API int helix_bench(int M, int N, int K, int warmup, int iters, int outer, size_t rotate_bytes, double* min_s,
                double* avg_s, double* max_s);

/* Same for the convolution entry point.
 * Replaces: `im2col ...` timing main (src_template/Ampere_FP16/im2col.cu:118-196) plus the GEMM run. */
HELIX_API int helix_bench_conv(int batch, int IC, int H, int W, int OC, int kH, int kW, int stride, int pad, int warmup,
                     int iters, int outer, double* min_s, double* avg_s, double* max_s);

#ifdef __cplusplus
}
#endif

#endif /* HELIX_ABI_H */
