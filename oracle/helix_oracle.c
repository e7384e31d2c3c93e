/*
 * helix_oracle.c -- CPU restatement of the reference's x86_CPU template path and of the
 * host-side checker loops in its CUDA templates.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the smoke check and the
 * cpu_baseline leg of the benchmark may load this library; the HIP product path never does.
 *
 * Every function cites the reference file:line whose arithmetic it restates (paths relative to
 * the reference checkout).  The reference x86 path is Python driving Apache TVM v0.12.0 (LLVM
 * 15.0.7 codegen); TVM is a third-party dependency that is absent here, so the loop nests its
 * schedule primitives describe are restated by hand below.
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   - oracle_f16_to_f32 / oracle_f32_to_f16 : exhaustive (65536 halves) and random floats vs numpy
 *   - oracle_sgemm_seqk        : float64 matmul with a normwise bound, identity / ones / unit-vector
 *                                closed forms, integer-valued inputs (exact), pure-Python brute force
 *   - oracle_hgemm_f32acc      : same set, plus numpy (A16->f32 @ B16->f32)->f16
 *   - oracle_x86_profile_kernel, oracle_x86_sch_gemm : bit-identical to oracle_sgemm_seqk (same
 *                                ascending-k order per output element) for every tiling tested
 *   - oracle_conv2d_nhwc_*     : 7-loop Python brute force on tiny tensors, torch.nn.functional.conv2d
 *                                on CPU, and the 1x1/stride-1 special case == GEMM
 *   - oracle_im2col_nchw       : brute-force index map; im2col followed by GEMM == direct conv
 */
#define _GNU_SOURCE
#include <stdint.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#include <time.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------------------------ */
/* IEEE binary16 <-> binary32, bit exact, round-to-nearest-even (what `(half)psum` and          */
/* `(float)a[...]` do in src_template/Ampere_FP16/gemm.cu:31-33).                               */
/* ------------------------------------------------------------------------------------------ */
static inline float f16_bits_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t out;
    if (exp == 0) {
        if (man == 0) {
            out = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3ffu;
            out = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        out = sign | 0x7f800000u | (man << 13);
    } else {
        out = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &out, 4);
    return f;
}

static inline uint16_t f32_to_f16_bits(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u) { /* inf / nan */
        if (absx > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((absx >> 13) & 0x3ffu));
        return (uint16_t)(sign | 0x7c00u);
    }
    if (absx >= 0x477ff000u) { /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (absx < 0x33000001u) { /* <= 2^-25 rounds to zero (tie at 2^-25 -> even = 0) */
        return (uint16_t)sign;
    }
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t m = (absx & 0x7fffffu) | 0x800000u; /* 24-bit significand */
    uint32_t shift;
    uint32_t hexp;
    if (e < -14) { /* subnormal half */
        shift = (uint32_t)(13 + (-14 - e));
        hexp = 0;
    } else {
        shift = 13;
        hexp = (uint32_t)(e + 15);
    }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    uint32_t out;
    if (hexp == 0) {
        out = q; /* q may carry into the exponent field: that is the correct encoding */
    } else {
        out = ((hexp - 1) << 10) + q; /* q includes the implicit bit (0x400) */
    }
    return (uint16_t)(sign | out);
}

void oracle_f16_to_f32(const uint16_t* src, float* dst, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] = f16_bits_to_f32(src[i]);
}

void oracle_f32_to_f16(const float* src, uint16_t* dst, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] = f32_to_f16_bits(src[i]);
}

/* ------------------------------------------------------------------------------------------ */
/* FP32 GEMM, sequential-k.  Restates cpuSgemm (src_template/Ampere_FP32/sgemm.cu:12-24) and is  */
/* the value semantics of the TIR definition C[m,n] = sum_k A[m,k]*B[k,n] with init 0           */
/* (scripts/x86_CPU/profile_x86_CPU.py:31-38): A is M x K, B is K x N, C is M x N, row-major.    */
/* use_fma != 0 contracts multiply+add into one rounding, as LLVM does for the TVM build.        */
/* ------------------------------------------------------------------------------------------ */
void oracle_sgemm_seqk(const float* A, const float* B, float* C, int M, int N, int K, int use_fma) {
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; m++) {
        for (int n = 0; n < N; n++) {
            float psum = 0.0f;
            if (use_fma) {
                for (int k = 0; k < K; k++) psum = fmaf(A[(size_t)m * K + k], B[(size_t)k * N + n], psum);
            } else {
                for (int k = 0; k < K; k++) {
                    volatile float prod = A[(size_t)m * K + k] * B[(size_t)k * N + n];
                    psum = psum + prod;
                }
            }
            C[(size_t)m * N + n] = psum;
        }
    }
}

/* ------------------------------------------------------------------------------------------ */
/* FP16 in, FP32 accumulate, FP16 out.  Restates cpuF16F16Gemm                                  */
/* (src_template/Ampere_FP16/gemm.cu:26-37): psum is float, each product is formed from the two */
/* operands widened to float (exact: 11-bit x 11-bit significands), summed in ascending k, and   */
/* the result is rounded once to half.  A is M x K, B is K x N (the checker's layout, before the */
/* host transposes B for the device, gemm.cu:597-601).                                           */
/* ------------------------------------------------------------------------------------------ */
void oracle_hgemm_f32acc(const uint16_t* A, const uint16_t* B, uint16_t* C, int M, int N, int K) {
    float* Bf = (float*)malloc((size_t)K * N * sizeof(float));
    oracle_f16_to_f32(B, Bf, (size_t)K * N);
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; m++) {
        float* acc = (float*)malloc((size_t)N * sizeof(float));
        for (int n = 0; n < N; n++) acc[n] = 0.0f;
        for (int k = 0; k < K; k++) {
            float a = f16_bits_to_f32(A[(size_t)m * K + k]);
            const float* brow = Bf + (size_t)k * N;
            /* product is exact in float, so mul+add and fma give the same bits */
            for (int n = 0; n < N; n++) acc[n] += a * brow[n];
        }
        for (int n = 0; n < N; n++) C[(size_t)m * N + n] = f32_to_f16_bits(acc[n]);
        free(acc);
    }
    free(Bf);
}

/* Same contraction, FP32 result kept (used to attribute rounding error in tests). */
void oracle_hgemm_f32out(const uint16_t* A, const uint16_t* B, float* C, int M, int N, int K) {
    float* Bf = (float*)malloc((size_t)K * N * sizeof(float));
    oracle_f16_to_f32(B, Bf, (size_t)K * N);
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; m++) {
        float* acc = C + (size_t)m * N;
        for (int n = 0; n < N; n++) acc[n] = 0.0f;
        for (int k = 0; k < K; k++) {
            float a = f16_bits_to_f32(A[(size_t)m * K + k]);
            const float* brow = Bf + (size_t)k * N;
            for (int n = 0; n < N; n++) acc[n] += a * brow[n];
        }
    }
    free(Bf);
}

/* ------------------------------------------------------------------------------------------ */
/* Convolution.  Shape algebra from scripts/Ampere_FP16/Ampere_FP16_conv.py:432-434:            */
/*   OH = (H + 2*pad - kH) / stride + 1,  M = batch*OH*OW,  N = OC,  K = IC*kH*kW.              */
/* Direct 7-loop convolution on NHWC activations and [OC][kH][kW][IC] weights, FP32 accumulate   */
/* in (kh, kw, c) order, zero padding.                                                           */
/* ------------------------------------------------------------------------------------------ */
void oracle_conv2d_nhwc_f32(const float* x, const float* w, float* y, int batch, int H, int W, int IC,
                            int OC, int kH, int kW, int stride, int pad) {
    int OH = (H + 2 * pad - kH) / stride + 1;
    int OW = (W + 2 * pad - kW) / stride + 1;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < batch; b++) {
        for (int oh = 0; oh < OH; oh++) {
            for (int ow = 0; ow < OW; ow++) {
                float* yo = y + (((size_t)b * OH + oh) * OW + ow) * OC;
                for (int oc = 0; oc < OC; oc++) {
                    float psum = 0.0f;
                    for (int kh = 0; kh < kH; kh++) {
                        int ih = oh * stride - pad + kh;
                        if (ih < 0 || ih >= H) continue;
                        for (int kw = 0; kw < kW; kw++) {
                            int iw = ow * stride - pad + kw;
                            if (iw < 0 || iw >= W) continue;
                            const float* xi = x + (((size_t)b * H + ih) * W + iw) * IC;
                            const float* wi = w + (((size_t)oc * kH + kh) * kW + kw) * IC;
                            for (int c = 0; c < IC; c++) psum = fmaf(xi[c], wi[c], psum);
                        }
                    }
                    yo[oc] = psum;
                }
            }
        }
    }
}

void oracle_conv2d_nhwc_f16(const uint16_t* x, const uint16_t* w, uint16_t* y, int batch, int H, int W,
                            int IC, int OC, int kH, int kW, int stride, int pad) {
    int OH = (H + 2 * pad - kH) / stride + 1;
    int OW = (W + 2 * pad - kW) / stride + 1;
    size_t nx = (size_t)batch * H * W * IC, nw = (size_t)OC * kH * kW * IC, ny = (size_t)batch * OH * OW * OC;
    float* xf = (float*)malloc(nx * sizeof(float));
    float* wf = (float*)malloc(nw * sizeof(float));
    float* yf = (float*)malloc(ny * sizeof(float));
    oracle_f16_to_f32(x, xf, nx);
    oracle_f16_to_f32(w, wf, nw);
    oracle_conv2d_nhwc_f32(xf, wf, yf, batch, H, W, IC, OC, kH, kW, stride, pad);
    oracle_f32_to_f16(yf, y, ny);
    free(xf); free(wf); free(yf);
}

/* ------------------------------------------------------------------------------------------ */
/* im2col index map of im2col_gpu_kernel (src_template/Ampere_FP16/im2col.cu:38-75): NCHW image, */
/* square kernel `ksize`, one stride/pad; per image the column buffer is                         */
/* col[(c*ksize*ksize + i*ksize + j)][oh][ow], zero where the tap falls in the padding.          */
/* ------------------------------------------------------------------------------------------ */
void oracle_im2col_nchw(const float* im, float* col, int batch, int channels, int height, int width,
                        int ksize, int pad, int stride) {
    int height_col = (height + 2 * pad - ksize) / stride + 1;
    int width_col = (width + 2 * pad - ksize) / stride + 1;
    int n = channels * height_col * width_col;
    size_t im_size = (size_t)height * width * channels;
    size_t col_size = (size_t)n * ksize * ksize;
    for (int b = 0; b < batch; b++) {
        for (int index = 0; index < n; index++) {
            int w_out = index % width_col;
            int h_index = index / width_col;
            int h_out = h_index % height_col;
            int channel_in = h_index / height_col;
            int channel_out = channel_in * ksize * ksize;
            int h_in = h_out * stride - pad;
            int w_in = w_out * stride - pad;
            float* cp = col + b * col_size + ((size_t)channel_out * height_col + h_out) * width_col + w_out;
            const float* ip = im + b * im_size + (size_t)channel_in * height * width;
            for (int i = 0; i < ksize; i++) {
                for (int j = 0; j < ksize; j++) {
                    int h = h_in + i, w = w_in + j;
                    *cp = (h >= 0 && w >= 0 && h < height && w < width) ? ip[(size_t)h * width + w] : 0.0f;
                    cp += (size_t)height_col * width_col;
                }
            }
        }
    }
}

/* ------------------------------------------------------------------------------------------ */
/* x86_CPU micro-kernels.  One call = the (vk1, vm1, vn1) innermost loops of the schedules:      */
/*   for k in k1 (unrolled): for i1 in m1 (unrolled): C[i1, 0:n1] += A[i1, k] * Bp[k, 0:n1]      */
/* with vn1 vectorised (scripts/x86_CPU/profile_x86_CPU.py:54-56,                                */
/* scripts/x86_CPU/benchmark_x86_CPU_gemm.py:88-91).  n1 is 16, 32 or 64 floats.  TVM JIT-builds  */
/* one specialised body per (m1, n1, k1); here the (m1, n1/16) pairs are instantiated by macro    */
/* and k1 stays a run-time trip count.                                                           */
/* ------------------------------------------------------------------------------------------ */
typedef float v16f __attribute__((vector_size(64), aligned(4)));

#define DEF_MK(M1, NV)                                                                              \
    static void mk_##M1##_##NV(float* restrict Cl, int ldc, const float* restrict A, int lda,        \
                               const float* restrict Bp, int ldb, int k1) {                          \
        v16f acc[M1][NV];                                                                            \
        for (int i = 0; i < M1; i++)                                                                 \
            for (int v = 0; v < NV; v++) acc[i][v] = *(const v16f*)(Cl + (size_t)i * ldc + v * 16);  \
        for (int k = 0; k < k1; k++) {                                                               \
            v16f bv[NV];                                                                             \
            for (int v = 0; v < NV; v++) bv[v] = *(const v16f*)(Bp + (size_t)k * ldb + v * 16);      \
            for (int i = 0; i < M1; i++) {                                                           \
                float a = A[(size_t)i * lda + k];                                                    \
                v16f av = {a, a, a, a, a, a, a, a, a, a, a, a, a, a, a, a};                          \
                for (int v = 0; v < NV; v++) acc[i][v] = acc[i][v] + av * bv[v];                     \
            }                                                                                        \
        }                                                                                            \
        for (int i = 0; i < M1; i++)                                                                 \
            for (int v = 0; v < NV; v++) *(v16f*)(Cl + (size_t)i * ldc + v * 16) = acc[i][v];        \
    }

#define DEF_MK_ROW(M1) DEF_MK(M1, 1) DEF_MK(M1, 2) DEF_MK(M1, 4)
DEF_MK_ROW(1) DEF_MK_ROW(2) DEF_MK_ROW(3) DEF_MK_ROW(4) DEF_MK_ROW(5)
DEF_MK_ROW(6) DEF_MK_ROW(7) DEF_MK_ROW(8) DEF_MK_ROW(9)

typedef void (*mk_fn)(float*, int, const float*, int, const float*, int, int);
#define MK_ROW(M1) { mk_##M1##_1, mk_##M1##_2, NULL, mk_##M1##_4 }
static const mk_fn mk_table[9][4] = { MK_ROW(1), MK_ROW(2), MK_ROW(3), MK_ROW(4), MK_ROW(5),
                                      MK_ROW(6), MK_ROW(7), MK_ROW(8), MK_ROW(9) };

/* generic fallback (any m1, any n1) with the same per-element operation order */
static void mk_generic(float* restrict Cl, int ldc, const float* restrict A, int lda,
                       const float* restrict Bp, int ldb, int k1, int m1, int n1) {
    for (int k = 0; k < k1; k++)
        for (int i = 0; i < m1; i++) {
            float a = A[(size_t)i * lda + k];
            for (int j = 0; j < n1; j++) Cl[(size_t)i * ldc + j] += a * Bp[(size_t)k * ldb + j];
        }
}

static inline void micro_kernel(float* Cl, int ldc, const float* A, int lda, const float* Bp, int ldb,
                                int k1, int m1, int n1) {
    if (m1 >= 1 && m1 <= 9 && (n1 == 16 || n1 == 32 || n1 == 64)) {
        mk_table[m1 - 1][n1 / 16 - 1](Cl, ldc, A, lda, Bp, ldb, k1);
    } else {
        mk_generic(Cl, ldc, A, lda, Bp, ldb, k1, m1, n1);
    }
}

/* ------------------------------------------------------------------------------------------ */
/* Profile-time schedule, single thread (scripts/x86_CPU/profile_x86_CPU.py:40-60):             */
/*   split m -> [m3, m2, m1], n -> [n3, n2, n1], k -> [k2, k1];                                 */
/*   reorder m3, n3, k2, m2, n2, k1, m1, n1; vectorize n1; unroll m1;                            */
/*   decompose_reduction at k2 => the (m2*m1) x (n2*n1) block of C is zeroed before the k2 loop. */
/* M, N, K must be multiples of m2*m1, n2*n1, k1.  Returns 0, or -1 on a shape that is not.      */
/* ------------------------------------------------------------------------------------------ */
int oracle_x86_profile_kernel(const float* A, const float* B, float* C, int M, int N, int K, int m1, int m2,
                              int n1, int n2, int k1) {
    int mb = m2 * m1, nb = n2 * n1;
    if (m1 <= 0 || m2 <= 0 || n1 <= 0 || n2 <= 0 || k1 <= 0) return -1;
    if (M % mb || N % nb || K % k1) return -1;
    for (int i3 = 0; i3 < M / mb; i3++) {
        for (int j3 = 0; j3 < N / nb; j3++) {
            for (int i = 0; i < mb; i++)
                for (int j = 0; j < nb; j++) C[(size_t)(i3 * mb + i) * N + j3 * nb + j] = 0.0f;
            for (int kk = 0; kk < K / k1; kk++) {
                for (int i2 = 0; i2 < m2; i2++) {
                    for (int j2 = 0; j2 < n2; j2++) {
                        int row = i3 * mb + i2 * m1;
                        int col = j3 * nb + j2 * n1;
                        micro_kernel(C + (size_t)row * N + col, N, A + (size_t)row * K + kk * k1, K,
                                     B + (size_t)(kk * k1) * N + col, N, k1, m1, n1);
                    }
                }
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* Run-time schedule (scripts/x86_CPU/benchmark_x86_CPU_gemm.py:71-117), Mc=m1*m2*m3,            */
/* Nc=n1*n2*n3:                                                                                  */
/*   parallel for nb in N/Nc                                  (sch.parallel(vn4), :92)           */
/*     Bp[n3][K/k1][n2][k1][n1] = pack(B[:, nb*Nc : +Nc])     (reindex_cache_read, :94-102)      */
/*     for mb in M/Mc                                         (vm4)                              */
/*       Cl[Mc][Nc] = 0                                       (decompose_reduction at vm3, :115) */
/*       for i3 in m3, j3 in n3, kk in K/k1, i2 in m2, j2 in n2: micro-kernel(k1, m1, n1)        */
/*     C[:, nb*Nc : +Nc] = Cl                                 (cache_write + reverse_compute_at, */
/*                                                             :104-113; here per mb block)      */
/* The reference pads M, N, K up to tile multiples before building (:78); this routine requires  */
/* already padded shapes (the Python wrapper pads with zeros) and returns -1 otherwise.          */
/* ------------------------------------------------------------------------------------------ */
int oracle_x86_sch_gemm(const float* A, const float* B, float* C, int M, int N, int K, int m1, int m2, int m3,
                        int n1, int n2, int n3, int k1, int nthreads) {
    if (m1 <= 0 || m2 <= 0 || m3 <= 0 || n1 <= 0 || n2 <= 0 || n3 <= 0 || k1 <= 0) return -1;
    int Mc = m1 * m2 * m3, Nc = n1 * n2 * n3;
    if (M % Mc || N % Nc || K % k1) return -1;
    int nblocks = N / Nc, K2 = K / k1;
    int fail = 0;
    if (nthreads <= 0) nthreads = 1;
#pragma omp parallel for schedule(static) num_threads(nthreads)
    for (int nb = 0; nb < nblocks; nb++) {
        float* Bp = (float*)aligned_alloc(64, (size_t)Nc * K * sizeof(float));
        float* Cl = (float*)aligned_alloc(64, (((size_t)Mc * Nc * sizeof(float)) + 63) / 64 * 64);
        if (!Bp || !Cl) {
            fail = 1;
            free(Bp); free(Cl);
            continue;
        }
        /* pack: Bp[j3][kk][j2][k][j1] = B[kk*k1 + k][nb*Nc + (j3*n2 + j2)*n1 + j1] */
        for (int j3 = 0; j3 < n3; j3++)
            for (int kk = 0; kk < K2; kk++)
                for (int j2 = 0; j2 < n2; j2++)
                    for (int k = 0; k < k1; k++) {
                        const float* src = B + (size_t)(kk * k1 + k) * N + (size_t)nb * Nc + (j3 * n2 + j2) * n1;
                        float* dst = Bp + ((((size_t)j3 * K2 + kk) * n2 + j2) * k1 + k) * n1;
                        memcpy(dst, src, (size_t)n1 * sizeof(float));
                    }
        for (int mb = 0; mb < M / Mc; mb++) {
            memset(Cl, 0, (size_t)Mc * Nc * sizeof(float));
            for (int i3 = 0; i3 < m3; i3++)
                for (int j3 = 0; j3 < n3; j3++)
                    for (int kk = 0; kk < K2; kk++)
                        for (int i2 = 0; i2 < m2; i2++)
                            for (int j2 = 0; j2 < n2; j2++) {
                                int lrow = (i3 * m2 + i2) * m1;
                                int lcol = (j3 * n2 + j2) * n1;
                                const float* a = A + (size_t)(mb * Mc + lrow) * K + kk * k1;
                                const float* bp = Bp + (((size_t)j3 * K2 + kk) * n2 + j2) * (size_t)k1 * n1;
                                micro_kernel(Cl + (size_t)lrow * Nc + lcol, Nc, a, K, bp, n1, k1, m1, n1);
                            }
            for (int i = 0; i < Mc; i++)
                memcpy(C + (size_t)(mb * Mc + i) * N + (size_t)nb * Nc, Cl + (size_t)i * Nc, (size_t)Nc * sizeof(float));
        }
        free(Bp); free(Cl);
    }
    return fail ? -2 : 0;
}

/* ------------------------------------------------------------------------------------------ */
/* Timing in the manner of tvm's time_evaluator(number=n).mean: one untimed call, then `number`   */
/* back-to-back calls, mean seconds (profile_x86_CPU.py:82-88, benchmark_x86_CPU_gemm.py:126-133).*/
/* ------------------------------------------------------------------------------------------ */
static double now_s(void) {
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

double oracle_x86_time_profile_kernel(const float* A, const float* B, float* C, int M, int N, int K, int m1,
                                      int m2, int n1, int n2, int k1, int number) {
    if (oracle_x86_profile_kernel(A, B, C, M, N, K, m1, m2, n1, n2, k1) != 0) return -1.0;
    double t0 = now_s();
    for (int r = 0; r < number; r++) oracle_x86_profile_kernel(A, B, C, M, N, K, m1, m2, n1, n2, k1);
    return (now_s() - t0) / (double)number;
}

double oracle_x86_time_sch_gemm(const float* A, const float* B, float* C, int M, int N, int K, int m1, int m2,
                                int m3, int n1, int n2, int n3, int k1, int nthreads, int number) {
    if (oracle_x86_sch_gemm(A, B, C, M, N, K, m1, m2, m3, n1, n2, n3, k1, nthreads) != 0) return -1.0;
    double t0 = now_s();
    for (int r = 0; r < number; r++) oracle_x86_sch_gemm(A, B, C, M, N, K, m1, m2, m3, n1, n2, n3, k1, nthreads);
    return (now_s() - t0) / (double)number;
}

int oracle_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
