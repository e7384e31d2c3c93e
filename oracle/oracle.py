"""ctypes front-end of the CPU oracle (oracle/helix_oracle.c) plus the host logic of the reference's
x86_CPU path restated without TVM.

TEST INFRASTRUCTURE ONLY: tests, the smoke check and the benchmark's cpu_baseline leg import this
module; the HIP product path never does.

Reference files restated here (paths relative to the reference checkout):
  scripts/x86_CPU/profile_x86_CPU.py:62-122          two-phase register-block / cache-block profile
  scripts/x86_CPU/benchmark_x86_CPU_gemm.py:46-68    get_tiling
  scripts/x86_CPU/benchmark_x86_CPU_gemm.py:71-136   sch_gemm (padding) + get_Helix_result (timing)
  scripts/x86_CPU/changed_profile_x86_CPU.py:62-127  the profile whose cache blocks are timed, not extrapolated
  scripts/x86_CPU/benchmark_x86_CPU_conv.py:119-140  convolution = the GEMM of its im2col extents
  scripts/x86_CPU/benchmark_x86_CPU_model_level_LLM.py:119-135, :180-195  per-GEMM seconds summed over a model's list
"""
import ctypes
import math
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_BUILD = os.path.join(_HERE, "_build")
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_u16p = ctypes.POINTER(ctypes.c_uint16)


def build(force=False):
    """Compile the oracle with the Makefile beside this file."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE, "all"], check=True, capture_output=True)


def _cpu_has_avx512():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("flags"):
                    flags = line.split()
                    return "avx512f" in flags and "avx512vl" in flags
    except OSError:
        pass
    return False


def isa():
    return "avx512" if _cpu_has_avx512() else "avx2"


def lib():
    global _lib
    if _lib is not None:
        return _lib
    path = os.path.join(_BUILD, f"libhelix_oracle_{isa()}.so")
    if not os.path.exists(path):
        build()
    L = ctypes.CDLL(path)
    i = ctypes.c_int
    L.oracle_f16_to_f32.argtypes = [_u16p, _f32p, ctypes.c_size_t]
    L.oracle_f32_to_f16.argtypes = [_f32p, _u16p, ctypes.c_size_t]
    L.oracle_sgemm_seqk.argtypes = [_f32p, _f32p, _f32p, i, i, i, i]
    L.oracle_hgemm_f32acc.argtypes = [_u16p, _u16p, _u16p, i, i, i]
    L.oracle_hgemm_f32out.argtypes = [_u16p, _u16p, _f32p, i, i, i]
    L.oracle_conv2d_nhwc_f32.argtypes = [_f32p, _f32p, _f32p] + [i] * 9
    L.oracle_conv2d_nhwc_f16.argtypes = [_u16p, _u16p, _u16p] + [i] * 9
    L.oracle_im2col_nchw.argtypes = [_f32p, _f32p] + [i] * 7
    L.oracle_x86_profile_kernel.argtypes = [_f32p, _f32p, _f32p] + [i] * 8
    L.oracle_x86_profile_kernel.restype = i
    L.oracle_x86_sch_gemm.argtypes = [_f32p, _f32p, _f32p] + [i] * 11
    L.oracle_x86_sch_gemm.restype = i
    L.oracle_x86_time_profile_kernel.argtypes = [_f32p, _f32p, _f32p] + [i] * 9
    L.oracle_x86_time_profile_kernel.restype = ctypes.c_double
    L.oracle_x86_time_sch_gemm.argtypes = [_f32p, _f32p, _f32p] + [i] * 12
    L.oracle_x86_time_sch_gemm.restype = ctypes.c_double
    L.oracle_max_threads.restype = i
    _lib = L
    return L


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(_f32p)


def _f16(a):
    a = np.ascontiguousarray(a, dtype=np.float16)
    return a, a.view(np.uint16).ctypes.data_as(_u16p)


# ---------------------------------------------------------------------------------------------
# value oracles
# ---------------------------------------------------------------------------------------------
def f16_to_f32(h):
    h, hp = _f16(h)
    out = np.empty(h.shape, dtype=np.float32)
    lib().oracle_f16_to_f32(hp, out.ctypes.data_as(_f32p), h.size)
    return out


def f32_to_f16(f):
    f, fp = _f32(f)
    out = np.empty(f.shape, dtype=np.float16)
    lib().oracle_f32_to_f16(fp, out.view(np.uint16).ctypes.data_as(_u16p), f.size)
    return out


def sgemm_seqk(A, B, use_fma=True):
    """C = A @ B, A (M,K), B (K,N), FP32, ascending-k per output (sgemm.cu:12-24)."""
    A, ap = _f32(A)
    B, bp = _f32(B)
    M, K = A.shape
    K2, N = B.shape
    assert K == K2
    C = np.empty((M, N), dtype=np.float32)
    lib().oracle_sgemm_seqk(ap, bp, C.ctypes.data_as(_f32p), M, N, K, 1 if use_fma else 0)
    return C


def hgemm_f32acc(A, B):
    """FP16 in, FP32 accumulate, FP16 out; A (M,K), B (K,N) (gemm.cu:26-37)."""
    A, ap = _f16(A)
    B, bp = _f16(B)
    M, K = A.shape
    K2, N = B.shape
    assert K == K2
    C = np.empty((M, N), dtype=np.float16)
    lib().oracle_hgemm_f32acc(ap, bp, C.view(np.uint16).ctypes.data_as(_u16p), M, N, K)
    return C


def hgemm_f32out(A, B):
    A, ap = _f16(A)
    B, bp = _f16(B)
    M, K = A.shape
    _, N = B.shape
    C = np.empty((M, N), dtype=np.float32)
    lib().oracle_hgemm_f32out(ap, bp, C.ctypes.data_as(_f32p), M, N, K)
    return C


def conv_out_hw(H, W, kH, kW, stride, pad):
    """Ampere_FP16_conv.py:432."""
    return (H + 2 * pad - kH) // stride + 1, (W + 2 * pad - kW) // stride + 1


def conv2d_nhwc(x, w, stride, pad):
    """x (B,H,W,IC), w (OC,kH,kW,IC) -> y (B,OH,OW,OC); dtype of x selects f16/f32."""
    batch, H, W, IC = x.shape
    OC, kH, kW, IC2 = w.shape
    assert IC == IC2
    OH, OW = conv_out_hw(H, W, kH, kW, stride, pad)
    if x.dtype == np.float16:
        x, xp = _f16(x)
        w, wp = _f16(w)
        y = np.empty((batch, OH, OW, OC), dtype=np.float16)
        lib().oracle_conv2d_nhwc_f16(xp, wp, y.view(np.uint16).ctypes.data_as(_u16p), batch, H, W, IC, OC, kH, kW,
                                     stride, pad)
    else:
        x, xp = _f32(x)
        w, wp = _f32(w)
        y = np.empty((batch, OH, OW, OC), dtype=np.float32)
        lib().oracle_conv2d_nhwc_f32(xp, wp, y.ctypes.data_as(_f32p), batch, H, W, IC, OC, kH, kW, stride, pad)
    return y


def im2col_nchw(im, ksize, pad, stride):
    """im (B,C,H,W) float32 -> col (B, C*k*k, OH, OW) (im2col.cu:38-75)."""
    im, ip = _f32(im)
    batch, C, H, W = im.shape
    OH, OW = conv_out_hw(H, W, ksize, ksize, stride, pad)
    col = np.empty((batch, C * ksize * ksize, OH, OW), dtype=np.float32)
    lib().oracle_im2col_nchw(ip, col.ctypes.data_as(_f32p), batch, C, H, W, ksize, pad, stride)
    return col


# ---------------------------------------------------------------------------------------------
# x86_CPU path: schedules
# ---------------------------------------------------------------------------------------------
def x86_profile_kernel(A, B, m1, m2, n1, n2, k1):
    A, ap = _f32(A)
    B, bp = _f32(B)
    M, K = A.shape
    _, N = B.shape
    C = np.empty((M, N), dtype=np.float32)
    rc = lib().oracle_x86_profile_kernel(ap, bp, C.ctypes.data_as(_f32p), M, N, K, m1, m2, n1, n2, k1)
    if rc != 0:
        raise ValueError(f"shape {M}x{N}x{K} is not a multiple of the blocks ({m1},{m2},{n1},{n2},{k1})")
    return C


def ceil_to(x, t):
    return math.ceil(x / t) * t


def x86_sch_gemm(A, B, tiling, nthreads=None):
    """Padded, packed-B, n-parallel schedule (benchmark_x86_CPU_gemm.py:71-117).

    Returns the unpadded (M,N) block of the padded result; zero padding of M, N, K up to tile
    multiples is what the reference's `math.ceil(m / tile) * tile` buffer shapes imply (:78)."""
    m1, m2, m3, n1, n2, n3, k1 = tiling
    M, K = A.shape
    _, N = B.shape
    Mp, Np, Kp = ceil_to(M, m1 * m2 * m3), ceil_to(N, n1 * n2 * n3), ceil_to(K, k1)
    Ap = np.zeros((Mp, Kp), dtype=np.float32)
    Ap[:M, :K] = A
    Bp = np.zeros((Kp, Np), dtype=np.float32)
    Bp[:K, :N] = B
    C = np.empty((Mp, Np), dtype=np.float32)
    if nthreads is None:
        nthreads = os.cpu_count() or 1
    rc = lib().oracle_x86_sch_gemm(Ap.ctypes.data_as(_f32p), Bp.ctypes.data_as(_f32p), C.ctypes.data_as(_f32p),
                                   Mp, Np, Kp, m1, m2, m3, n1, n2, n3, k1, nthreads)
    if rc != 0:
        raise RuntimeError(f"oracle_x86_sch_gemm failed rc={rc}")
    return C[:M, :N]


# the (N1, N2) pairs the reference's profile loop visits; it rewrites N1 in {3,5} to N2=N1, N1=1 and
# the rewrite sticks for the remaining K1 iterations (profile_x86_CPU.py:70-79)
X86_N_PAIRS = [(1, 1), (2, 1), (1, 3), (4, 1), (1, 5)]
X86_PEAK_GFLOPS = 153  # profile_x86_CPU.py:16


def x86_register_blocks():
    """The 270 (M1, M2, N1, N2, K1) points of profile_x86_CPU.py:70-78 in visiting order."""
    out = []
    for M1 in range(1, 10):
        for M2 in range(1, 2):
            for (N1, N2) in X86_N_PAIRS:
                for K1 in range(1, 7):
                    out.append((M1, M2, N1, N2, K1))
    return out


def x86_profile(peak_gflops=X86_PEAK_GFLOPS, number=1000, time_fn=None, keep=0.6, timed_cache_blocks=False):
    """Two-phase profile (profile_x86_CPU.py:62-118): time every register block on a
    (20*M1*M2) x (16*N1*N2) x (16*K1) problem, keep those above `keep`*peak, then extrapolate cache
    blocks up to 256 x 256.  Returns (register_block_dict, cache_block_dict).

    `time_fn(M,N,K,m1,m2,n1,n2,k1) -> seconds` may be injected (tests use a deterministic one).
    `peak_gflops=None` calibrates the peak to the fastest measured register block, for hosts
    whose core is not the Skylake-AVX512 the constant 153 presumes.
    `timed_cache_blocks=True` is changed_profile_x86_CPU.py:62-127: the only difference (its lines 110-119
    against profile_x86_CPU.py:110) is that every cache block is run and timed with the profile-time
    schedule of its register block instead of being priced as a multiple of the register block's time."""
    L = lib()
    rng = np.random.default_rng(0)
    measured = {}
    for (M1, M2, N1, N2, K1) in x86_register_blocks():
        M, N, K = M1 * M2 * 20, N1 * N2 * 16, K1 * 16
        if time_fn is not None:
            cost = time_fn(M, N, K, M1, M2, N1 * 16, N2, K1)
        else:
            A = rng.random((M, K), dtype=np.float32)
            B = rng.random((K, N), dtype=np.float32)
            C = np.zeros((M, N), dtype=np.float32)
            cost = L.oracle_x86_time_profile_kernel(A.ctypes.data_as(_f32p), B.ctypes.data_as(_f32p),
                                                    C.ctypes.data_as(_f32p), M, N, K, M1, M2, N1 * 16, N2, K1, number)
        flops = (2 * M * N * K * 1e-9) / cost
        measured[(M1 * M2, N1 * N2 * 16, K1)] = (cost, flops)
    if peak_gflops is None:
        peak_gflops = max(v[1] for v in measured.values())
    register_block_dict = {k: v for k, v in measured.items() if v[1] > peak_gflops * keep}

    cache_block_dict = {}
    for key, value in register_block_dict.items():
        M1, N1, K1 = key
        M2, N2 = 1, 1
        if N1 == 48 or N1 == 80:
            N2 = N1 // 16
            N1 = 16
        for Mx in range(1, 256 // M1 + 1):
            for Nx in range(1, 256 // (N1 * N2) + 1):
                M = Mx * M1 * M2
                N = Nx * N1 * N2
                K = 16 * K1
                if not timed_cache_blocks:
                    cost = value[0] / (20 * 16) * (Mx * Nx)
                elif time_fn is not None:
                    cost = time_fn(M, N, K, M1, M2, N1, N2, K1)
                else:
                    A = rng.random((M, K), dtype=np.float32)
                    B = rng.random((K, N), dtype=np.float32)
                    C = np.zeros((M, N), dtype=np.float32)
                    cost = L.oracle_x86_time_profile_kernel(A.ctypes.data_as(_f32p), B.ctypes.data_as(_f32p),
                                                            C.ctypes.data_as(_f32p), M, N, K, M1, M2, N1, N2, K1, number)
                flops = (2 * M * N * K * 1e-9) / cost
                if flops > peak_gflops * keep:
                    if (M, N, K) in cache_block_dict:
                        if cache_block_dict[(M, N, K)][1] > cost:
                            cache_block_dict[(M, N, K)] = (key, cost, flops)
                    else:
                        cache_block_dict[(M, N, K)] = (key, cost, flops)
    return register_block_dict, cache_block_dict


def x86_get_tiling(prof_dict, M, N, K, num_thread=48):
    """benchmark_x86_CPU_gemm.py:46-68 (num_thread is hard-coded to 48 there, :22)."""
    min_cost = float("inf")
    min_cache = (1, 1, 1)
    min_reg = (1, 1, 1)
    for k, v in prof_dict.items():
        thread = math.ceil(N / k[1])
        cost = v[1] * math.ceil(M / k[0]) * math.ceil(thread / num_thread)
        if min_cost > cost:
            min_cost = cost
            min_cache = k
            min_reg = v[0]
    M1, M2, M3 = min_reg[0], 1, min_cache[0] // min_reg[0]
    N1, N2, N3 = min_reg[1], 1, min_cache[1] // min_reg[1]
    if N1 == 48 or N1 == 80:
        N2 = N1 // 16
        N1 = 16
    K1 = min_reg[2]
    return M1, M2, M3, N1, N2, N3, K1


def x86_time_gemm(prof_dict, M, N, K, num_thread=None, number=100, A=None, B=None):
    """get_Helix_result (benchmark_x86_CPU_gemm.py:119-136): pick the tiling, pad, run `number`
    times, return (mean seconds, GFLOP/s on the PADDED shape as the reference does, padded shape,
    tiling)."""
    if num_thread is None:
        num_thread = os.cpu_count() or 1
    tiling = x86_get_tiling(prof_dict, M, N, K, num_thread)
    m1, m2, m3, n1, n2, n3, k1 = tiling
    Mp, Np, Kp = ceil_to(M, m1 * m2 * m3), ceil_to(N, n1 * n2 * n3), ceil_to(K, k1)
    rng = np.random.default_rng(0)
    Ap = np.zeros((Mp, Kp), dtype=np.float32)
    Bp = np.zeros((Kp, Np), dtype=np.float32)
    Ap[:M, :K] = rng.random((M, K), dtype=np.float32) if A is None else A
    Bp[:K, :N] = rng.random((K, N), dtype=np.float32) if B is None else B
    C = np.zeros((Mp, Np), dtype=np.float32)
    cost = lib().oracle_x86_time_sch_gemm(Ap.ctypes.data_as(_f32p), Bp.ctypes.data_as(_f32p), C.ctypes.data_as(_f32p),
                                          Mp, Np, Kp, m1, m2, m3, n1, n2, n3, k1, num_thread, number)
    if cost < 0:
        raise RuntimeError("oracle_x86_time_sch_gemm failed")
    gflops = 2 * Mp * Np * Kp / 1e9 / cost
    return cost, gflops, (Mp, Np, Kp), tiling, C[:M, :N]


def x86_changed_profile(peak_gflops=X86_PEAK_GFLOPS, number=1000, time_fn=None, keep=0.6):
    """changed_profile_x86_CPU.py:62-127 (profile_Helix_x86_CPU_gemm_kernel of that file)."""
    return x86_profile(peak_gflops=peak_gflops, number=number, time_fn=time_fn, keep=keep, timed_cache_blocks=True)


def x86_conv_gemm_extents(batch, input_channel, H, W, output_channel, kH, kW, stride, pad):
    """The GEMM a convolution is timed as (benchmark_x86_CPU_conv.py:123-125)."""
    M = batch * ((H + 2 * pad - kH) // stride + 1) * ((W + 2 * pad - kW) // stride + 1)
    return M, output_channel, input_channel * kH * kW


def x86_time_conv(prof_dict, batch, input_channel, H, W, output_channel, kH, kW, stride, pad, num_thread=None,
                  number=100):
    """get_Helix_result of benchmark_x86_CPU_conv.py:119-140: the convolution is timed as the GEMM of its
    im2col extents on random matrices (no gather is run); returns what x86_time_gemm returns, GFLOP/s on the
    padded extents as there (:138)."""
    M, N, K = x86_conv_gemm_extents(batch, input_channel, H, W, output_channel, kH, kW, stride, pad)
    return x86_time_gemm(prof_dict, M, N, K, num_thread=num_thread, number=number)


def x86_time_model(prof_dict, mnk_list, num_thread=None, number=100):
    """Model-level cost (benchmark_x86_CPU_model_level_LLM.py:180-195): get_Helix_result (:119-135) returns the
    mean seconds of one GEMM and the benchmark adds them over the model's (M, N, K) list, repeats included (the
    reference prints that sum of seconds with an "ms" label; the value is restated, not the label).  Each
    distinct shape is timed once here and weighted by its multiplicity.  Returns total seconds."""
    counts = {}
    for mnk in mnk_list:
        counts[tuple(mnk)] = counts.get(tuple(mnk), 0) + 1
    total = 0.0
    for (M, N, K), count in counts.items():
        total += x86_time_gemm(prof_dict, M, N, K, num_thread=num_thread, number=number)[0] * count
    return total
