"""Cost model and single-GEMM runner of the MI355X_FP32 backend.
Mirrors scripts/Ampere_FP32/Ampere_FP32_gemm.py:89-107 (`cost_model`, `get_Ampere_FP32_gemm_Helix_result`);
the TVM alternative backend (:16-86, :108-136) has no counterpart."""
import math
import os

from utils.helix_runtime import load
from utils.roofline import NUM_CU, HBM_BYTES_PER_S, gemm_bytes
from MI355X_FP32.build_MI355X_FP32 import library_for_key, kernel_library
from MI355X_FP32.profile_MI355X_FP32 import PROFILE_K, GEMV_PROFILE_K

root_path = os.getcwd()

HBM_SUSTAINED_FRACTION = 0.6
GEMV_LAUNCH_FLOOR_S = 3e-6


def config_cost(k, v, M, N, K):
    """rounds * time-per-round as in Ampere_FP32_gemm.py:93-95, with 256 compute units for 108 SMs and
    the round time scaled by K / K_profile (the reference ignores K)."""
    if k[2] == 0:
        small, big = (M, N) if M <= N else (N, M)
        num_block = math.ceil(small / k[0]) * math.ceil(big / k[1])
        return max(num_block / NUM_CU * v * max(K, 256) / GEMV_PROFILE_K, GEMV_LAUNCH_FLOOR_S)
    num_block = math.ceil(M / k[0]) * math.ceil(N / k[1])
    w = math.ceil(num_block / NUM_CU)
    return max(w * v * max(K, 32) / PROFILE_K, gemm_bytes(M, N, K, 4) / (HBM_SUSTAINED_FRACTION * HBM_BYTES_PER_S))


def cost_model(prof_dict, M, N, K):
    min_cost = float("inf")
    best_config = (1, 1, 1, 1, 1, 1, 1, 1)
    for k, v in prof_dict.items():
        cost = config_cost(k, v, M, N, K)
        if min_cost > cost:
            min_cost = cost
            best_config = k
    return best_config


def run_config(k, M, N, K, warmup=10, iters=10, outer=1):
    """Seconds per launch (mean) on the real M, N, K (edges are predicated in the kernel; the reference
    pads M and N up to the tile instead, Ampere_FP32_gemm.py:103)."""
    lib = load(library_for_key(k))
    if k[2] == 0:
        if M > N:
            M, N = N, M
        K = math.ceil(K / 4) * 4
    _, avg, _ = lib.bench(M, N, K, warmup=warmup, iters=iters, outer=outer, rotate_bytes=0)
    return avg


def get_MI355X_FP32_gemm_Helix_result(prof_dict, M, N, K, backend="hip"):
    if backend != "hip":
        raise ValueError(f"backend {backend!r} is not available for MI355X_FP32 (only 'hip')")
    best_config = cost_model(prof_dict, M, N, K)
    cost = run_config(best_config, M, N, K) * 1e3
    tflops = 2 * M * N * K / 1e9 / cost

    return cost, tflops


def get_MI355X_FP32_gemm_rocblas_result(M, N, K):
    """The vendor library (rocblas_sgemm) on the same problem and operand layouts, timed the same way.
    Mirrors get_Ampere_FP32_gemm_cublas_result (Ampere_FP32_gemm.py)."""
    lib = load(kernel_library("rocblas_f32"))
    _, avg, _ = lib.bench(M, N, K, warmup=10, iters=10, outer=1, rotate_bytes=0)
    cost = avg * 1e3
    return cost, 2 * M * N * K / 1e9 / cost


def get_MI355X_FP32_gemm_Oracle_result(prof_dict, M, N, K):
    """Exhaustive per-shape search.  Returns (cost_ms, tflops, key)."""
    min_cost, best = float("inf"), None
    for k in prof_dict.keys():
        if k[2] == 0 and min(M, N) > 16:
            continue
        try:
            cost = run_config(k, M, N, K, warmup=2, iters=5)
        except Exception:
            continue
        if min_cost > cost:
            min_cost, best = cost, k
    return min_cost * 1e3, 2 * M * N * K / 1e12 / min_cost, best
