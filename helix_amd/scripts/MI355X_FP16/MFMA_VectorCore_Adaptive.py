"""Where the dispatch between the weight-streaming kernel (vector dot products) and the MFMA tile kernels
crosses over as the skinny extent M grows: for every shape, the cost model's pick over all libraries, the
GEMV library alone, and the best-predicted MFMA tile configuration alone.

Mirrors scripts/Ampere_FP16/TensorCore_CUDACore_Adaptive.py:8-75 (same shape sweep: M in 1..16,
N in {1024, 2048, 4096}, K = 1024; the reference computes the three numbers and prints nothing, :70-75 --
here they are printed).  As there, split-K rows are left out of the two cost models (:12-13, :26-27).
"""
import os

from utils.helix_runtime import read_prof_dict
from MI355X_FP16.MI355X_FP16_gemm import short_value, config_cost, run_config

root_path = os.getcwd()

ADAPTIVE_SHAPES = [(m, n, 1024) for n in [1024, 2048, 4096] for m in [1, 2, 4, 6, 8, 10, 12, 14, 16]]


def cost_model(prof_dict, M, N, K, with_gemv=True):
    min_cost, best_config = float("inf"), None
    for k, v in prof_dict.items():
        if k[5] == 1 or (k[0] == 0 and not with_gemv):
            continue
        cost = config_cost(k, v, M, N, K, short_value(prof_dict, k))
        if min_cost > cost:
            min_cost, best_config = cost, k
    return best_config


def cost_model_without_gemv(prof_dict, M, N, K):
    return cost_model(prof_dict, M, N, K, with_gemv=False)


def _tflops(k, M, N, K):
    return 2 * M * N * K / 1e12 / run_config(k, M, N, K)


def get_Helix_result(prof_dict, M, N, K):
    return _tflops(cost_model(prof_dict, M, N, K), M, N, K)


def get_gemv_result(prof_dict, M, N, K):
    gemv_keys = [k for k in prof_dict if k[0] == 0 and k[5] == 0]
    k = min(gemv_keys, key=lambda k: config_cost(k, prof_dict[k], M, N, K, short_value(prof_dict, k)))
    return _tflops(k, M, N, K)


def get_gemm_result(prof_dict, M, N, K):
    return _tflops(cost_model_without_gemv(prof_dict, M, N, K), M, N, K)


if __name__ == "__main__":

    prof_dict = read_prof_dict("MI355X_FP16")
    for M, N, K in ADAPTIVE_SHAPES:
        helix_tflops = get_Helix_result(prof_dict, M, N, K)
        gemv_tflops = get_gemv_result(prof_dict, M, N, K)
        gemm_tflops = get_gemm_result(prof_dict, M, N, K)
        print(f'{M}x{N}x{K}: Helix: {helix_tflops:.2f} TFLOPS, GEMV: {gemv_tflops:.2f} TFLOPS, '
              f'MFMA GEMM: {gemm_tflops:.2f} TFLOPS')
