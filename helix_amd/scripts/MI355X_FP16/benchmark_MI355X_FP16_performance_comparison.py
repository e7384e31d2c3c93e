"""Search-quality ablation of the MI355X_FP16 backend: exhaustive search (Oracle), the cost model
(Default), the fastest of the cost model's first few candidates (Verified), block tile == wave tile only (Static1) and the globally fastest tile (Static2).
Mirrors scripts/Ampere_FP16/benchmark_Ampere_FP16_performance_comparison.py:8-106."""
import math
import os

from utils.get_benchmark_shape_list import get_gemm_op_MNKList
from utils.helix_runtime import read_prof_dict
from MI355X_FP16.MI355X_FP16_gemm import short_value, config_cost, cost_model, run_config, get_MI355X_FP16_gemm_Oracle_result, get_MI355X_FP16_gemm_Verified_result

root_path = os.getcwd()


def cost_model_static1(prof_dict, M, N, K):
    min_cost = float("inf")
    best_config = (1, 1, 1, 1, 1, 0, 32)
    for k, v in prof_dict.items():
        if k[1] != k[3] or k[2] != k[4]:
            continue
        cost = config_cost(k, v, M, N, K, short_value(prof_dict, k))
        if min_cost > cost:
            min_cost = cost
            best_config = k
    return best_config


def cost_model_static2(prof_dict, M, N, K):
    min_cost = float("inf")
    best_config = (1, 1, 1, 1, 1, 0, 32)
    for k, v in prof_dict.items():
        if k[0] == 0:
            continue
        # profiled time per unit of tile area: the tile that is fastest regardless of shape
        cost = v / (k[1] * k[2])
        if min_cost > cost:
            min_cost = cost
            best_config = k
    return best_config


def _tflops(k, M, N, K):
    return 2 * M * N * K / 1e12 / run_config(k, M, N, K)


def get_Helix_Default_result(prof_dict, M, N, K):
    return _tflops(cost_model(prof_dict, M, N, K), M, N, K)


def get_Helix_Oracle_result(prof_dict, M, N, K):
    return get_MI355X_FP16_gemm_Oracle_result(prof_dict, M, N, K)[1]


def get_Helix_Verified_result(prof_dict, M, N, K):
    return get_MI355X_FP16_gemm_Verified_result(prof_dict, M, N, K)[1]


def get_Helix_Static1_result(prof_dict, M, N, K):
    return _tflops(cost_model_static1(prof_dict, M, N, K), M, N, K)


def get_Helix_Static2_result(prof_dict, M, N, K):
    return _tflops(cost_model_static2(prof_dict, M, N, K), M, N, K)


if __name__ == "__main__":

    prof_dict = read_prof_dict("MI355X_FP16")

    MNKList = get_gemm_op_MNKList()
    for M, N, K in MNKList:
        helix_oracle_flops = get_Helix_Oracle_result(prof_dict, M, N, K)
        helix_default_flops = get_Helix_Default_result(prof_dict, M, N, K)
        helix_verified_flops = get_Helix_Verified_result(prof_dict, M, N, K)
        helix_static1_flops = get_Helix_Static1_result(prof_dict, M, N, K)
        helix_static2_flops = get_Helix_Static2_result(prof_dict, M, N, K)
        print(f'{M}x{N}x{K}: Helix_Oracle: {helix_oracle_flops:.2f} TFlops, Helix_Default: {helix_default_flops:.2f} TFlops, Helix_Verified: {helix_verified_flops:.2f} TFlops, Helix_Static1: {helix_static1_flops:.2f} TFlops, Helix_Static2: {helix_static2_flops:.2f} TFlops')
