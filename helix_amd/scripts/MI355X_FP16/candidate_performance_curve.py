"""Measured throughput of every candidate configuration on a few shapes, next to the cost model's pick:
the data behind a "how sharp is the optimum" curve.

Mirrors scripts/Ampere_FP16/candidate_performance_curve.py:6-40 (same four shapes, same two printed
lines per shape).  The reference prints the best candidate's id on every line (`min_id`, :32); here
each line carries the candidate's own id.
"""
import os

from utils.helix_runtime import read_prof_dict
from MI355X_FP16.MI355X_FP16_gemm import short_value, config_cost, run_config

root_path = os.getcwd()

CURVE_SHAPES = [(476, 1024, 1024), (128, 512, 1000), (5124, 700, 2048), (32, 50515, 100)]


def get_all_candidate_performance(prof_dict, M, N, K):
    """Returns (best_id, best_config, [(id, config, tflops or None)]) and prints them."""
    min_cost, min_config, min_id = float("inf"), None, 0
    for id, (k, v) in enumerate(prof_dict.items(), start=1):
        cost = config_cost(k, v, M, N, K, short_value(prof_dict, k))
        if min_cost > cost:
            min_cost, min_config, min_id = cost, k, id
    print(f'Best candidate id: {min_id}, config = {min_config}')
    rows = []
    for id, k in enumerate(prof_dict.keys(), start=1):
        try:
            cost = run_config(k, M, N, K)
            tflops = 2 * M * N * K / 1e12 / cost
            print(f'candidate id: {id}, flops = {tflops} Tflops')
        except Exception as e:       # a configuration that refuses the shape (GEMV libraries on wide problems)
            tflops = None
            print(f'candidate id: {id}, skipped ({e})')
        rows.append((id, k, tflops))
    return min_id, min_config, rows


if __name__ == "__main__":

    prof_dict = read_prof_dict("MI355X_FP16")
    for M, N, K in CURVE_SHAPES:
        get_all_candidate_performance(prof_dict, M, N, K)
