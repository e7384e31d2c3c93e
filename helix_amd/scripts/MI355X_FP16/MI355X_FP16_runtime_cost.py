"""Selection overhead of the MI355X_FP16 backend: time of one cost-model lookup next to the time of
the selected kernel.  Mirrors scripts/Ampere_FP16/Ampere_FP16_runtime_cost.py:7-40 (same shapes, same
print; the reference divides by an extra 1000 and labels the result ms, :29 -- here both numbers
really are milliseconds).
"""
import time
import os

from utils.helix_runtime import read_prof_dict
from MI355X_FP16.MI355X_FP16_gemm import short_value, config_cost, run_config

root_path = os.getcwd()


def cost_model(prof_dict, M, N, K):
    cost_map = {}
    for k, v in prof_dict.items():
        cost_map[k] = config_cost(k, v, M, N, K, short_value(prof_dict, k))
    best_config = min(cost_map, key=cost_map.get)
    return best_config


def get_Helix_runtime_cost(prof_dict, M, N, K):
    T1 = time.perf_counter()
    for i in range(100):
        best_config = cost_model(prof_dict, M, N, K)
    T2 = time.perf_counter()
    cost = run_config(best_config, M, N, K)

    return (T2 - T1) / 100 * 1000, cost * 1000


def MI355X_FP16_runtime_cost():

    prof_dict = read_prof_dict("MI355X_FP16")

    MNKList = [(64, 64, 64), (128, 128, 128), (256, 256, 256), (512, 512, 512), (1024, 1024, 1024), (2048, 2048, 2048), (4096, 4096, 4096)]
    for M, N, K in MNKList:
        runtime_cost, op_cost = get_Helix_runtime_cost(prof_dict, M, N, K)
        print(f'The runtime cost of {M}x{N}x{K} is {runtime_cost} ms, and the op cost is {op_cost} ms.')


if __name__ == '__main__':

    MI355X_FP16_runtime_cost()
