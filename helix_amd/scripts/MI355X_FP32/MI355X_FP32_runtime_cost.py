"""Selection overhead of the MI355X_FP32 backend.  Mirrors scripts/Ampere_FP32/Ampere_FP32_runtime_cost.py:7-38."""
import time
import os

from utils.helix_runtime import read_prof_dict
from MI355X_FP32.MI355X_FP32_gemm import cost_model, run_config

root_path = os.getcwd()


def get_Helix_runtime_cost(prof_dict, M, N, K):
    T1 = time.perf_counter()
    for i in range(100):
        best_config = cost_model(prof_dict, M, N, K)
    T2 = time.perf_counter()
    cost = run_config(best_config, M, N, K)

    return (T2 - T1) / 100 * 1000, cost * 1000


def MI355X_FP32_runtime_cost():

    prof_dict = read_prof_dict("MI355X_FP32")

    MNKList = [(64, 64, 64), (128, 128, 128), (256, 256, 256), (512, 512, 512), (1024, 1024, 1024), (2048, 2048, 2048), (4096, 4096, 4096)]
    for M, N, K in MNKList:
        runtime_cost, op_cost = get_Helix_runtime_cost(prof_dict, M, N, K)
        print(f'The runtime cost of {M}x{N}x{K} is {runtime_cost} ms, and the op cost is {op_cost} ms.')


if __name__ == '__main__':

    MI355X_FP32_runtime_cost()
