"""Op-level GEMM benchmark of the MI355X_FP16 backend.
Mirrors scripts/Ampere_FP16/benchmark_Ampere_FP16_gemm.py:9-23 (same loop, same output line)."""
import math
import os

from utils.get_benchmark_shape_list import get_gemm_op_MNKList
from utils.helix_runtime import read_prof_dict
from MI355X_FP16.MI355X_FP16_gemm import get_MI355X_FP16_gemm_Helix_result, get_MI355X_FP16_gemm_rocblas_result

root_path = os.getcwd()


def MI355X_FP16_Helix_op_level_GEMM_benchmark(backend="hip"):
    prof_dict = read_prof_dict("MI355X_FP16")

    MNKList = get_gemm_op_MNKList()
    for M, N, K in MNKList:
        _, helix_tflops = get_MI355X_FP16_gemm_Helix_result(prof_dict, M, N, K, backend)
        print(f'{M}x{N}x{K}: Helix: {helix_tflops:.2f} TFLOPS')


def MI355X_FP16_rocblas_op_level_GEMM_benchmark():
    """Vendor column: mirrors Ampere_FP16_cublas_op_level_GEMM_benchmark (benchmark_Ampere_FP16_gemm.py:19-23)."""
    MNKList = get_gemm_op_MNKList()
    for M, N, K in MNKList:
        _, rocblas_tflops = get_MI355X_FP16_gemm_rocblas_result(M, N, K)
        print(f'{M}x{N}x{K}: rocblas: {rocblas_tflops:.2f} TFLOPS')


if __name__ == "__main__":

    MI355X_FP16_Helix_op_level_GEMM_benchmark(backend="hip")
    MI355X_FP16_rocblas_op_level_GEMM_benchmark()
