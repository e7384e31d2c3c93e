"""Model-level LLM benchmark of the MI355X_FP32 backend: summed per-GEMM latency of the BERT,
LLaMA-2 and GPT-2 op-sets.  Mirrors scripts/Ampere_FP32/benchmark_Ampere_FP32_model_level_LLM.py:9-27."""
import math
import os

from utils.get_benchmark_shape_list import get_llm_opset_MNKList, get_baseline_bert_MNKList
from utils.helix_runtime import read_prof_dict
from MI355X_FP32.MI355X_FP32_gemm import get_MI355X_FP32_gemm_Helix_result, get_MI355X_FP32_gemm_rocblas_result

root_path = os.getcwd()


def _summed_cost(prof_dict, MNKList, backend):
    # identical shapes repeat many times in the op-sets; measure each distinct shape once
    memo, total = {}, 0
    for M, N, K in MNKList:
        if (M, N, K) not in memo:
            memo[(M, N, K)], _ = get_MI355X_FP32_gemm_Helix_result(prof_dict, M, N, K, backend)
        total += memo[(M, N, K)]
    return total


def MI355X_FP32_Helix_model_level_LLM_benchmark(backend="hip"):
    prof_dict = read_prof_dict("MI355X_FP32")

    Bert_MNKList, LLAMA2_MNKList, GPT2_MNKList = get_llm_opset_MNKList()

    helix_Bert_cost = _summed_cost(prof_dict, Bert_MNKList, backend)
    helix_LLAMA2_cost = _summed_cost(prof_dict, LLAMA2_MNKList, backend)
    helix_GPT2_cost = _summed_cost(prof_dict, GPT2_MNKList, backend)

    print(f'Bert: {helix_Bert_cost:.2f} ms, LLAMA2: {helix_LLAMA2_cost:.2f} ms, GPT2: {helix_GPT2_cost:.2f} ms')


def MI355X_FP32_rocblas_model_level_LLM_benchmark():
    """Vendor column: mirrors Ampere_FP32_cublas_model_level_LLM_benchmark."""
    costs = []
    for MNKList in get_llm_opset_MNKList():
        memo, total = {}, 0
        for M, N, K in MNKList:
            if (M, N, K) not in memo:
                memo[(M, N, K)], _ = get_MI355X_FP32_gemm_rocblas_result(M, N, K)
            total += memo[(M, N, K)]
        costs.append(total)
    print(f'Bert: {costs[0]:.2f} ms, LLAMA2: {costs[1]:.2f} ms, GPT2: {costs[2]:.2f} ms')


def MI355X_FP32_Helix_baseline_bert_benchmark(backend="hip"):
    """BERT-base encoder GEMMs at M = 4096, x12 layers, plus the irregular 4000x2300x770 GEMM."""
    prof_dict = read_prof_dict("MI355X_FP32")
    cost = _summed_cost(prof_dict, get_baseline_bert_MNKList(), backend)
    print(f'Bert-base (M=4096, 12 layers + 4000x2300x770): {cost:.3f} ms')
    return cost


if __name__ == "__main__":

    MI355X_FP32_Helix_model_level_LLM_benchmark(backend="hip")
