"""python3 benchmark_model_level_eval.py -m {LLM,CNN} -b <backend> -s <system>.
Same command line, table shape and fall-through message as the reference's
scripts/benchmark_model_level_eval.py:12-44."""
import argparse

from _dispatch import resolve, MI355X_BACKENDS

func_dict = {
    ('LLM', 'MI355X_FP16', 'Helix'): ('MI355X_FP16.benchmark_MI355X_FP16_model_level_LLM', 'MI355X_FP16_Helix_model_level_LLM_benchmark'),
    ('CNN', 'MI355X_FP16', 'Helix'): ('MI355X_FP16.benchmark_MI355X_FP16_model_level_CNN', 'MI355X_FP16_Helix_model_level_CNN_benchmark'),
    ('LLM', 'MI355X_FP32', 'Helix'): ('MI355X_FP32.benchmark_MI355X_FP32_model_level_LLM', 'MI355X_FP32_Helix_model_level_LLM_benchmark'),
    ('CNN', 'MI355X_FP32', 'Helix'): ('MI355X_FP32.benchmark_MI355X_FP32_model_level_CNN', 'MI355X_FP32_Helix_model_level_CNN_benchmark'),
    ('LLM', 'MI355X_FP16', 'rocblas'): ('MI355X_FP16.benchmark_MI355X_FP16_model_level_LLM', 'MI355X_FP16_rocblas_model_level_LLM_benchmark'),
    ('LLM', 'MI355X_FP32', 'rocblas'): ('MI355X_FP32.benchmark_MI355X_FP32_model_level_LLM', 'MI355X_FP32_rocblas_model_level_LLM_benchmark'),
    ('CNN', 'MI355X_FP16', 'miopen'): ('MI355X_FP16.benchmark_MI355X_FP16_model_level_CNN', 'MI355X_FP16_miopen_model_level_CNN_benchmark'),
    ('CNN', 'MI355X_FP32', 'miopen'): ('MI355X_FP32.benchmark_MI355X_FP32_model_level_CNN', 'MI355X_FP32_miopen_model_level_CNN_benchmark'),
}

if __name__ == "__main__":
    parser = argparse.ArgumentParser(description="Benchmark Model level performance")
    parser.add_argument("-m", "--model", type=str, choices=['LLM', 'CNN'], default='LLM', help="model name")
    parser.add_argument("-b", "--backend", type=str, choices=MI355X_BACKENDS, default='MI355X_FP16', help="backend")
    parser.add_argument("-s", "--system", type=str, choices=['Helix', 'rocblas', 'miopen'], default='Helix', help="system")
    args = parser.parse_args()

    if (args.model, args.backend, args.system) in func_dict.keys():
        resolve(func_dict[(args.model, args.backend, args.system)])()
    else:
        print(f'{args.model} {args.backend} {args.system} is not supported')
