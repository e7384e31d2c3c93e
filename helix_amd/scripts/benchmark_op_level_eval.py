"""python3 benchmark_op_level_eval.py -o {GEMM,Conv} -b <backend> -s <system>.
Same command line, table shape and fall-through message as the reference's
scripts/benchmark_op_level_eval.py:12-44."""
import argparse

from _dispatch import resolve, MI355X_BACKENDS

func_dict = {
    ('GEMM', 'MI355X_FP16', 'Helix'): ('MI355X_FP16.benchmark_MI355X_FP16_gemm', 'MI355X_FP16_Helix_op_level_GEMM_benchmark'),
    ('Conv', 'MI355X_FP16', 'Helix'): ('MI355X_FP16.benchmark_MI355X_FP16_conv', 'MI355X_FP16_Helix_op_level_Conv_benchmark'),
    ('GEMM', 'MI355X_FP32', 'Helix'): ('MI355X_FP32.benchmark_MI355X_FP32_gemm', 'MI355X_FP32_Helix_op_level_GEMM_benchmark'),
    ('Conv', 'MI355X_FP32', 'Helix'): ('MI355X_FP32.benchmark_MI355X_FP32_conv', 'MI355X_FP32_Helix_op_level_Conv_benchmark'),
    ('GEMM', 'MI355X_FP16', 'rocblas'): ('MI355X_FP16.benchmark_MI355X_FP16_gemm', 'MI355X_FP16_rocblas_op_level_GEMM_benchmark'),
    ('GEMM', 'MI355X_FP32', 'rocblas'): ('MI355X_FP32.benchmark_MI355X_FP32_gemm', 'MI355X_FP32_rocblas_op_level_GEMM_benchmark'),
    ('Conv', 'MI355X_FP16', 'miopen'): ('MI355X_FP16.benchmark_MI355X_FP16_conv', 'MI355X_FP16_miopen_op_level_Conv_benchmark'),
    ('Conv', 'MI355X_FP32', 'miopen'): ('MI355X_FP32.benchmark_MI355X_FP32_conv', 'MI355X_FP32_miopen_op_level_Conv_benchmark'),
}

if __name__ == "__main__":
    parser = argparse.ArgumentParser(description="Benchmark OP level performance")
    parser.add_argument("-o", "--op", type=str, choices=['GEMM', 'Conv'], default='GEMM', help="op type")
    parser.add_argument("-b", "--backend", type=str, choices=MI355X_BACKENDS, default='MI355X_FP16', help="backend")
    parser.add_argument("-s", "--system", type=str, choices=['Helix', 'rocblas', 'miopen'], default='Helix', help="system")
    args = parser.parse_args()

    if (args.op, args.backend, args.system) in func_dict.keys():
        resolve(func_dict[(args.op, args.backend, args.system)])()
    else:
        print(f'{args.op} {args.backend} {args.system} is not supported')
