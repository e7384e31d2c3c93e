"""python3 build_template.py -b <backend>: compile every kernel-template configuration.
Same command line as the reference's scripts/build_template.py:6-18, with the MI355X backends."""
import argparse

from _dispatch import resolve, MI355X_BACKENDS

func_dict = {
    'MI355X_FP16': [('MI355X_FP16.build_MI355X_FP16', 'build_Helix_MI355X_FP16_gemm_kernel')],
    'MI355X_FP32': [('MI355X_FP32.build_MI355X_FP32', 'build_Helix_MI355X_FP32_gemm_kernel')],
}

if __name__ == "__main__":
    parser = argparse.ArgumentParser(description="Get runtime cost of an operation")
    parser.add_argument("-b", "--backend", type=str, choices=MI355X_BACKENDS, default='MI355X_FP16', help="backend")
    args = parser.parse_args()

    import time
    T1 = time.perf_counter()
    for row in func_dict[args.backend]:
        resolve(row)()
    T2 = time.perf_counter()
    print(f'Building time: {T2-T1} seconds')
