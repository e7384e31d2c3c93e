"""python3 profile_template.py -b <backend>: time every configuration and write the cost-model dict.
Same command line and closing line as the reference's scripts/profile_template.py:9-24."""
import argparse
import time

from _dispatch import resolve, MI355X_BACKENDS

func_dict = {
    'MI355X_FP16': ('MI355X_FP16.profile_MI355X_FP16', 'profile_Helix_MI355X_FP16_gemm_kernel'),
    'MI355X_FP32': ('MI355X_FP32.profile_MI355X_FP32', 'profile_Helix_MI355X_FP32_gemm_kernel'),
}

if __name__ == "__main__":
    parser = argparse.ArgumentParser(description="Get runtime cost of an operation")
    parser.add_argument("-b", "--backend", type=str, choices=MI355X_BACKENDS, default='MI355X_FP16', help="backend")
    args = parser.parse_args()

    T1 = time.perf_counter()
    resolve(func_dict[args.backend])()
    T2 = time.perf_counter()
    print(f'Profiling time: {T2-T1} seconds')
