"""python3 runtime_cost.py -b <backend>: cost-model lookup overhead next to kernel time.
Same command line as the reference's scripts/runtime_cost.py:8-21."""
import argparse

from _dispatch import resolve, MI355X_BACKENDS

func_dict = {
    'MI355X_FP16': ('MI355X_FP16.MI355X_FP16_runtime_cost', 'MI355X_FP16_runtime_cost'),
    'MI355X_FP32': ('MI355X_FP32.MI355X_FP32_runtime_cost', 'MI355X_FP32_runtime_cost'),
}

if __name__ == "__main__":
    parser = argparse.ArgumentParser(description="Get runtime cost of an operation")
    parser.add_argument("-b", "--backend", type=str, choices=MI355X_BACKENDS, default='MI355X_FP16', help="backend")
    args = parser.parse_args()

    if args.backend in func_dict:
        resolve(func_dict[args.backend])()
    else:
        raise ValueError("Invalid backend")
