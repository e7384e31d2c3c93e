"""python3 helix_run.py <library.so> M N K [warmup iters]

Runs one kernel-template library on an M x N x K problem the way the reference runs one of its executables
(`os.popen(f"{exe} {M} {N} {K}")`, scripts/Ampere_FP16/profile_Ampere_FP16.py:36-37) and prints the reference's
result line (src_template/Ampere_FP16/gemm.cu:687-689):

    M N K = %6d %6d %6d, Time = %12.8lf %12.8lf %12.8lf s, AVG Performance = %10.4lf Tflops

so a consumer that parses the whitespace-split token [-8] (the mean seconds) keeps working.  The timing
itself is helix_bench of include/helix_abi.h (warm-up launches, then event-timed groups of launches on
initialised buffers).
"""
import sys

from utils.helix_runtime import load, reference_line


def main(argv):
    if len(argv) not in (5, 7):
        print(__doc__.splitlines()[0], file=sys.stderr)
        return 2
    path = argv[1]
    M, N, K = (int(v) for v in argv[2:5])
    warmup, iters = (int(argv[5]), int(argv[6])) if len(argv) == 7 else (10, 10)
    mn, avg, mx = load(path).bench(M, N, K, warmup=warmup, iters=iters, outer=3)
    print(reference_line(M, N, K, mn, avg, mx))
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
