"""Cost model and single-GEMM runner of the MI355X_FP16 backend.

Mirrors scripts/Ampere_FP16/Ampere_FP16_gemm.py:420-446 (`cost_model`, `get_Ampere_FP16_gemm_Helix_result`)
and :548-553 (vendor-library result).  The TVM-on-GPU alternative backend of the reference (:17-417)
has no counterpart: the only backend value is "hip".
"""
import math
import os

from utils.helix_runtime import load, tuned_config, fastest_of
from utils.roofline import NUM_CU, HBM_BYTES_PER_S, gemm_bytes
from MI355X_FP16.build_MI355X_FP16 import library_for_key, kernel_library, SPLITK_MAX
from MI355X_FP16.profile_MI355X_FP16 import PROFILE_K, PROFILE_K_SHORT

root_path = os.getcwd()

HBM_SUSTAINED_FRACTION = 0.8  # share of the datasheet HBM rate a streaming kernel sustains
# ... and what the tile kernels sustain when a problem is a pass over a cold operand (on 8192 x 28672 weights the
# fastest 32-row tile measures 5.2 - 5.5 TB/s, the one the model ranks first 4.4 - 4.9): their profile point is a hot
# 16 x 16-tile problem, so this floor is what ranks them against the weight-streaming kernels, whose profile point
# is cold
TILE_HBM_SUSTAINED_FRACTION = 0.60
GEMV_LAUNCH_FLOOR_S = 3.4e-6       # a kernel launch on an idle queue; keeps tiny problems from looking free
GEMV_MFMA_FLOOR_S = 4.4e-6         # 9 or more activation rows: the LDS-streamed MFMA variant (staging + cross-wave sum)
GEMV_MFMA_MIN_M = 9                # MFMA_MIN_M of src_template/MI355X_FP16/gemv.hip
# the weight-streaming kernels pass over the weights once per 16 activation rows: beyond one pass a tile kernel,
# which reads them once per BLOCK_ROWS rows, is the better streamer, and the per-round share the model assumes
# for them no longer holds (measured: 661 x 768 x 3072 FP32, 103 us against 27 us)
GEMV_MAX_ROWS = 16
# Timing loops (the reference's and these) launch again and again on the same buffers, so weights that fit the 256 MB
# memory-side cache stream from it: measured on M = 1 and 2, 33 MB of weights take 0.45 of their share of the profiled
# (268 MB, HBM-bound) launch, 75 MB 0.66, 100 MB 0.72, 150 MB 0.83
GEMV_RESIDENT_BYTES = 32e6
GEMV_STREAMED_BYTES = 200e6
GEMV_RESIDENT_SHARE = 0.45
GEMV_WIDE_STREAM_ROWS = 4          # activation-row tiles up to this many rows keep 8 KiB of loads in flight per wave
GEMV_SPLITK_EXTRA_S = 2e-6         # the K-partitioned GEMV library's reduction pass on a problem too small to need it
SPLITK_REDUCE_LAUNCH_S = 3e-6      # adding the partitions (the tail of the launch behind the last partial store, measured 3.3 us
                                   # at eight partitions), beyond what the profiled value already holds
ROUND_OVERLAP_S = 1e-6             # part of a round's fixed time that later rounds of one launch do not pay again


def split_factor(k, M, N, K):
    """K partitions a split-K library uses for this problem (same rule as the library's host side):
    enough to give each of the 256 compute units a workgroup, between 2 and SPLITK_MAX, and at least two
    K tiles per partition.  The reference's split is always 2 (`* (k[5] + 1)`, Ampere_FP16_gemm.py:424)."""
    if k[5] == 0 or k[0] == 0:
        return 1
    tiles = math.ceil(M / k[1]) * math.ceil(N / k[2])
    ktiles = math.ceil(K / k[6])
    s = min(NUM_CU // max(tiles, 1), SPLITK_MAX, ktiles // 2)
    return max(s, 2)


def resident_share(weight_bytes):
    """Share of the profiled (HBM-bound) streaming time that weights of this size take in a timing loop."""
    if weight_bytes <= GEMV_RESIDENT_BYTES:
        return GEMV_RESIDENT_SHARE
    if weight_bytes >= GEMV_STREAMED_BYTES:
        return 1.0
    ramp = (weight_bytes - GEMV_RESIDENT_BYTES) / (GEMV_STREAMED_BYTES - GEMV_RESIDENT_BYTES)
    return GEMV_RESIDENT_SHARE + (1.0 - GEMV_RESIDENT_SHARE) * ramp


def round_time(v, v_short, K):
    """Seconds of one round of tiles walking K: the line through the two profiled points (K_short, v_short)
    and (K_profile, v); proportional to K, as the first version of this model was, when only the long point
    exists."""
    if v_short is None or not (v_short < float("inf")) or not (v < float("inf")):
        return v * K / PROFILE_K
    t = v_short + (v - v_short) * (K - PROFILE_K_SHORT) / (PROFILE_K - PROFILE_K_SHORT)
    return max(t, 0.25 * v_short)


def config_cost(k, v, M, N, K, v_short=None):
    """Predicted seconds of configuration k (profiled round time v, and v_short at the short K when the
    profile holds it) on an M x N x K problem.

    Reference form (Ampere_FP16_gemm.py:424-426): rounds = ceil(blocks / SMs), cost = rounds * v with
    108 SMs and K ignored.  Here SMs -> 256 compute units and the round time follows the K each tile walks
    (split-K divides it)."""
    if k[0] == 0:
        # weight-streaming kernel: HBM-bound, so a partial round costs its share of a round (no
        # quantisation), never less than a launch; the streamed operand is the larger of M and N
        small, big = (M, N) if M <= N else (N, M)
        if small > GEMV_MAX_ROWS or small > k[1]:
            # the three rows of a family are one library profiled at 1, 4 and 16 activation rows: a row describes
            # problems of up to its own row count (the reference's ceil(M / rows) passes, Ampere_FP16_gemm.py:420,
            # would charge a pass per row tile for what the kernel does in one)
            return float("inf")
        num_block = math.ceil(big / k[2])
        floor = GEMV_LAUNCH_FLOOR_S if small < GEMV_MFMA_MIN_M else GEMV_MFMA_FLOOR_S
        k_walk = max(K, 512)
        # the profiled launch holds one launch's fixed time, which does not scale with the problem
        stream = max(v - GEMV_LAUNCH_FLOOR_S, 0.0) * num_block / NUM_CU * k_walk / PROFILE_K
        # the eight-row tile of the dot-product variant keeps half as many loads in flight and streams cache-resident
        # weights no faster than cold ones (4096 x 4096 at 8 rows 10.3 us against 5.4 us at one row)
        if small <= GEMV_WIDE_STREAM_ROWS or small >= GEMV_MFMA_MIN_M:
            stream *= resident_share(big * k_walk * 2)
        cost = floor + stream
        return cost + (GEMV_SPLITK_EXTRA_S if k[5] == 1 else 0.0)
    splits = split_factor(k, M, N, K)
    num_block = math.ceil(M / k[1]) * math.ceil(N / k[2]) * splits
    w = math.ceil(num_block / NUM_CU)
    # a tile walks K in whole BLOCK_K steps
    k_walk = math.ceil(K / k[6]) * k[6]
    if k[5] == 1:
        # the profiled value is two rounds of half-K partitions; a round of this problem walks K / splits
        per_round = round_time(v, v_short, 2 * k_walk / splits) / 2
        # the FP32 partials are written and read back by a second kernel
        extra = SPLITK_REDUCE_LAUNCH_S + (splits + 1) * M * N * 4 / (HBM_SUSTAINED_FRACTION * HBM_BYTES_PER_S)
    else:
        per_round = round_time(v, v_short, k_walk)
        extra = 0.0
    cost = w * per_round + extra
    if v_short is not None:
        cost -= ROUND_OVERLAP_S * (w - 1)
    # a tile round cannot beat streaming every operand once from HBM at the sustained rate
    return max(cost, gemm_bytes(M, N, K, 2) / (TILE_HBM_SUSTAINED_FRACTION * HBM_BYTES_PER_S))


def short_value(prof_dict, k):
    """The short-K profile point of configuration k, or None (plain dicts, files without the second point)."""
    return getattr(prof_dict, "short", {}).get(k)


def cost_model(prof_dict, M, N, K):
    min_cost = float("inf")
    best_config = (1, 1, 1, 1, 1, 0, 32)
    for k, v in prof_dict.items():
        cost = config_cost(k, v, M, N, K, short_value(prof_dict, k))
        if min_cost > cost:
            min_cost = cost
            best_config = k
    return best_config


# "Verified" selection: the cost model ranks, the device decides among the first few.  Predictions of the leading
# configurations lie within a few per cent of each other while their measured times differ by 5 - 25 %; timing
# VERIFY_TOP of them once per shape (a handful of launches, against hundreds for the exhaustive search) recovers
# most of that (measured over 30 convolution layers: picked / fastest 1.07 -> 1.03 with four candidates, 1.02 with six,
# 1.015 with eight).  The runners keep the winner per problem (utils.helix_runtime.tuned_config), so the candidates of
# a problem are timed once per profile: twelve of them.
VERIFY_TOP = 12


def ranked_configs(prof_dict, M, N, K, top=VERIFY_TOP):
    """The `top` configurations with the lowest predicted cost, best first; cost_model returns the first of them."""
    ranked = sorted(prof_dict.items(), key=lambda kv: config_cost(kv[0], kv[1], M, N, K, short_value(prof_dict, kv[0])))
    return [k for k, _ in ranked[:top]]


def padded_k(K):
    """The FP16 kernels load 16-byte chunks along K; a K that is not a multiple of 8 halves is run on
    buffers whose rows are zero-padded to the next multiple (zeros add nothing to the dot products)."""
    return math.ceil(K / 8) * 8


def run_config(k, M, N, K, warmup=10, iters=10, outer=1):
    """Seconds per launch (mean) of configuration k on the real, unpadded M and N.  The reference pads
    M and N up to the tile (Ampere_FP16_gemm.py:438) because its kernel has no bounds checks; the
    MI355X kernels predicate their edges instead."""
    lib = load(library_for_key(k))
    if k[0] == 0 and M > N:
        M, N = N, M   # the GEMV kernel streams its second operand; gemv.cu:384-386 swaps the same way
    _, avg, _ = lib.bench(M, N, padded_k(K), warmup=warmup, iters=iters, outer=outer, rotate_bytes=0)
    return avg


def verified_config(prof_dict, M, N, K, top=VERIFY_TOP):
    """The fastest of the cost model's first `top` configurations on this problem (utils.helix_runtime.fastest_of:
    2 + 5 launches each, the leaders timed again)."""
    return fastest_of(ranked_configs(prof_dict, M, N, K, top),
                      lambda k, warmup, iters: run_config(k, M, N, K, warmup=warmup, iters=iters), f"{M}x{N}x{K}")


def select_config(prof_dict, M, N, K):
    """The configuration the runner launches: the cost model's ranking, settled on the device the first time a
    problem is met and remembered beside the profile (utils.helix_runtime.tuned_config); the cost model's first
    choice alone with HELIX_SELECTION=model."""
    return tuned_config("MI355X_FP16", ("gemm", M, N, K), prof_dict, lambda: cost_model(prof_dict, M, N, K),
                        lambda: verified_config(prof_dict, M, N, K))


def get_MI355X_FP16_gemm_Helix_result(prof_dict, M, N, K, backend="hip"):
    if backend != "hip":
        raise ValueError(f"backend {backend!r} is not available for MI355X_FP16 (only 'hip')")
    best_config = select_config(prof_dict, M, N, K)
    cost = run_config(best_config, M, N, K) * 1e3
    tflops = 2 * M * N * K / 1e9 / cost

    return cost, tflops


def get_MI355X_FP16_gemm_rocblas_result(M, N, K):
    """The vendor library on the same problem (rocblas_gemm_ex, FP16 in / FP32 compute), timed the same way.
    Mirrors get_Ampere_FP16_gemm_cublas_result (Ampere_FP16_gemm.py:548-553)."""
    lib = load(kernel_library("rocblas_f16"))
    _, avg, _ = lib.bench(M, N, K, warmup=10, iters=10, outer=1, rotate_bytes=0)
    cost = avg * 1e3
    return cost, 2 * M * N * K / 1e9 / cost


def get_MI355X_FP16_gemm_Verified_result(prof_dict, M, N, K, top=VERIFY_TOP):
    """The fastest of the cost model's first `top` configurations: each timed briefly, the winner timed again with
    the runner's launch counts.  Returns (cost_ms, tflops, key)."""
    best = verified_config(prof_dict, M, N, K, top)
    cost = run_config(best, M, N, K)
    return cost * 1e3, 2 * M * N * K / 1e12 / cost, best


def get_MI355X_FP16_gemm_Oracle_result(prof_dict, M, N, K):
    """Exhaustive per-shape search: run every candidate, keep the fastest
    (benchmark_Ampere_FP16_performance_comparison.py:56-69).  Returns (cost_ms, tflops, key)."""
    min_cost, best = float("inf"), None
    for k in prof_dict.keys():
        if k[0] == 0 and min(M, N) > 16:
            continue   # the weight-streaming kernel re-reads the weights per 16 activation rows
        try:
            cost = run_config(k, M, N, K, warmup=2, iters=5)
        except Exception:
            continue
        if min_cost > cost:
            min_cost, best = cost, k
    return min_cost * 1e3, 2 * M * N * K / 1e12 / min_cost, best
