"""Cost model and single-GEMM runner of the MI355X_FP32 backend.
Mirrors scripts/Ampere_FP32/Ampere_FP32_gemm.py:89-107 (`cost_model`, `get_Ampere_FP32_gemm_Helix_result`);
the TVM alternative backend (:16-86, :108-136) has no counterpart."""
import math
import os

from utils.helix_runtime import load, tuned_config, fastest_of
from utils.roofline import NUM_CU, HBM_BYTES_PER_S, gemm_bytes
from MI355X_FP32.build_MI355X_FP32 import library_for_key, kernel_library
from MI355X_FP32.profile_MI355X_FP32 import PROFILE_K, PROFILE_K_SHORT, GEMV_PROFILE_K

root_path = os.getcwd()

HBM_SUSTAINED_FRACTION = 0.8
GEMV_LAUNCH_FLOOR_S = 3.4e-6
# the weight-streaming kernels pass over the weights once per 16 activation rows: beyond one pass a tile kernel,
# which reads them once per BLOCK_ROWS rows, is the better streamer, and the per-round share the model assumes
# for them no longer holds (measured: 661 x 768 x 3072 FP32, 103 us against 27 us)
GEMV_MAX_ROWS = 16
GEMV_SPLITK_EXTRA_S = 2e-6        # the K-partitioned library's reduction pass on a problem too small to need it
# a further round of tiles costs what the two-round profile shows beyond one round, but never less than the matrix
# pipes need for it at this fraction of their peak: the small-tile configurations fit several workgroups on a
# compute unit, so their second round is almost free in the profile and stays so only until the pipes are full
FP32_MFMA_FLOPS = 157.3e12
LATER_ROUND_MFMA_FRACTION = 0.85
# configurations with BK = 32 (one wave group) measure about this much slower over several rounds than their
# one- and two-round profile points predict (140 GEMM shapes, every configuration timed on each)
BK32_MULTI_ROUND_COST = 0.05

# rate at which the compute units take A and B tiles in (bytes of M*N*K*4*(1/BM + 1/BN) per second): what the
# small-tile configurations reach on 2048^3 ... 8192^3
OPERAND_BYTES_PER_S = 6.5e12


SPLITK_MAX, SPLITK_TARGET = 8, 768   # as in src_template/MI355X_FP32/sgemm.hip
SPLITK_MIN_K_FEW, SPLITK_FEW_TILES = 256, 128
SPLITK_MIN_K_TINY, SPLITK_TINY_TILES = 64, 32
SPLITK_MFMA_FRACTION, SPLITK_REDUCE_BYTES_PER_S, SPLITK_MIN_GAIN, SPLITK_MIN_K_BALANCE = 0.8, 5e12, 0.98, 128
SPLITK_REDUCE_LAUNCH_S = 4e-6   # the reduction kernel of a K-partitioned launch


def split_factor(k, M, N, K):
    """K partitions the SGEMM libraries use for this problem (same rule, same arithmetic as their host side).  At
    most SPLITK_FEW_TILES tiles: as many as reach SPLITK_TARGET workgroups, at most SPLITK_MAX, at least
    SPLITK_MIN_K_FEW of K per partition (SPLITK_MIN_K_TINY up to SPLITK_TINY_TILES tiles).  More tiles: the count
    that makes rounds of 256 workgroups x one partition's K walk, plus a fixed cost per workgroup and the
    reduction pass, smallest."""
    if k[2] == 0:
        return 1
    BM, BN, BK = k[0], k[1], k[2]
    tiles = math.ceil(M / BM) * math.ceil(N / BN)
    if tiles <= 0:
        return 1
    if tiles <= SPLITK_FEW_TILES:
        min_k = SPLITK_MIN_K_TINY if tiles <= SPLITK_TINY_TILES else SPLITK_MIN_K_FEW
        return max(min(math.ceil(SPLITK_TARGET / tiles), SPLITK_MAX, K // min_k), 1)
    per_k = 2.0 * BM * BN * NUM_CU / (SPLITK_MFMA_FRACTION * FP32_MFMA_FLOPS)
    fixed = 1e-6 + 1.5e-6 * (BM * BN) / (128.0 * 128.0)
    ktiles = (K + BK - 1) // BK
    best, best_t = 1, 0.0
    s = 1
    while s <= SPLITK_MAX and (s == 1 or K // s >= SPLITK_MIN_K_BALANCE):
        walk = float(((ktiles + s - 1) // s) * BK)
        rounds = float((tiles * s + NUM_CU - 1) // NUM_CU)
        reduce = SPLITK_REDUCE_LAUNCH_S + (s + 1.0) * float(M) * float(N) * 4.0 / SPLITK_REDUCE_BYTES_PER_S if s > 1 else 0.0
        t = rounds * (walk * per_k + fixed) + reduce
        if s == 1 or t < best_t * SPLITK_MIN_GAIN:
            best, best_t = s, t
        s += 1
    return best


def _line(x0, y0, x1, y1, x):
    return y0 + (y1 - y0) * (x - x0) / (x1 - x0)


def _finite(*values):
    return all(v is not None and v < float("inf") for v in values)


def config_cost(k, v, M, N, K, points=None):
    """rounds * time-per-round as in Ampere_FP32_gemm.py:93-95, with 256 compute units for 108 SMs and
    the round time following K (the reference ignores K).  `points` = (short, two_rounds, short_two_rounds)
    of the profile when it holds them: then the first round costs the line through the two one-round points
    and each further round the line through the two-round increments, floored by the matrix pipes' time for it."""
    if k[2] == 0:
        small, big = (M, N) if M <= N else (N, M)
        if small > GEMV_MAX_ROWS:
            return float("inf")
        num_block = math.ceil(small / k[0]) * math.ceil(big / k[1])
        cost = max(num_block / NUM_CU * v * max(K, 256) / GEMV_PROFILE_K, GEMV_LAUNCH_FLOOR_S)
        return cost + (GEMV_SPLITK_EXTRA_S if k[5] == 1 else 0.0)
    tiles_m, tiles_n = math.ceil(M / k[0]), math.ceil(N / k[1])
    splits = split_factor(k, M, N, K)
    w = math.ceil(tiles_m * tiles_n * splits / NUM_CU)
    hbm_floor = gemm_bytes(M, N, K, 4) / (HBM_SUSTAINED_FRACTION * HBM_BYTES_PER_S)
    # K a workgroup walks, in whole BK steps
    k_walk = math.ceil(math.ceil(K / k[2]) / splits) * k[2]
    # the partial sums are written and read back by a second kernel
    reduce = 0.0 if splits == 1 else (SPLITK_REDUCE_LAUNCH_S +
                                      (splits + 1) * M * N * 4 / (HBM_SUSTAINED_FRACTION * HBM_BYTES_PER_S))
    if points is None or not _finite(v, *points):
        return max(w * v * max(k_walk, 32) / PROFILE_K + reduce, hbm_floor)
    short, two, short_two = points
    first = max(_line(PROFILE_K_SHORT, short, PROFILE_K, v, k_walk), 0.25 * short)
    later = _line(PROFILE_K_SHORT, short_two - short, PROFILE_K, two - v, k_walk)
    mfma_round = 2.0 * NUM_CU * k[0] * k[1] * k_walk / (LATER_ROUND_MFMA_FRACTION * FP32_MFMA_FLOPS)
    later = min(max(later, mfma_round), first)
    operand_floor = 4.0 * tiles_m * k[0] * tiles_n * k[1] * K * (1 / k[0] + 1 / k[1]) / OPERAND_BYTES_PER_S
    cost = max(first + (w - 1) * later + reduce, hbm_floor, operand_floor)
    if k[2] == 32 and k[6] == 1 and w >= 2:
        cost *= 1.0 + BK32_MULTI_ROUND_COST
    return cost


def extra_points(prof_dict, k):
    """(short, two_rounds, short_two_rounds) of configuration k, or None when the profile lacks any of them."""
    try:
        return (prof_dict.short[k], prof_dict.two_rounds[k], prof_dict.short_two_rounds[k])
    except (AttributeError, KeyError):
        return None


def cost_model(prof_dict, M, N, K):
    min_cost = float("inf")
    best_config = (1, 1, 1, 1, 1, 1, 1, 1)
    for k, v in prof_dict.items():
        cost = config_cost(k, v, M, N, K, extra_points(prof_dict, k))
        if min_cost > cost:
            min_cost = cost
            best_config = k
    return best_config


# "Verified" selection: the cost model ranks, the device decides among the first few (the leading predictions lie
# within a per cent of each other for configurations that measure 5 - 10 % apart).
VERIFY_TOP = 12


def ranked_configs(prof_dict, M, N, K, top=VERIFY_TOP):
    """The `top` configurations with the lowest predicted cost, best first; cost_model returns the first of them."""
    ranked = sorted(prof_dict.items(), key=lambda kv: config_cost(kv[0], kv[1], M, N, K, extra_points(prof_dict, kv[0])))
    return [k for k, _ in ranked[:top]]


def run_config(k, M, N, K, warmup=10, iters=10, outer=1):
    """Seconds per launch (mean) on the real M, N, K (edges are predicated in the kernel; the reference
    pads M and N up to the tile instead, Ampere_FP32_gemm.py:103)."""
    lib = load(library_for_key(k))
    if k[2] == 0:
        if M > N:
            M, N = N, M
        K = math.ceil(K / 4) * 4
    _, avg, _ = lib.bench(M, N, K, warmup=warmup, iters=iters, outer=outer, rotate_bytes=0)
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
    return tuned_config("MI355X_FP32", ("gemm", M, N, K), prof_dict, lambda: cost_model(prof_dict, M, N, K),
                        lambda: verified_config(prof_dict, M, N, K))


def get_MI355X_FP32_gemm_Helix_result(prof_dict, M, N, K, backend="hip"):
    if backend != "hip":
        raise ValueError(f"backend {backend!r} is not available for MI355X_FP32 (only 'hip')")
    best_config = select_config(prof_dict, M, N, K)
    cost = run_config(best_config, M, N, K) * 1e3
    tflops = 2 * M * N * K / 1e9 / cost

    return cost, tflops


def get_MI355X_FP32_gemm_rocblas_result(M, N, K):
    """The vendor library (rocblas_sgemm) on the same problem and operand layouts, timed the same way.
    Mirrors get_Ampere_FP32_gemm_cublas_result (Ampere_FP32_gemm.py)."""
    lib = load(kernel_library("rocblas_f32"))
    _, avg, _ = lib.bench(M, N, K, warmup=10, iters=10, outer=1, rotate_bytes=0)
    cost = avg * 1e3
    return cost, 2 * M * N * K / 1e9 / cost


def get_MI355X_FP32_gemm_Verified_result(prof_dict, M, N, K, top=VERIFY_TOP):
    """The fastest of the cost model's first `top` configurations: each timed briefly, the winner timed again with
    the runner's launch counts.  Returns (cost_ms, tflops, key)."""
    best = verified_config(prof_dict, M, N, K, top)
    cost = run_config(best, M, N, K)
    return cost * 1e3, 2 * M * N * K / 1e12 / cost, best


def get_MI355X_FP32_gemm_Oracle_result(prof_dict, M, N, K):
    """Exhaustive per-shape search.  Returns (cost_ms, tflops, key)."""
    min_cost, best = float("inf"), None
    for k in prof_dict.keys():
        if k[2] == 0 and min(M, N) > 16:
            continue
        try:
            cost = run_config(k, M, N, K, warmup=2, iters=5)
        except Exception:
            continue
        if min_cost > cost:
            min_cost, best = cost, k
    return min_cost * 1e3, 2 * M * N * K / 1e12 / min_cost, best
