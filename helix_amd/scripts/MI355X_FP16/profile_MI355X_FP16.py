"""Profile step of the MI355X_FP16 backend: time every compiled configuration once and store
{config-tuple: seconds} as a dict literal in build/prof_dict/MI355X_FP16_cost_model.dict.

Mirrors scripts/Ampere_FP16/profile_Ampere_FP16.py:17-62.  The reference times one lonely tile
(`gemm_... BLOCK_ROWS BLOCK_COLS 4096`, :36); a single workgroup on a 256-CU part sees neither HBM
nor L2 contention, so here every configuration is timed on one full round of tiles over the 256 compute
units (16 x 16 tiles): the cost model's `ceil(blocks / 256) * value` then has the reference's meaning
(rounds x time per round), and a one-round problem is predicted with its launch and pipeline-fill
latency included.  Every MFMA configuration is timed a second time at a short K (PROFILE_K_SHORT), stored in
a second dict file: the two points give the cost model a round's fixed part and its per-K part.
"""
import os
from tqdm import tqdm

from utils.helix_runtime import load, write_prof_dict, ProfDict, kernel_resources
from utils.roofline import NUM_CU
from MI355X_FP16.build_MI355X_FP16 import iter_configs, iter_splitk_configs, iter_dtl_configs, library_for_key

root_path = os.getcwd()

PROFILE_K = 4096            # reference: K = 4096 for every GEMM tile (profile_Ampere_FP16.py:36)
PROFILE_K_SHORT = 512       # second point: launch + pipeline fill + epilogue dominate at this K
PROFILE_ROUNDS = 1          # rounds of 256 tiles in the timed problem
PROFILE_GRID = 16           # 16 x 16 = 256 tiles = one tile per compute unit
# GEMV rows keep the reference's tag (first field 0, profile_Ampere_FP16.py:51,57) and its
# block_rows / block_cols reading of fields 1 and 2: one "block" = GEMV_BLOCK_ROWS activation rows times 128
# weight rows.  The reference has the single row (0, 1, 128, 0, 0, s); the activation-row tiles 4 and 16
# are added because the kernel's time is flat in M up to its tile, not linear.
GEMV_ROW_TILES = [1, 4, 16]
GEMV_KEYS = [(0, mt, 128, 0, 0, 0, 0) for mt in GEMV_ROW_TILES]
GEMV_SPLITK_KEYS = [(0, mt, 128, 0, 0, 1, 0) for mt in GEMV_ROW_TILES]
GEMV_KEY, GEMV_SPLITK_KEY = GEMV_KEYS[0], GEMV_SPLITK_KEYS[0]
GEMV_PROFILE_ROWS = 128 * NUM_CU   # one 128-row block per compute unit


def profile_problem(key, K=PROFILE_K):
    """(M, N, K) of the timed problem and the number of 256-tile rounds it holds."""
    if key[0] == 0:
        return key[1], GEMV_PROFILE_ROWS, K, 1
    return key[1] * PROFILE_GRID, key[2] * PROFILE_GRID * PROFILE_ROUNDS, K, PROFILE_ROUNDS


def time_config(key, warmup=3, iters=10, K=PROFILE_K):
    """Seconds for one round of 256 tiles of this configuration at this K (inf if it cannot run)."""
    M, N, K, rounds = profile_problem(key, K)
    try:
        lib = load(library_for_key(key))
        rotate = (1 << 30) if key[0] == 0 else 0
        _, avg, _ = lib.bench(M, N, K, warmup=warmup, iters=iters, outer=1, rotate_bytes=rotate)
    except Exception as e:  # missing library or a launch error: skip like profile_Ampere_FP32.py:41-45
        print(f"Skip config {key}: {e}")
        return float("inf")
    return avg / rounds


def gemm_kernel_scratch(key):
    """Scratch bytes per lane (register spills) of the GEMM kernel of configuration `key`, as recorded when its
    library was built; 0 when the build left no record."""
    for name, res in kernel_resources(library_for_key(key)).items():
        if "helix_gemm_f16_kernelILi0E" in name:
            return res.get("scratch", 0)
    return 0


def all_keys():
    keys = []
    for (K_STAGES, BLOCK_ROWS, BLOCK_COLS, WAVE_ROWS, WAVE_COLS, BLOCK_K) in iter_configs():
        key = (K_STAGES, BLOCK_ROWS, BLOCK_COLS, WAVE_ROWS, WAVE_COLS, 0, BLOCK_K)
        # the second staging set of a three-stage pipeline is admitted on a register estimate; a configuration
        # whose GEMM kernel spills all the same is left out of the profile (it is never the fastest)
        if K_STAGES > 2 and gemm_kernel_scratch(key) > 0:
            continue
        keys.append(key)
    for (K_STAGES, BLOCK_ROWS, BLOCK_COLS, WAVE_ROWS, WAVE_COLS, BLOCK_K) in iter_splitk_configs():
        keys.append((K_STAGES, BLOCK_ROWS, BLOCK_COLS, WAVE_ROWS, WAVE_COLS, 1, BLOCK_K))
    for (K_STAGES, BLOCK_ROWS, BLOCK_COLS, WAVE_ROWS, WAVE_COLS, BLOCK_K) in iter_dtl_configs():
        keys.append((K_STAGES, BLOCK_ROWS, BLOCK_COLS, WAVE_ROWS, WAVE_COLS, 0, BLOCK_K, 1))   # direct-to-LDS family
    keys.extend(GEMV_KEYS)
    keys.extend(GEMV_SPLITK_KEYS)
    return keys


def profile_Helix_MI355X_FP16_gemm_kernel():
    if not os.path.exists(f"{root_path}/build/prof_dict"):
        os.makedirs(f"{root_path}/build/prof_dict")

    prof_dict = ProfDict()
    print("Start profiling MI355X FP16 GEMM kernel ...")
    keys = all_keys()
    with tqdm(total=len(keys), desc="profiling") as pbar:
        for key in keys:
            prof_dict[key] = time_config(key)
            if key[0] != 0:
                prof_dict.short[key] = time_config(key, K=PROFILE_K_SHORT)
            pbar.update(1)

    write_prof_dict("MI355X_FP16", prof_dict)
    print("Profile finished.")
    return prof_dict


if __name__ == "__main__":

    profile_Helix_MI355X_FP16_gemm_kernel()
