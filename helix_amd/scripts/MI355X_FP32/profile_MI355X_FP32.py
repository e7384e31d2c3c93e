"""Profile step of the MI355X_FP32 backend.  Mirrors scripts/Ampere_FP32/profile_Ampere_FP32.py:16-51
(one timing per configuration, K = 1024, failures recorded as inf, dict literal on disk).  As in the FP16
backend every configuration is timed on one full round of tiles over the 256 compute units rather than
on one lonely tile.  Three more points per MFMA configuration go to files of their own (one round at a short K,
two rounds at either K): the FP32 tiles are small enough for workgroups of consecutive rounds to share a
compute unit, which one round alone cannot show."""
import os
from tqdm import tqdm

from utils.helix_runtime import load, write_prof_dict, ProfDict
from utils.roofline import NUM_CU
from MI355X_FP32.build_MI355X_FP32 import iter_configs, iter_kgroup_configs, config_key, library_for_key

root_path = os.getcwd()

PROFILE_K = 1024            # reference: K = 1024 (profile_Ampere_FP32.py:39)
PROFILE_K_SHORT = 256
PROFILE_ROUNDS = 1
PROFILE_GRID = 16
GEMV_ROW_TILES = [1, 4, 16]
GEMV_KEYS = [(mt, 128, 0, 0, 0, 0, 4, 4) for mt in GEMV_ROW_TILES]
GEMV_SPLITK_KEYS = [(mt, 128, 0, 0, 0, 1, 4, 4) for mt in GEMV_ROW_TILES]
GEMV_PROFILE_ROWS = 128 * NUM_CU
GEMV_PROFILE_K = 4096


def profile_problem(key, K=PROFILE_K, rounds=PROFILE_ROUNDS):
    if key[2] == 0:
        return key[0], GEMV_PROFILE_ROWS, GEMV_PROFILE_K, 1
    return key[0] * PROFILE_GRID, key[1] * PROFILE_GRID * rounds, K, rounds


def time_config(key, warmup=3, iters=10, K=PROFILE_K, rounds=PROFILE_ROUNDS, per_round=True):
    """Seconds of `rounds` rounds of 256 tiles at this K, per round or (per_round=False) for the launch."""
    M, N, K, rounds = profile_problem(key, K, rounds)
    try:
        lib = load(library_for_key(key))
        rotate = (1 << 30) if key[2] == 0 else 0
        _, avg, _ = lib.bench(M, N, K, warmup=warmup, iters=iters, outer=1, rotate_bytes=rotate)
    except Exception as e:
        print(f"Skip config {key}: {e}")
        return float("inf")
    return avg / rounds if per_round else avg


def all_keys():
    keys = [config_key(*cfg) for cfg in iter_configs()] + [config_key(*cfg) for cfg in iter_kgroup_configs()]
    return keys + GEMV_KEYS + GEMV_SPLITK_KEYS


def profile_Helix_MI355X_FP32_gemm_kernel():
    if not os.path.exists(f"{root_path}/build/prof_dict"):
        os.makedirs(f"{root_path}/build/prof_dict")

    prof_dict = ProfDict()
    print("Start profiling MI355X FP32 GEMM kernel ...")
    keys = all_keys()
    with tqdm(total=len(keys), desc="profiling") as pbar:
        for key in keys:
            prof_dict[key] = time_config(key)
            if key[2] != 0:
                prof_dict.short[key] = time_config(key, K=PROFILE_K_SHORT)
                prof_dict.two_rounds[key] = time_config(key, rounds=2, per_round=False)
                prof_dict.short_two_rounds[key] = time_config(key, K=PROFILE_K_SHORT, rounds=2, per_round=False)
            pbar.update(1)

    write_prof_dict("MI355X_FP32", prof_dict)
    print("Profile finished.")
    return prof_dict


if __name__ == "__main__":

    profile_Helix_MI355X_FP32_gemm_kernel()
