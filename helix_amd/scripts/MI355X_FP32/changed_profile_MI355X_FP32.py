"""Cheap profile of the MI355X_FP32 backend: time the configurations whose workgroup tile equals the wave
tile and scale by the block-tile factors.  Mirrors scripts/Ampere_FP32/changed_profile_Ampere_FP32.py:16-48."""
import os
from tqdm import tqdm

from utils.helix_runtime import write_prof_dict
from MI355X_FP32.build_MI355X_FP32 import WAVE_TILE_LIST, BLOCK_SCALE_LIST, BK_LIST, is_valid_config, config_key, \
    iter_kgroup_configs
from MI355X_FP32.profile_MI355X_FP32 import time_config, GEMV_KEYS, GEMV_SPLITK_KEYS

root_path = os.getcwd()


def profile_Helix_MI355X_FP32_gemm_kernel():
    if not os.path.exists(f"{root_path}/build/prof_dict"):
        os.makedirs(f"{root_path}/build/prof_dict")

    prof_dict = {}
    print("Start profiling MI355X FP32 GEMM kernel ...")
    with tqdm(total=len(WAVE_TILE_LIST) ** 2 * len(BK_LIST) + 1, desc="profiling") as pbar:
        for WAVE_M in WAVE_TILE_LIST:
            for WAVE_N in WAVE_TILE_LIST:
                for BK in BK_LIST:
                    pbar.update(1)
                    if not is_valid_config(1, 1, WAVE_M, WAVE_N, BK, WAVE_M, WAVE_N):
                        continue
                    cost = time_config(config_key(WAVE_M, WAVE_N, BK, WAVE_M, WAVE_N))
                    for BMt in BLOCK_SCALE_LIST:
                        for BNt in BLOCK_SCALE_LIST:
                            BM, BN = BMt * WAVE_M, BNt * WAVE_N
                            if not is_valid_config(BMt, BNt, BM, BN, BK, WAVE_M, WAVE_N):
                                continue
                            prof_dict[config_key(BM, BN, BK, WAVE_M, WAVE_N)] = float(cost) * BMt * BNt
        # the few K-group configurations and the GEMV rows are timed one by one
        for key in [config_key(*cfg) for cfg in iter_kgroup_configs()] + GEMV_KEYS + GEMV_SPLITK_KEYS:
            prof_dict[key] = time_config(key)
        pbar.update(1)

    write_prof_dict("MI355X_FP32", prof_dict)
    print("Profile finished.")
    return prof_dict


if __name__ == "__main__":

    profile_Helix_MI355X_FP32_gemm_kernel()
