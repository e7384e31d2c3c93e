"""Cheap profile of the MI355X_FP16 backend: time only the configurations whose workgroup tile
equals the wave tile and scale the result to the larger block tiles.

Mirrors scripts/Ampere_FP16/changed_profile_Ampere_FP16.py:17-70, where the time of the 1x1-scale
tile is multiplied by BLOCK_ROWS_SCALE * BLOCK_COLS_SCALE (:41).
"""
import os
from tqdm import tqdm

from utils.helix_runtime import write_prof_dict, ProfDict
from MI355X_FP16.build_MI355X_FP16 import (K_STAGES_LIST, WAVE_TILE_LIST, WAVE_COLS_LIST, BLOCK_SCALE_LIST, BLOCK_K_LIST,
                                           is_valid_config, SPLITK_STAGES_LIST)
from MI355X_FP16.profile_MI355X_FP16 import time_config, GEMV_KEYS, GEMV_SPLITK_KEYS, PROFILE_K_SHORT

root_path = os.getcwd()


def profile_Helix_MI355X_FP16_gemm_kernel():
    if not os.path.exists(f"{root_path}/build/prof_dict"):
        os.makedirs(f"{root_path}/build/prof_dict")

    prof_dict = ProfDict()
    print("Start profiling MI355X FP16 GEMM kernel ...")
    total = len(K_STAGES_LIST) * len(WAVE_TILE_LIST) * len(WAVE_COLS_LIST) * len(BLOCK_K_LIST) * 2 + 2
    with tqdm(total=total, desc="profiling") as pbar:
        for K_STAGES in K_STAGES_LIST:
            for WAVE_ROWS in WAVE_TILE_LIST:
                for WAVE_COLS in WAVE_COLS_LIST:
                    for BLOCK_K in BLOCK_K_LIST:
                        for splitK in (0, 1):
                            pbar.update(1)
                            if splitK == 1 and K_STAGES not in SPLITK_STAGES_LIST:
                                continue
                            if not is_valid_config(1, 1, WAVE_ROWS, WAVE_COLS, WAVE_ROWS, WAVE_COLS, BLOCK_K, K_STAGES,
                                                   splitK):
                                continue
                            base_key = (K_STAGES, WAVE_ROWS, WAVE_COLS, WAVE_ROWS, WAVE_COLS, splitK, BLOCK_K)
                            cost = time_config(base_key)
                            cost_short = time_config(base_key, K=PROFILE_K_SHORT)
                            for BLOCK_ROWS_SCALE in BLOCK_SCALE_LIST:
                                for BLOCK_COLS_SCALE in BLOCK_SCALE_LIST:
                                    BLOCK_ROWS = BLOCK_ROWS_SCALE * WAVE_ROWS
                                    BLOCK_COLS = BLOCK_COLS_SCALE * WAVE_COLS
                                    if not is_valid_config(BLOCK_ROWS_SCALE, BLOCK_COLS_SCALE, BLOCK_ROWS, BLOCK_COLS,
                                                           WAVE_ROWS, WAVE_COLS, BLOCK_K, K_STAGES, splitK):
                                        continue
                                    key = (K_STAGES, BLOCK_ROWS, BLOCK_COLS, WAVE_ROWS, WAVE_COLS, splitK, BLOCK_K)
                                    prof_dict[key] = float(cost) * BLOCK_ROWS_SCALE * BLOCK_COLS_SCALE
                                    prof_dict.short[key] = float(cost_short) * BLOCK_ROWS_SCALE * BLOCK_COLS_SCALE

        for key in GEMV_KEYS + GEMV_SPLITK_KEYS:
            prof_dict[key] = time_config(key)
        pbar.update(2)

    write_prof_dict("MI355X_FP16", prof_dict)
    print("Profile finished.")
    return prof_dict


if __name__ == "__main__":

    profile_Helix_MI355X_FP16_gemm_kernel()
