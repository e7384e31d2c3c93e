"""Build step of the MI355X_FP32 backend: instantiate the FP32 MFMA SGEMM template space and compile
every point with hipcc into its own shared library (plus the FP32 GEMV libraries).

Mirrors scripts/Ampere_FP32/build_Ampere_FP32.py (is_valid_config :7-12, compile_sgemm :17-28, the six
nested loops :43-50) with the same entry-point names modulo the backend tag.  The reference's
register-tile parameters (TM, TN, WARP_ROW_THREAD, COPY_A/B) describe a CUDA-core thread tile; the
MFMA template is parameterised by workgroup tile BM x BN, stage depth BK and wave tile WAVE_M x WAVE_N
instead.  Unlike the reference, which fires `os.popen(nvcc ...)` without waiting (:28), the build
returns only when every library exists, and it does build the FP32 GEMV (the reference never compiles
gemv_template_fp32.cu, :59-61).
"""
import os
from tqdm import tqdm

from utils.helix_runtime import SRC_ROOT, bin_dir, compile_many

root_path = os.getcwd()

WAVE_TILE_LIST = [32, 64, 128]
BLOCK_SCALE_LIST = [1, 2, 4]
BK_LIST = [8, 16, 32]
LDS_LIMIT = 160 * 1024
# K-group configurations: several waves per 32 x 32 wave tile, each multiplying a slice of every K tile.  An
# accumulator is a chain of K / 2 dependent MFMAs whatever the tile shape, so problems of few tiles and long K
# (transformer projections of a few hundred tokens, the last layers of a CNN) finish sooner with the chain cut
# inside the workgroup; deep K tiles keep enough bytes in flight for the few workgroups there are.
KGROUP_BLOCK_SCALES = [(1, 1), (1, 2), (2, 1), (2, 2)]
KGROUP_BK_KG_LIST = [(32, 2), (32, 4), (64, 2), (64, 4), (128, 8)]


def is_valid_config(BMt, BNt, BM, BN, BK=16, WAVE_M=64, WAVE_N=64, KG=1):
    # reference rules (build_Ampere_FP32.py:7-12): fewer than 512 threads' worth of tiles, tile extent bounds
    # (a full 1024-thread workgroup when the waves also divide K among themselves)
    if BMt * BNt * 64 * KG > (512 if KG == 1 else 1024):
        return False
    if BM > 256 or BN > 256 or BM < 32 or BN < 32:
        return False
    # gfx950 resources
    threads = 64 * BMt * BNt * KG
    if (BK // 2) % KG:                                             # whole MFMA k steps per wave group
        return False
    if (KG - 1) * BM * BN * 4 > LDS_LIMIT:                         # partial tiles of the groups, added through LDS
        return False
    if (BK * BM // 4) % threads or (BK * BN // 4) % threads:       # GEMM tile copy, 16-byte chunks along M / N
        return False
    if (BM * BK // 4) % threads or (BN * BK // 4) % threads:       # conv tile copy, 16-byte chunks along K
        return False
    conv_pad = 32 + max(64 // BK, 1)  # LDS row padding of the convolution mode, the wider of the two
    if 2 * BK * (BM + conv_pad + BN + conv_pad) * 4 > LDS_LIMIT:
        return False
    if WAVE_M * WAVE_N // 64 > 256:
        return False
    return True


def iter_configs():
    """Yields (BM, BN, BK, WAVE_M, WAVE_N) in build order."""
    for WAVE_M in WAVE_TILE_LIST:
        for WAVE_N in WAVE_TILE_LIST:
            for BK in BK_LIST:
                for BMt in BLOCK_SCALE_LIST:
                    for BNt in BLOCK_SCALE_LIST:
                        BM = BMt * WAVE_M
                        BN = BNt * WAVE_N
                        if not is_valid_config(BMt, BNt, BM, BN, BK, WAVE_M, WAVE_N):
                            continue
                        yield (BM, BN, BK, WAVE_M, WAVE_N)


def iter_kgroup_configs():
    """Yields (BM, BN, BK, WAVE_M, WAVE_N, K_GROUPS) of the K-group configurations in build order."""
    WAVE_M = WAVE_N = 32
    for (BK, KG) in KGROUP_BK_KG_LIST:
        for (BMt, BNt) in KGROUP_BLOCK_SCALES:
            BM, BN = BMt * WAVE_M, BNt * WAVE_N
            if is_valid_config(BMt, BNt, BM, BN, BK, WAVE_M, WAVE_N, KG):
                yield (BM, BN, BK, WAVE_M, WAVE_N, KG)


def sgemm_library(BM, BN, BK, WAVE_M, WAVE_N, KG=1):
    suffix = "" if KG == 1 else f"_kg{KG}"
    return f"{bin_dir('fp32')}/libsgemm_{BM}_{BN}_{BK}_{WAVE_M}_{WAVE_N}{suffix}.so"


def kernel_library(kernel_name):
    return f"{bin_dir('fp32')}/lib{kernel_name}.so"


def default_library():
    """A mid-sized configuration used by smoke checks."""
    return sgemm_library(128, 128, 16, 64, 64)


def library_for_key(key):
    """prof-dict key -> library.  key = (BM, BN, BK, WAVE_M, WAVE_N, LDS_STAGES, K_GROUPS, COPY_VEC) keeps the
    reference's eight fields with BM, BN, BK in the same places (profile_Ampere_FP32.py:46); BK == 0 marks
    the GEMV rows, whose first two fields are the activation-row tile and 128 weight rows."""
    if key[2] == 0:
        return kernel_library("gemv_fp32" if key[5] == 0 else "gemv_fp32_splitK")
    return sgemm_library(key[0], key[1], key[2], key[3], key[4], key[6])


def config_key(BM, BN, BK, WAVE_M, WAVE_N, KG=1):
    return (BM, BN, BK, WAVE_M, WAVE_N, 2, KG, 4)


def compile_sgemm(BM, BN, BK, WAVE_M, WAVE_N, KG=1):
    defines = {"BM": BM, "BN": BN, "BK": BK, "WAVE_M": WAVE_M, "WAVE_N": WAVE_N}
    if KG != 1:
        defines["K_GROUPS"] = KG
    return (f"{SRC_ROOT}/MI355X_FP32/sgemm.hip", sgemm_library(BM, BN, BK, WAVE_M, WAVE_N, KG), defines)


def compile_kernel(kernel_name):
    defines = {}
    src_name = kernel_name
    if kernel_name == "gemv_fp32_splitK":
        src_name = "gemv_fp32"
        defines["SPLIT_K"] = 4
    return (f"{SRC_ROOT}/MI355X_FP32/{src_name}.hip", kernel_library(kernel_name), defines)


def build_jobs():
    jobs = [compile_sgemm(*cfg) for cfg in iter_configs()]
    jobs += [compile_sgemm(*cfg) for cfg in iter_kgroup_configs()]
    jobs.append(compile_kernel("gemv_fp32"))
    jobs.append(compile_kernel("gemv_fp32_splitK"))
    jobs.append(rocblas_job())
    jobs.append(miopen_job())
    return jobs


def rocblas_job():
    """The vendor comparator, like the reference's cublas_f32 (build_Ampere_FP32.py:59-61)."""
    return (f"{SRC_ROOT}/MI355X_FP32/rocblas_f32.hip", kernel_library("rocblas_f32"), {}, "-lrocblas")


def miopen_job():
    """The vendor convolution comparator, like the reference's cudnn_fp32 (build_Ampere_FP32.py)."""
    return (f"{SRC_ROOT}/MI355X_FP32/miopen_f32.hip", kernel_library("miopen_f32"), {}, "-lMIOpen")


def build_Helix_MI355X_FP32_gemm_kernel():
    if not os.path.exists(f"{root_path}/build/bin_fp32"):
        os.makedirs(f"{root_path}/build/bin_fp32")

    print("Start building MI355X FP32 GEMM kernel ...")
    jobs = build_jobs()
    with tqdm(total=len(jobs), desc="building") as pbar:
        failed = compile_many(jobs, progress=pbar)
    for out, err in failed:
        print(f"Build failed: {out}\n{err}")
    print("Build finished.")
    return failed


if __name__ == "__main__":

    build_Helix_MI355X_FP32_gemm_kernel()
