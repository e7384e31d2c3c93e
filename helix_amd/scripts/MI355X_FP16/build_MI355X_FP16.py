"""Build step of the MI355X_FP16 backend: instantiate the tile / wave / LDS parameter space of the
FP16 templates and compile every point with hipcc into its own shared library.

Mirrors scripts/Ampere_FP16/build_Ampere_FP16.py (compile_kernel :7-28, is_valid_config :30-39, the
five nested loops :47-53, the fixed kernels gemv / gemv_splitK :62-65) with the same entry-point
names modulo the backend tag.  Differences that follow from the target:
  * output is build/bin_fp16/lib<kernel>_<params>.so exporting the C ABI of include/helix_abi.h instead of
    an executable; the convolution path lives in the same library as the GEMM of each configuration
    (implicit GEMM), so there is no im2col artifact;
  * wave tiles are multiples of 32 rows x 16 columns of the 16x16x32 MFMA tile, K_STAGE becomes K_STAGES (the
    pipeline holds the K tile being multiplied in LDS and K_STAGES - 1 more on their way through staging
    registers: 2, and 3 for the tiles whose registers allow a second staging set), and BLOCK_K is a template
    parameter too (it is fixed to 32 in the reference, gemm.cu:77);
  * the deeper pipelines of the reference (K_STAGE 3 .. 5 are rings of cp.async stages, gemm.cu:156-198) are the
    direct-to-LDS family, src_template/MI355X_FP16/gemm_dtl.hip: eight-wave tiles whose K tiles go from global
    memory straight into a ring of K_STAGES LDS stages of BLOCK_K columns.  Its prof-dict keys carry a
    trailing eighth field 1 (DIRECT_TO_LDS); keys of the other families keep seven fields;
  * the space is pruned by measurement (keeps_up): points that were never within reach of the fastest configuration
    on a table of 162 problems are not built;
  * compiles run in parallel worker threads instead of one os.system at a time.
"""
import os
from tqdm import tqdm

from utils.helix_runtime import SRC_ROOT, bin_dir, compile_many

root_path = os.getcwd()

K_STAGES_LIST = [2, 3]
SPLITK_MAX = 8              # a split-K library partitions K 2 .. 8 ways, chosen per problem
SPLITK_STAGES_LIST = [2]    # pipeline depths a split-K variant is built for
WAVE_TILE_LIST = [32, 64, 128]              # wave-tile rows (the epilogue pairs 16-row MFMA tiles)
# wave-tile columns: 48 and 96 give block tiles of 96 and 192 columns, which divide the 768 / 2304 / 3072-wide
# transformer projections into whole rounds of 256 tiles where the powers of two leave a quarter of the
# compute units idle
WAVE_COLS_LIST = [32, 48, 64, 96, 128]
BLOCK_SCALE_LIST = [1, 2, 4]
BLOCK_K_LIST = [64, 128]
# direct-to-LDS family: (BLOCK_K, K_STAGES) points.  The template also builds rings of three or four 32-column stages
# and three 64-column ones; measured over the shape table below they are never ahead, so the 256 x 256 tile with two
# 64-column stages (the one LDS holds twice, and the family's only winner: 8192^3 and 4096^3 on some boxes) is what
# the build keeps
DTL_BK_STAGES_LIST = [(64, 2)]
DTL_BLOCK_SCALES = [(2, 4), (4, 2)]     # eight waves: two per SIMD
DTL_TILE = (256, 256)
LDS_LIMIT = 160 * 1024
VGPR_FILE = 512             # registers per lane of one SIMD (arch + accumulation), shared by its resident waves


STAGES3_VGPR_MARGIN = 56     # three stages, two waves per SIMD: registers the compiler needs beyond the estimate
STAGES3_NONACC_LIMIT = 200    # three stages, one wave per SIMD: fragments + staging + addresses in the architectural half

def vgpr_estimate(block_rows, block_cols, wave_rows, wave_cols, block_k, k_stages=2):
    """Registers per lane the kernel keeps live in its main loop: FP32 accumulators, the double-buffered
    fragments of the operand with more 16-row fragments, the 4-deep window of the other one, the staging
    registers of K_STAGES - 1 K tiles, and about 16 for addresses."""
    threads = 64 * (block_rows // wave_rows) * (block_cols // wave_cols)
    tm, tn = wave_rows // 16, wave_cols // 16
    acc = wave_rows * wave_cols // 64
    frags = 2 * max(tm, tn) * 4 + 4 * 4
    staging = (block_rows + block_cols) * (block_k // 8) // threads * 4 * (k_stages - 1)
    return acc + frags + staging + 16


# ---- measured pruning -------------------------------------------------------------------------------------------
# Every point that fits the hardware (fits_hardware: 159 two-stage points, each with a split-K twin, 86 three-stage
# points, 68 direct-to-LDS points) was built once and timed on a table of 140 GEMM shapes (squares, BERT, LLM token
# sweeps, DeepBench, GNN, CNN fully-connected layers) and 22 convolution layers.  173 of the 472 were within 5 % of
# the fastest configuration on at least one problem; the rules below keep 251 and lose, against the fastest of all
# 472, 0.07 % in the geometric mean over the table, 3.9 % on its worst shape and under 2 % on every other:
#   * split-K pays on small wave tiles only (few tiles, long K): wave tiles of up to 32 x 64;
#   * a second staging set (three stages) never won with 128-row wave tiles;
#   * among the two-stage tiles, workgroups of two waves were never ahead of the one- and four-wave tiles around them;
#   * direct-to-LDS: see DTL_BK_STAGES_LIST.
# Building them takes half the time of the full space.
SPLITK_MAX_WAVE_TILE = 32 * 64
STAGES3_MAX_WAVE_ROWS = 64


def keeps_up(block_rows_scale, block_cols_scale, wave_rows, wave_cols, k_stages=2, split_k=0):
    """False for the points the measured table showed never to be within reach of the fastest configuration."""
    if split_k:
        return wave_rows * wave_cols <= SPLITK_MAX_WAVE_TILE
    if k_stages == 3:
        return wave_rows <= STAGES3_MAX_WAVE_ROWS
    return block_rows_scale * block_cols_scale != 2


def is_valid_config(block_rows_scale, block_cols_scale, block_rows, block_cols, wave_rows, wave_cols,
                    block_k=64, k_stages=2, split_k=0):
    """A point of the template space that is built: it fits the hardware and the measured pruning keeps it."""
    return (fits_hardware(block_rows_scale, block_cols_scale, block_rows, block_cols, wave_rows, wave_cols, block_k,
                          k_stages)
            and keeps_up(block_rows_scale, block_cols_scale, wave_rows, wave_cols, k_stages, split_k))


def fits_hardware(block_rows_scale, block_cols_scale, block_rows, block_cols, wave_rows, wave_cols,
                  block_k=64, k_stages=2):
    # the reference's four rules (build_Ampere_FP16.py:30-39)
    if block_rows_scale == 4 and block_cols_scale == 4:
        return False
    if block_rows > 256 or block_cols > 256:
        return False
    if wave_cols == wave_rows * 8 or wave_rows == wave_cols * 8:
        return False
    if block_cols == block_rows * 16 or block_rows == block_cols * 16:
        return False
    # gfx950 resources: two LDS stages, even split of the tile copy over threads, registers
    if k_stages not in (2, 3):
        return False
    if 2 * (block_rows + block_cols) * block_k * 2 > LDS_LIMIT:
        return False
    threads = 64 * block_rows_scale * block_cols_scale
    chunks_per_row = block_k // 8
    if (block_rows * chunks_per_row) % threads or (block_cols * chunks_per_row) % threads:
        return False
    if threads % chunks_per_row:
        return False
    # the streamed operand's fragments of a K tile go through a window of 2 * min(fragments, 2) registers
    tm, tn = wave_rows // 16, wave_cols // 16
    streamed = tn if tm > tn else tm
    if ((block_k // 32) * streamed) % (2 * min(streamed, 2)):
        return False
    waves_per_simd = (threads // 64 + 3) // 4
    estimate = vgpr_estimate(block_rows, block_cols, wave_rows, wave_cols, block_k, k_stages)
    if k_stages == 2:
        return estimate <= VGPR_FILE // waves_per_simd
    # Three stages: the loop is unrolled over both staging sets and the compiler needs more than the estimate.  With
    # one wave per SIMD the accumulators can live in the accumulation half of the file, but everything else has
    # to fit the architectural half; with two waves per SIMD everything shares 256 registers.  (The limits are what
    # separates the configurations that compile without scratch from those that spill.)
    if waves_per_simd == 1:
        return estimate - wave_rows * wave_cols // 64 <= STAGES3_NONACC_LIMIT
    return estimate + STAGES3_VGPR_MARGIN <= VGPR_FILE // waves_per_simd


def iter_configs(split_k=0):
    """Yields (K_STAGES, BLOCK_ROWS, BLOCK_COLS, WAVE_ROWS, WAVE_COLS, BLOCK_K) in build order: the plain tile
    libraries, or with split_k=1 the points a split-K library is built for."""
    for K_STAGES in (SPLITK_STAGES_LIST if split_k else K_STAGES_LIST):
        for WAVE_ROWS in WAVE_TILE_LIST:
            for WAVE_COLS in WAVE_COLS_LIST:
                for BLOCK_ROWS_SCALE in BLOCK_SCALE_LIST:
                    for BLOCK_COLS_SCALE in BLOCK_SCALE_LIST:
                        for BLOCK_K in BLOCK_K_LIST:
                            BLOCK_ROWS = BLOCK_ROWS_SCALE * WAVE_ROWS
                            BLOCK_COLS = BLOCK_COLS_SCALE * WAVE_COLS
                            if not is_valid_config(BLOCK_ROWS_SCALE, BLOCK_COLS_SCALE, BLOCK_ROWS, BLOCK_COLS,
                                                   WAVE_ROWS, WAVE_COLS, BLOCK_K, K_STAGES, split_k):
                                continue
                            yield (K_STAGES, BLOCK_ROWS, BLOCK_COLS, WAVE_ROWS, WAVE_COLS, BLOCK_K)


def iter_splitk_configs():
    return iter_configs(split_k=1)


def is_valid_dtl_config(block_rows_scale, block_cols_scale, block_rows, block_cols, wave_rows, wave_cols, block_k,
                        k_stages):
    """Validity of a point of the direct-to-LDS family (the static_asserts of gemm_dtl.hip)."""
    # the reference's tile rules (build_Ampere_FP16.py:30-39)
    if block_rows > 256 or block_cols > 256:
        return False
    if wave_cols == wave_rows * 8 or wave_rows == wave_cols * 8:
        return False
    if block_cols == block_rows * 16 or block_rows == block_cols * 16:
        return False
    if block_rows_scale * block_cols_scale != 8:
        return False
    if (block_rows, block_cols) != DTL_TILE:     # the one tile of the family that the measured table keeps
        return False
    # each of the four copying waves fills whole 1 KiB pieces of a stage: 16 / 8 / 4 matrix rows per instruction
    rows_per_copy = {32: 16, 64: 8, 128: 4}[block_k]
    if (block_rows // 4) % rows_per_copy or (block_cols // 4) % rows_per_copy:
        return False
    copies = (block_rows // 4 + block_cols // 4) // rows_per_copy
    if (k_stages - 2) * copies > 63:
        return False
    strips = 8 * 32 * (wave_cols * 2 + 16)
    if max(k_stages * (block_rows + block_cols) * block_k * 2, strips) + 64 > LDS_LIMIT:
        return False
    # accumulators plus a whole K tile of fragments in the 256 registers of a wave
    tm, tn = wave_rows // 16, wave_cols // 16
    if (block_k // 32) * (tm + tn) * 4 + tm * tn * 4 > 236:
        return False
    return True


def iter_dtl_configs():
    """Yields (K_STAGES, BLOCK_ROWS, BLOCK_COLS, WAVE_ROWS, WAVE_COLS, BLOCK_K) of the direct-to-LDS family."""
    for (BLOCK_K, K_STAGES) in DTL_BK_STAGES_LIST:
        for WAVE_ROWS in WAVE_TILE_LIST:
            for WAVE_COLS in WAVE_COLS_LIST:
                for (BLOCK_ROWS_SCALE, BLOCK_COLS_SCALE) in DTL_BLOCK_SCALES:
                    BLOCK_ROWS = BLOCK_ROWS_SCALE * WAVE_ROWS
                    BLOCK_COLS = BLOCK_COLS_SCALE * WAVE_COLS
                    if is_valid_dtl_config(BLOCK_ROWS_SCALE, BLOCK_COLS_SCALE, BLOCK_ROWS, BLOCK_COLS, WAVE_ROWS,
                                           WAVE_COLS, BLOCK_K, K_STAGES):
                        yield (K_STAGES, BLOCK_ROWS, BLOCK_COLS, WAVE_ROWS, WAVE_COLS, BLOCK_K)


def is_dtl_key(key):
    """Keys of the direct-to-LDS family carry a trailing eighth field 1."""
    return len(key) > 7 and key[7] == 1


def kernel_library(kernel_name, k_stages=None, block_rows=None, block_cols=None, wave_rows=None, wave_cols=None,
                   block_k=None):
    """Path of the shared library of one configuration (same naming scheme as the reference's
    executables, build_Ampere_FP16.py:13-27, plus the BLOCK_K field)."""
    output_name = kernel_name
    for v in (k_stages, block_rows, block_cols, wave_rows, wave_cols, block_k):
        if v is not None:
            output_name += f"_{v}"
    return f"{bin_dir('fp16')}/lib{output_name}.so"


def library_for_key(key):
    """prof-dict key -> library path.  key = (K_STAGES, BLOCK_ROWS, BLOCK_COLS, WAVE_ROWS, WAVE_COLS,
    splitK flag, BLOCK_K); key[0] == 0 marks the GEMV kernels, as in the reference
    (scripts/Ampere_FP16/Ampere_FP16_gemm.py:435)."""
    if key[0] == 0:
        return kernel_library("gemv" if key[5] == 0 else "gemv_splitK")
    if is_dtl_key(key):
        return kernel_library("gemm_dtl", key[0], key[1], key[2], key[3], key[4], key[6])
    return kernel_library("gemm" if key[5] == 0 else "gemm_splitK", key[0], key[1], key[2], key[3], key[4], key[6])


def compile_job(kernel_name, k_stages=None, block_rows=None, block_cols=None, wave_rows=None, wave_cols=None,
                block_k=None):
    defines = {}
    src_name = kernel_name
    if kernel_name == "gemm_splitK":
        src_name = "gemm"
        defines["SPLIT_K"] = SPLITK_MAX
    elif kernel_name == "gemv_splitK":
        src_name = "gemv"
        defines["SPLIT_K"] = 4
    elif kernel_name == "gemv_nomfma":
        # the wave-reduction kernel for every batch up to 16 rows (no MFMA at all): the number the MFMA variant of
        # 9 .. 16 rows is reported against
        src_name = "gemv"
        defines["MFMA_MIN_M"] = 17
    if k_stages is not None:
        defines["K_STAGES"] = k_stages
    if block_rows is not None:
        defines["BLOCK_ROWS"] = block_rows
    if block_cols is not None:
        defines["BLOCK_COLS"] = block_cols
    if wave_rows is not None:
        defines["WAVE_ROWS"] = wave_rows
    if wave_cols is not None:
        defines["WAVE_COLS"] = wave_cols
    if block_k is not None:
        defines["BLOCK_K"] = block_k
    src = f"{SRC_ROOT}/MI355X_FP16/{src_name}.hip"
    out = kernel_library(kernel_name, k_stages, block_rows, block_cols, wave_rows, wave_cols, block_k)
    return (src, out, defines)


def build_jobs():
    jobs = []
    for cfg in iter_configs():
        jobs.append(compile_job("gemm", *cfg))
    for cfg in iter_splitk_configs():
        jobs.append(compile_job("gemm_splitK", *cfg))
    for cfg in iter_dtl_configs():
        jobs.append(compile_job("gemm_dtl", *cfg))
    jobs.append(compile_job("gemv"))
    jobs.append(compile_job("gemv_splitK"))
    jobs.append(compile_job("gemv_nomfma"))
    jobs.append(rocblas_job())
    jobs.append(miopen_job())
    return jobs


def rocblas_job():
    """The vendor comparator, like the reference's `compile_kernel("cublas_f16")` (build_Ampere_FP16.py:72-76)."""
    return (f"{SRC_ROOT}/MI355X_FP16/rocblas_f16.hip", kernel_library("rocblas_f16"), {}, "-lrocblas")


def miopen_job():
    """The vendor convolution comparator, like the reference's `compile_kernel("cudnn_fp16")`
    (build_Ampere_FP16.py)."""
    return (f"{SRC_ROOT}/MI355X_FP16/miopen_f16.hip", kernel_library("miopen_f16"), {}, "-lMIOpen")


def build_rocblas_FP16_gemm_kernel():
    print("Start building rocBLAS FP16 GEMM comparator ...")
    failed = compile_many([rocblas_job()])
    for out, err in failed:
        print(f"Build failed: {out}\n{err}")
    print("Build finished.")
    return failed


def build_Helix_MI355X_FP16_gemm_kernel():
    if not os.path.exists(f"{root_path}/build/bin_fp16"):
        os.makedirs(f"{root_path}/build/bin_fp16")

    print("Start building MI355X FP16 GEMM kernel ...")
    jobs = build_jobs()
    with tqdm(total=len(jobs), desc="building") as pbar:
        failed = compile_many(jobs, progress=pbar)
    for out, err in failed:
        print(f"Build failed: {out}\n{err}")
    print("Build finished.")
    return failed


if __name__ == "__main__":

    build_Helix_MI355X_FP16_gemm_kernel()
