"""MI355X (gfx950 / CDNA4) datasheet constants used for every roofline fraction, in one place.

Source: AMD's public Instinct MI355X / CDNA4 datasheet (dense figures; the sparsity figures are twice
these and are never used).  The reference hard-codes its device model as the constant 108 (A100 SM
count) inside its cost models (scripts/Ampere_FP16/Ampere_FP16_gemm.py:425); the MI355X scripts take
theirs from here.
"""

NUM_CU = 256                  # compute units (8 XCDs x 32)
NUM_XCD = 8
CLOCK_GHZ = 2.4               # peak engine clock
LDS_BYTES_PER_CU = 160 * 1024
HBM_BYTES_PER_S = 8.0e12      # HBM3E
FP16_MFMA_FLOPS = 2516.6e12   # dense FP16 matrix
FP32_MFMA_FLOPS = 157.3e12    # FP32 matrix (== packed FP32 vector)
LAST_LEVEL_CACHE_BYTES = 256 * 1024 * 1024


def gemm_flops(M, N, K):
    return 2.0 * M * N * K


def gemm_bytes(M, N, K, elem_bytes):
    """Algorithmic traffic of one GEMM/GEMV: every operand element moved once."""
    return float(elem_bytes) * (M * K + N * K + M * N)


def conv_flops(batch, IC, H, W, OC, kH, kW, stride, pad):
    OH = (H + 2 * pad - kH) // stride + 1
    OW = (W + 2 * pad - kW) // stride + 1
    return 2.0 * batch * OH * OW * OC * IC * kH * kW


def conv_bytes(batch, IC, H, W, OC, kH, kW, stride, pad, elem_bytes):
    OH = (H + 2 * pad - kH) // stride + 1
    OW = (W + 2 * pad - kW) // stride + 1
    return float(elem_bytes) * (batch * H * W * IC + OC * kH * kW * IC + batch * OH * OW * OC)


def frac_of_mfma_peak(flops, seconds, fp32=False):
    return flops / seconds / (FP32_MFMA_FLOPS if fp32 else FP16_MFMA_FLOPS)


def frac_of_hbm_peak(nbytes, seconds):
    return nbytes / seconds / HBM_BYTES_PER_S
