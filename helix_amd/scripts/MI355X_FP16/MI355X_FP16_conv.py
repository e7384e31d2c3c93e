"""Convolution runner of the MI355X_FP16 backend (implicit GEMM, NHWC).

Mirrors scripts/Ampere_FP16/Ampere_FP16_conv.py:420-446: the conv is mapped to GEMM extents
M = batch*OH*OW, N = OC, K = IC*kH*kW (:432-434), the GEMM cost model picks the configuration, and
the cost is measured.  The reference runs an im2col executable plus the GEMM executable and adds the
two times (:437-445); here the selected configuration's library gathers the A tile on the fly (one
kernel, one time) when IC is a multiple of 8, and runs im2col + weight repack + GEMM on one stream
inside the same entry point otherwise (one time for the three kernels).
"""
import math
import os

from utils.helix_runtime import load
from MI355X_FP16.build_MI355X_FP16 import library_for_key, kernel_library
from MI355X_FP16.MI355X_FP16_gemm import short_value, config_cost

root_path = os.getcwd()


# Every column of output tiles gathers the im2col rows of its row block again (index arithmetic per
# 16-byte chunk, which the plain GEMM the profile times does not have): measured over ResNet / GoogleNet /
# AlexNet layers, a configuration's conv time exceeds its GEMM prediction by about this fraction per tile
# column.
GATHER_COST_PER_TILE_COLUMN = 0.2


def conv_config_cost(k, v, M, N, K, v_short=None):
    return config_cost(k, v, M, N, K, v_short) * (1.0 + GATHER_COST_PER_TILE_COLUMN * math.ceil(N / k[2]))


def cost_model(prof_dict, M, N, K):
    """GEMM cost model restricted to the MFMA configurations (the GEMV kernels have no conv path), with the
    gather term above."""
    min_cost = float("inf")
    best_config = (1, 1, 1, 1, 1, 0, 32)
    for k, v in prof_dict.items():
        if k[0] == 0:
            continue
        cost = conv_config_cost(k, v, M, N, K, short_value(prof_dict, k))
        if min_cost > cost:
            min_cost = cost
            best_config = k
    return best_config


def get_MI355X_FP16_conv_Helix_result(prof_dict, batch, input_channel, H, W, output_channel, kH, kW, stride, pad,
                                      backend="hip"):
    if backend != "hip":
        raise ValueError(f"backend {backend!r} is not available for MI355X_FP16 (only 'hip')")
    M = batch * ((H + 2 * pad - kH) // stride + 1) * ((W + 2 * pad - kW) // stride + 1)
    N = output_channel
    K = input_channel * kH * kW
    best_config = cost_model(prof_dict, M, N, K)
    lib = load(library_for_key(best_config))
    _, avg, _ = lib.bench_conv(batch, input_channel, H, W, output_channel, kH, kW, stride, pad, warmup=10, iters=10)
    cost = avg * 1e3
    tflops = 2 * M * N * K / 1e9 / cost

    return cost, tflops


def get_MI355X_FP16_conv_miopen_result(batch, input_channel, H, W, output_channel, kH, kW, stride, pad):
    """The vendor library on the same problem and layouts (miopenConvolutionForward with the algorithm MIOpen's own
    search finds fastest), timed the same way.  Mirrors get_Ampere_FP16_conv_cudnn_result (Ampere_FP16_conv.py)."""
    M = batch * ((H + 2 * pad - kH) // stride + 1) * ((W + 2 * pad - kW) // stride + 1)
    N = output_channel
    K = input_channel * kH * kW
    lib = load(kernel_library("miopen_f16"))
    _, avg, _ = lib.bench_conv(batch, input_channel, H, W, output_channel, kH, kW, stride, pad, warmup=10, iters=10)
    cost = avg * 1e3
    return cost, 2 * M * N * K / 1e9 / cost
