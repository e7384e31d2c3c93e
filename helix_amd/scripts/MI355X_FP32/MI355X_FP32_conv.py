"""Convolution runner of the MI355X_FP32 backend (implicit GEMM, NHWC, FP32).
Mirrors scripts/Ampere_FP32/Ampere_FP32_conv.py:89-110; one kernel instead of im2col + SGEMM when IC is
a multiple of 4 (the reference even borrows the FP16 im2col binary here, :107), FP32 im2col + SGEMM
inside the same entry point otherwise."""
import math
import os

from utils.helix_runtime import load
from MI355X_FP32.build_MI355X_FP32 import library_for_key, kernel_library
from MI355X_FP32.MI355X_FP32_gemm import config_cost, extra_points

root_path = os.getcwd()


# In conv mode both operands arrive K-contiguous and every 16-byte chunk goes to LDS as four scalar writes; the
# BK / 4 lanes of one tile row write to the same banks, so the copy costs more the wider BK is.  Measured over
# ResNet / GoogleNet / AlexNet layers: a configuration's conv time exceeds its GEMM prediction by about this
# fraction at BK = 32 (half of it at 16, a quarter at 8).
CONV_COPY_COST_AT_BK32 = 0.2


def conv_config_cost(k, v, M, N, K, points=None):
    return config_cost(k, v, M, N, K, points) * (1.0 + CONV_COPY_COST_AT_BK32 * k[2] / 32)


def cost_model(prof_dict, M, N, K):
    min_cost = float("inf")
    best_config = (1, 1, 1, 1, 1, 1, 1, 1)
    for k, v in prof_dict.items():
        if k[2] == 0:
            continue
        cost = conv_config_cost(k, v, M, N, K, extra_points(prof_dict, k))
        if min_cost > cost:
            min_cost = cost
            best_config = k
    return best_config


def get_MI355X_FP32_conv_Helix_result(prof_dict, batch, input_channel, H, W, output_channel, kH, kW, stride, pad,
                                      backend="hip"):
    if backend != "hip":
        raise ValueError(f"backend {backend!r} is not available for MI355X_FP32 (only 'hip')")
    M = batch * ((H + 2 * pad - kH) // stride + 1) * ((W + 2 * pad - kW) // stride + 1)
    N = output_channel
    K = input_channel * kH * kW
    best_config = cost_model(prof_dict, M, N, K)
    lib = load(library_for_key(best_config))
    _, avg, _ = lib.bench_conv(batch, input_channel, H, W, output_channel, kH, kW, stride, pad, warmup=10, iters=10)
    cost = avg * 1e3
    tflops = 2 * M * N * K / 1e9 / cost

    return cost, tflops


def get_MI355X_FP32_conv_miopen_result(batch, input_channel, H, W, output_channel, kH, kW, stride, pad):
    """The vendor library on the same problem and layouts (miopenConvolutionForward with the algorithm MIOpen's own
    search finds fastest), timed the same way.  Mirrors get_Ampere_FP32_conv_cudnn_result (Ampere_FP32_conv.py)."""
    M = batch * ((H + 2 * pad - kH) // stride + 1) * ((W + 2 * pad - kW) // stride + 1)
    N = output_channel
    K = input_channel * kH * kW
    lib = load(kernel_library("miopen_f32"))
    _, avg, _ = lib.bench_conv(batch, input_channel, H, W, output_channel, kH, kW, stride, pad, warmup=10, iters=10)
    cost = avg * 1e3
    return cost, 2 * M * N * K / 1e9 / cost
