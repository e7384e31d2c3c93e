"""Convolution runner of the MI355X_FP32 backend (implicit GEMM, NHWC, FP32).
Mirrors scripts/Ampere_FP32/Ampere_FP32_conv.py:89-110; one kernel instead of im2col + SGEMM when IC is
a multiple of 4 (the reference even borrows the FP16 im2col binary here, :107); otherwise the same entry
point pads the channels to a multiple of 4 in its workspace first (IC = 1: FP32 im2col + SGEMM)."""
import math
import os

from utils.helix_runtime import load, tuned_config, fastest_of
from MI355X_FP32.build_MI355X_FP32 import library_for_key, kernel_library
from MI355X_FP32.MI355X_FP32_gemm import config_cost, extra_points, VERIFY_TOP

root_path = os.getcwd()


def conv_config_cost(k, v, M, N, K, points=None):
    """The GEMM prediction as it is: with the gather offsets computed among the previous tile's MFMAs, a
    configuration's convolution time follows its GEMM time closely enough (22 layers, every configuration timed on
    each) that a separate copy term no longer improves the picks."""
    return config_cost(k, v, M, N, K, points)


GATHER_CHUNK = 4   # floats per 16-byte chunk of the implicit gather


def gather_channels(input_channel):
    """The channel count the kernel walks: a count off the gather chunk is padded to it in the workspace when
    that is at most 8/3 of the real one (helix_im2col::pads_channels), otherwise the column-buffer path runs
    on the real count."""
    padded = -(-input_channel // GATHER_CHUNK) * GATHER_CHUNK
    return padded if 3 * padded <= 8 * input_channel else input_channel


def cost_model(prof_dict, M, N, K, IC=None):
    """IC (the channel count the kernel walks) is accepted for symmetry with the FP16 backend; the FP32 gather
    decomposes the tap per chunk in every case, so no term depends on it."""
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


def ranked_configs(prof_dict, M, N, K, top=VERIFY_TOP):
    """The `top` SGEMM configurations with the lowest predicted cost, best first; cost_model returns the first."""
    cand = sorted((conv_config_cost(k, v, M, N, K, extra_points(prof_dict, k)), k) for k, v in prof_dict.items() if k[2] != 0)
    return [k for _, k in cand[:top]]


def verified_config(prof_dict, batch, input_channel, H, W, output_channel, kH, kW, stride, pad, top=VERIFY_TOP):
    """The fastest of the cost model's first `top` configurations on this layer (utils.helix_runtime.fastest_of:
    2 + 5 launches each, the leaders timed again)."""
    M = batch * ((H + 2 * pad - kH) // stride + 1) * ((W + 2 * pad - kW) // stride + 1)

    def time_config(k, warmup, iters):
        return load(library_for_key(k)).bench_conv(batch, input_channel, H, W, output_channel, kH, kW, stride, pad,
                                                   warmup=warmup, iters=iters)[1]

    return fastest_of(ranked_configs(prof_dict, M, output_channel, gather_channels(input_channel) * kH * kW, top),
                      time_config, "this layer")


def get_MI355X_FP32_conv_Verified_result(prof_dict, batch, input_channel, H, W, output_channel, kH, kW, stride, pad,
                                         top=VERIFY_TOP):
    """The fastest of the cost model's first `top` configurations on this layer: each timed briefly, the winner timed
    again with the runner's launch counts.  Returns (cost_ms, tflops, key)."""
    M = batch * ((H + 2 * pad - kH) // stride + 1) * ((W + 2 * pad - kW) // stride + 1)
    flops = 2.0 * M * output_channel * input_channel * kH * kW
    best = verified_config(prof_dict, batch, input_channel, H, W, output_channel, kH, kW, stride, pad, top)
    _, cost, _ = load(library_for_key(best)).bench_conv(batch, input_channel, H, W, output_channel, kH, kW, stride, pad,
                                                        warmup=10, iters=10)
    return cost * 1e3, flops / 1e12 / cost, best


def layer_cost_model(prof_dict, batch, input_channel, H, W, output_channel, kH, kW, stride, pad):
    """cost_model on the GEMM extents of a layer (Ampere_FP32_conv.py's mapping)."""
    M = batch * ((H + 2 * pad - kH) // stride + 1) * ((W + 2 * pad - kW) // stride + 1)
    return cost_model(prof_dict, M, output_channel, gather_channels(input_channel) * kH * kW)


def select_config(prof_dict, batch, input_channel, H, W, output_channel, kH, kW, stride, pad):
    """The configuration the runner launches for this layer: the cost model's ranking, settled on the device the first
    time the layer is met and remembered beside the profile (utils.helix_runtime.tuned_config); the cost model's
    first choice alone with HELIX_SELECTION=model."""
    layer = (batch, input_channel, H, W, output_channel, kH, kW, stride, pad)
    return tuned_config("MI355X_FP32", ("conv",) + layer, prof_dict,
                        lambda: layer_cost_model(prof_dict, *layer),
                        lambda: verified_config(prof_dict, *layer))


def get_MI355X_FP32_conv_Helix_result(prof_dict, batch, input_channel, H, W, output_channel, kH, kW, stride, pad,
                                      backend="hip"):
    if backend != "hip":
        raise ValueError(f"backend {backend!r} is not available for MI355X_FP32 (only 'hip')")
    M = batch * ((H + 2 * pad - kH) // stride + 1) * ((W + 2 * pad - kW) // stride + 1)
    N = output_channel
    K = input_channel * kH * kW
    best_config = select_config(prof_dict, batch, input_channel, H, W, output_channel, kH, kW, stride, pad)
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
