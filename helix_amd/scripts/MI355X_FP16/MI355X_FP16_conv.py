"""Convolution runner of the MI355X_FP16 backend (implicit GEMM, NHWC).

Mirrors scripts/Ampere_FP16/Ampere_FP16_conv.py:420-446: the conv is mapped to GEMM extents
M = batch*OH*OW, N = OC, K = IC*kH*kW (:432-434), the GEMM cost model picks the configuration, and
the cost is measured.  The reference runs an im2col executable plus the GEMM executable and adds the
two times (:437-445); here the selected configuration's library gathers the A tile on the fly (one
kernel, one time) when IC is a multiple of 8 (a 1 x 1 filter with stride 1 and no padding gathers nothing and runs
as the plain GEMM on the activations as they lie); otherwise the same entry point first pads the channels of
activations and weights to a multiple of 8 in its workspace (or, for IC = 1 and 2, runs im2col + weight
repack + GEMM), all on one stream and timed as one.
"""
import math
import os

from utils.helix_runtime import load, kernel_resources, tuned_config, fastest_of
from MI355X_FP16.build_MI355X_FP16 import library_for_key, kernel_library, is_dtl_key
from MI355X_FP16.MI355X_FP16_gemm import short_value, config_cost, VERIFY_TOP

root_path = os.getcwd()


# Every column of output tiles gathers the im2col rows of its row block again (index arithmetic per
# 16-byte chunk, which the plain GEMM the profile times does not have): measured over ResNet / GoogleNet /
# AlexNet layers, a configuration's conv time exceeds its GEMM prediction by about this fraction per tile
# column.
GATHER_COST_PER_TILE_COLUMN = 0.2
# A K tile that spans several filter taps (IC not a multiple of BLOCK_K: first layers after channel padding,
# 16- and 24-channel inputs) decomposes the tap per 16-byte chunk instead of once per tile; measured over such
# layers the time grows by about these fractions per 64 of BLOCK_K and per 128 tile rows.
GENERAL_GATHER_COST_PER_64_K = 0.3
GENERAL_GATHER_COST_PER_128_ROWS = 0.2


# A layer of few K tiles (1x1 layers, first layers) is mostly first loads and result stores around a short multiply.
# Workgroups that share a compute unit overlap those phases, a workgroup that fills the unit alone runs them one
# after the other: over such layers the measured time follows 1 + this / (workgroups resident per compute unit),
# and the gather term per tile column is half as large.
SHORT_K_TILES = 8
SHORT_K_ALONE_COST = 0.6
SHORT_K_GATHER_COST_PER_TILE_COLUMN = 0.1
LDS_BYTES_PER_CU = 160 * 1024
WAVES_PER_CU = 16


def resident_workgroups(k):
    """Workgroups of configuration k that fit one compute unit: two LDS stages of (rows + columns) x BLOCK_K halves
    each, at most 16 waves, at most 8 workgroups."""
    lds = 2 * (k[1] + k[2]) * k[6] * 2
    waves = (k[1] // k[3]) * (k[2] // k[4])
    return max(1, min(LDS_BYTES_PER_CU // lds, WAVES_PER_CU // waves, 8))


def is_pointwise(kH, kW, stride, pad):
    """A 1 x 1 filter walked pixel by pixel: the library runs such a layer as the plain GEMM on the activations as they
    lie (gemm.hip, conv2d), so no gather term applies and no gather kernel's registers matter."""
    return kH == 1 and kW == 1 and stride == 1 and pad == 0


def conv_config_cost(k, v, M, N, K, v_short=None, IC=None, pointwise=False):
    if pointwise:
        return config_cost(k, v, M, N, K, v_short)
    short = math.ceil(K / k[6]) <= SHORT_K_TILES
    per_column = SHORT_K_GATHER_COST_PER_TILE_COLUMN if short else GATHER_COST_PER_TILE_COLUMN
    cost = config_cost(k, v, M, N, K, v_short) * (1.0 + per_column * math.ceil(N / k[2]))
    if short:
        cost *= 1.0 + SHORT_K_ALONE_COST / resident_workgroups(k)
    if IC is not None and IC % k[6]:
        cost *= (1.0 + GENERAL_GATHER_COST_PER_64_K * k[6] / 64) * (1.0 + GENERAL_GATHER_COST_PER_128_ROWS * k[1] / 128)
    return cost


GATHER_CHUNK = 8   # halves per 16-byte chunk of the implicit gather


def gather_channels(input_channel):
    """The channel count the kernel walks: a count off the gather chunk is padded to it in the workspace when
    that is at most 8/3 of the real one (helix_im2col::pads_channels), otherwise the column-buffer path runs
    on the real count."""
    padded = -(-input_channel // GATHER_CHUNK) * GATHER_CHUNK
    return padded if 3 * padded <= 8 * input_channel else input_channel


def conv_kernel_scratch(k, IC=None):
    """Scratch bytes per lane (register spills) of the convolution kernel configuration k runs for this channel count,
    as recorded when the library was built; 0 when the build left no record.  The gather keeps per-copy-slot state
    in registers beside the accumulators, so the largest tiles fit the GEMM but spill in a convolution mode."""
    mode = 2 if (IC is not None and IC % k[6] == 0) else 1     # a K tile inside one filter tap, or the general gather
    for name, res in kernel_resources(library_for_key(k)).items():
        if f"helix_gemm_f16_kernelILi{mode}E" in name:
            return res.get("scratch", 0)
    return 0


def cost_model(prof_dict, M, N, K, IC=None, pointwise=False):
    """GEMM cost model restricted to the MFMA configurations with a conv entry (gemm.hip's), with the
    gather terms above; IC is the channel count the kernel walks (gather_channels); pointwise: is_pointwise()."""
    min_cost = float("inf")
    best_config = (1, 1, 1, 1, 1, 0, 32)
    for k, v in prof_dict.items():
        if k[0] == 0 or is_dtl_key(k):      # neither the GEMV nor the direct-to-LDS libraries have a conv entry
            continue
        if not pointwise and conv_kernel_scratch(k, IC) > 0:  # a spilling gather is never the fastest one
            continue
        cost = conv_config_cost(k, v, M, N, K, short_value(prof_dict, k), IC, pointwise)
        if min_cost > cost:
            min_cost = cost
            best_config = k
    return best_config


def ranked_configs(prof_dict, M, N, K, IC=None, top=VERIFY_TOP, pointwise=False):
    """The `top` convolution-capable configurations with the lowest predicted cost, best first; cost_model returns
    the first of them."""
    cand = []
    for k, v in prof_dict.items():
        if k[0] == 0 or is_dtl_key(k) or (not pointwise and conv_kernel_scratch(k, IC) > 0):
            continue
        cand.append((conv_config_cost(k, v, M, N, K, short_value(prof_dict, k), IC, pointwise), k))
    cand.sort()
    return [k for _, k in cand[:top]]


def verified_config(prof_dict, batch, input_channel, H, W, output_channel, kH, kW, stride, pad, top=VERIFY_TOP):
    """The fastest of the cost model's first `top` configurations on this layer (utils.helix_runtime.fastest_of:
    2 + 5 launches each, the leaders timed again)."""
    M = batch * ((H + 2 * pad - kH) // stride + 1) * ((W + 2 * pad - kW) // stride + 1)
    ICg = gather_channels(input_channel)

    def time_config(k, warmup, iters):
        return load(library_for_key(k)).bench_conv(batch, input_channel, H, W, output_channel, kH, kW, stride, pad,
                                                   warmup=warmup, iters=iters)[1]

    return fastest_of(ranked_configs(prof_dict, M, output_channel, ICg * kH * kW, ICg, top,
                                     is_pointwise(kH, kW, stride, pad) and input_channel % GATHER_CHUNK == 0),
                      time_config, "this layer")


def get_MI355X_FP16_conv_Verified_result(prof_dict, batch, input_channel, H, W, output_channel, kH, kW, stride, pad,
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
    """cost_model on the GEMM extents of a layer (Ampere_FP16_conv.py:432-435)."""
    M = batch * ((H + 2 * pad - kH) // stride + 1) * ((W + 2 * pad - kW) // stride + 1)
    ICg = gather_channels(input_channel)
    return cost_model(prof_dict, M, output_channel, ICg * kH * kW, ICg,
                      is_pointwise(kH, kW, stride, pad) and input_channel % GATHER_CHUNK == 0)


def select_config(prof_dict, batch, input_channel, H, W, output_channel, kH, kW, stride, pad):
    """The configuration the runner launches for this layer: the cost model's ranking, settled on the device the first
    time the layer is met and remembered beside the profile (utils.helix_runtime.tuned_config); the cost model's
    first choice alone with HELIX_SELECTION=model."""
    layer = (batch, input_channel, H, W, output_channel, kH, kW, stride, pad)
    return tuned_config("MI355X_FP16", ("conv",) + layer, prof_dict,
                        lambda: layer_cost_model(prof_dict, *layer),
                        lambda: verified_config(prof_dict, *layer))


def get_MI355X_FP16_conv_Helix_result(prof_dict, batch, input_channel, H, W, output_channel, kH, kW, stride, pad,
                                      backend="hip"):
    if backend != "hip":
        raise ValueError(f"backend {backend!r} is not available for MI355X_FP16 (only 'hip')")
    M = batch * ((H + 2 * pad - kH) // stride + 1) * ((W + 2 * pad - kW) // stride + 1)
    N = output_channel
    K = input_channel * kH * kW
    best_config = select_config(prof_dict, batch, input_channel, H, W, output_channel, kH, kW, stride, pad)
    lib = load(library_for_key(best_config))
    _, avg, _ = lib.bench_conv(batch, input_channel, H, W, output_channel, kH, kW, stride, pad, warmup=10, iters=10)
    cost = avg * 1e3
    tflops = 2 * M * N * K / 1e9 / cost

    return cost, tflops


def get_MI355X_FP16_conv_Oracle_result(prof_dict, batch, input_channel, H, W, output_channel, kH, kW, stride, pad):
    """Exhaustive per-layer search: run every configuration that has a conv entry, keep the fastest (the conv
    counterpart of benchmark_Ampere_FP16_performance_comparison.py:56-69).  Returns (cost_ms, tflops, key)."""
    M = batch * ((H + 2 * pad - kH) // stride + 1) * ((W + 2 * pad - kW) // stride + 1)
    flops = 2.0 * M * output_channel * input_channel * kH * kW
    min_cost, best = float("inf"), None
    for k in prof_dict.keys():
        if k[0] == 0 or is_dtl_key(k):
            continue
        try:
            _, avg, _ = load(library_for_key(k)).bench_conv(batch, input_channel, H, W, output_channel, kH, kW, stride,
                                                            pad, warmup=2, iters=5)
        except Exception:
            continue
        if avg < min_cost:
            min_cost, best = avg, k
    if best is not None:     # the winner once more with the runner's launch counts
        _, min_cost, _ = load(library_for_key(best)).bench_conv(batch, input_channel, H, W, output_channel, kH, kW,
                                                                stride, pad, warmup=10, iters=10)
    return min_cost * 1e3, flops / 1e12 / min_cost, best


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
