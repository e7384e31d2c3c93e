"""Op-level convolution benchmark of the MI355X_FP16 backend.
Mirrors scripts/Ampere_FP16/benchmark_Ampere_FP16_conv.py:9-23 (same loop, same output line)."""
import math
import os

from utils.get_benchmark_shape_list import get_conv_op_shape_list
from utils.helix_runtime import read_prof_dict
from MI355X_FP16.MI355X_FP16_conv import get_MI355X_FP16_conv_Helix_result, get_MI355X_FP16_conv_miopen_result

root_path = os.getcwd()


def MI355X_FP16_Helix_op_level_Conv_benchmark(backend="hip"):
    prof_dict = read_prof_dict("MI355X_FP16")

    shape_list = get_conv_op_shape_list()
    for batch, input_channel, H, W, output_channel, kH, kW, stride, pad in shape_list:
        _, helix_tflops = get_MI355X_FP16_conv_Helix_result(prof_dict, batch, input_channel, H, W, output_channel, kH, kW, stride, pad, backend)
        print(f'Helix: {helix_tflops:.2f} TFLOPS')


def MI355X_FP16_miopen_op_level_Conv_benchmark():
    """Mirrors Ampere_FP16_cudnn_op_level_Conv_benchmark (benchmark_Ampere_FP16_conv.py)."""
    shape_list = get_conv_op_shape_list()
    for batch, input_channel, H, W, output_channel, kH, kW, stride, pad in shape_list:
        _, miopen_tflops = get_MI355X_FP16_conv_miopen_result(batch, input_channel, H, W, output_channel, kH, kW, stride, pad)
        print(f'miopen: {miopen_tflops:.2f} TFLOPS')


if __name__ == "__main__":

    MI355X_FP16_Helix_op_level_Conv_benchmark(backend="hip")
    MI355X_FP16_miopen_op_level_Conv_benchmark()
