"""Model-level CNN benchmark of the MI355X_FP16 backend: summed per-layer latency.
Mirrors scripts/Ampere_FP16/benchmark_Ampere_FP16_model_level_CNN.py:9-27."""
import math
import os

from utils.get_benchmark_shape_list import get_cnn_opset_shape_List
from utils.helix_runtime import read_prof_dict
from MI355X_FP16.MI355X_FP16_conv import get_MI355X_FP16_conv_Helix_result, get_MI355X_FP16_conv_miopen_result

root_path = os.getcwd()


def _summed_cost(prof_dict, shape_list, backend):
    total = 0
    for batch, input_channel, H, W, output_channel, kH, kW, stride, pad in shape_list:
        cost, _ = get_MI355X_FP16_conv_Helix_result(prof_dict, batch, input_channel, H, W, output_channel, kH, kW, stride, pad, backend)
        total += cost
    return total


def MI355X_FP16_Helix_model_level_CNN_benchmark(backend="hip"):
    prof_dict = read_prof_dict("MI355X_FP16")

    AlexNet_shape_list, ResNet_shape_list, GoogleNet_shape_list = get_cnn_opset_shape_List()

    helix_AlexNet_cost = _summed_cost(prof_dict, AlexNet_shape_list, backend)
    helix_ResNet_cost = _summed_cost(prof_dict, ResNet_shape_list, backend)
    helix_GoogleNet_cost = _summed_cost(prof_dict, GoogleNet_shape_list, backend)

    print(f'AlexNet: {helix_AlexNet_cost:.2f} ms, ResNet: {helix_ResNet_cost:.2f} ms, GoogleNet: {helix_GoogleNet_cost:.2f} ms')


def MI355X_FP16_miopen_model_level_CNN_benchmark():
    """Mirrors Ampere_FP16_cudnn_model_level_CNN_benchmark (benchmark_Ampere_FP16_model_level_CNN.py)."""
    totals = []
    for shape_list in get_cnn_opset_shape_List():
        total, memo = 0, {}
        for shape in shape_list:
            if shape not in memo:
                memo[shape], _ = get_MI355X_FP16_conv_miopen_result(*shape)
            total += memo[shape]
        totals.append(total)
    print(f'AlexNet: {totals[0]:.2f} ms, ResNet: {totals[1]:.2f} ms, GoogleNet: {totals[2]:.2f} ms')


if __name__ == "__main__":

    MI355X_FP16_Helix_model_level_CNN_benchmark(backend="hip")
    MI355X_FP16_miopen_model_level_CNN_benchmark()
