"""Lazy function table used by the command-line dispatchers.

The reference's dispatchers import every backend at module top
(scripts/benchmark_op_level_eval.py:3-10), so `-b Ampere_FP16` still needs tvm and onnxruntime
importable.  Here a row names its module and function as strings and is imported when selected.
"""
import importlib


def resolve(row):
    module_name, func_name = row
    return getattr(importlib.import_module(module_name), func_name)


MI355X_BACKENDS = ['MI355X_FP16', 'MI355X_FP32']
