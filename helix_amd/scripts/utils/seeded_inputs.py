"""Seeded synthetic inputs for the five benchmark configurations.

The reference draws unseeded `np.random.rand` operands (scripts/x86_CPU/benchmark_x86_CPU_gemm.py:127-128)
or times uninitialised device memory (src_template/Ampere_FP16/gemm.cu:630-634); the seeds and
distributions below are this backend's own so that CPU and GPU runs see the same numbers.
Generation is float32 from numpy's default_rng, cast afterwards.
"""
import numpy as np

SEED_A = 0
SEED_B = 1


def uniform_pm1(shape, seed):
    """config 1: FP32 GEMM operands ~ U[-1, 1)."""
    return np.random.default_rng(seed).uniform(-1.0, 1.0, size=shape).astype(np.float32)


def normal(shape, std, seed, dtype=np.float32):
    return (np.random.default_rng(seed).standard_normal(size=shape, dtype=np.float32) * np.float32(std)).astype(dtype)


def gemm_operands(M, N, K, dtype):
    """config 2 / 5: A (M,K), B (K,N) ~ N(0, 0.1^2)."""
    return normal((M, K), 0.1, SEED_A, dtype), normal((K, N), 0.1, SEED_B, dtype)


def gemv_operands(M, N, K, dtype=np.float16):
    """config 3: activations x (M,K) ~ N(0,1); weights W (K,N) ~ N(0, 0.02^2)."""
    return normal((M, K), 1.0, SEED_A, dtype), normal((K, N), 0.02, SEED_B, dtype)


def conv_operands(batch, IC, H, W, OC, kH, kW, dtype=np.float16):
    """config 4: NHWC activations and [OC][kH][kW][IC] weights ~ N(0, 0.05^2)."""
    return normal((batch, H, W, IC), 0.05, SEED_A, dtype), normal((OC, kH, kW, IC), 0.05, SEED_B, dtype)
