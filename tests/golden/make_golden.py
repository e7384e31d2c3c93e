"""Generates the small golden vectors under tests/golden/ (numpy only; the reference is not involved:
it ships no fixtures for this path, so expected outputs come from float64 arithmetic).

    python tests/golden/make_golden.py

Each .npz holds seeded inputs and the float64-derived expected output of one case:
  gemm_f32_*.npz : A (M,K) f32, B (K,N) f32, C64 = A@B in float64
  gemm_f16_*.npz : A (M,K) f16, B (K,N) f16, C64 = f64(A)@f64(B)         (exact products, f64 sums)
  conv_f16_*.npz : x (B,H,W,IC) f16, w (OC,kH,kW,IC) f16, stride, pad, y64 (B,OH,OW,OC) float64
"""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def conv_nhwc_f64(x, w, stride, pad):
    B, H, W, IC = x.shape
    OC, kH, kW, _ = w.shape
    OH = (H + 2 * pad - kH) // stride + 1
    OW = (W + 2 * pad - kW) // stride + 1
    xp = np.zeros((B, H + 2 * pad, W + 2 * pad, IC), dtype=np.float64)
    xp[:, pad:pad + H, pad:pad + W, :] = x
    y = np.zeros((B, OH, OW, OC), dtype=np.float64)
    w64 = w.astype(np.float64)
    for oh in range(OH):
        for ow in range(OW):
            patch = xp[:, oh * stride:oh * stride + kH, ow * stride:ow * stride + kW, :]
            y[:, oh, ow, :] = np.einsum("bhwc,ohwc->bo", patch, w64)
    return y


def main():
    rng = np.random.default_rng(20240)
    for (M, N, K) in [(64, 64, 64), (33, 47, 40), (1, 64, 72), (48, 16, 8)]:
        A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
        B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
        np.savez(os.path.join(HERE, f"gemm_f32_{M}x{N}x{K}.npz"), A=A, B=B,
                 C64=A.astype(np.float64) @ B.astype(np.float64))
        A16 = (rng.standard_normal((M, K)) * 0.1).astype(np.float16)
        B16 = (rng.standard_normal((K, N)) * 0.1).astype(np.float16)
        np.savez(os.path.join(HERE, f"gemm_f16_{M}x{N}x{K}.npz"), A=A16, B=B16,
                 C64=A16.astype(np.float64) @ B16.astype(np.float64))
    for name, (B_, H, W, IC, OC, k, s, p) in {"3x3s1p1": (2, 9, 7, 8, 16, 3, 1, 1), "1x1s2p0": (2, 8, 8, 16, 8, 1, 2, 0),
                                              "3x3s2p1": (1, 11, 10, 8, 24, 3, 2, 1)}.items():
        x = (rng.standard_normal((B_, H, W, IC)) * 0.05).astype(np.float16)
        w = (rng.standard_normal((OC, k, k, IC)) * 0.05).astype(np.float16)
        np.savez(os.path.join(HERE, f"conv_f16_{name}.npz"), x=x, w=w, stride=s, pad=p,
                 y64=conv_nhwc_f64(x, w, s, p))


if __name__ == "__main__":
    main()
