"""Helpers shared by the GPU test files: host arrays -> device buffers -> one call through the C ABI
(helix_gemm / helix_conv2d of one kernel-template library) -> host array, plus the error measures the
parity tests use."""
import os

import numpy as np
import torch

TOL16 = 2e-2    # FP16 in / FP32 accumulate / FP16 out, normwise
TOL32 = 1e-5    # FP32, normwise


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")


def normwise(got, want):
    want = np.asarray(want, dtype=np.float64)
    return float(np.max(np.abs(np.asarray(got, dtype=np.float64) - want)) / max(np.max(np.abs(want)), 1e-30))


def run_gemm_f16(lib, A, B, ldpad=0):
    """A (M,K) f16, B (K,N) f16 -> C (M,N) f16 through helix_gemm (device layout: B as N x K)."""
    M, K = A.shape
    N = B.shape[1]
    Kp = (K + 7) // 8 * 8 + ldpad
    Ap = np.zeros((M, Kp), np.float16)
    Ap[:, :K] = A
    Bt = np.zeros((N, Kp), np.float16)
    Bt[:, :K] = B.T
    return run_gemm_f16_dev(lib, dev(Ap), dev(Bt), M, N, (K + 7) // 8 * 8, Kp).cpu().numpy()


def run_gemm_f16_dev(lib, dA, dBt, M, N, K, ld):
    """Device operands already in the kernel's layout (A M x ld, B N x ld, K a multiple of 8)."""
    dC = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda:0")
    wsb = lib.workspace_bytes(M, N, K)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda:0")
    lib.gemm(dA.data_ptr(), dBt.data_ptr(), dC.data_ptr(), M, N, K, ld, ld, N, ws.data_ptr(), wsb,
             torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return dC


def run_sgemm_f32(lib, A, B, workspace=True):
    """A (M,K) f32, B (K,N) f32 -> C (M,N) f32 through helix_gemm (device layout: A as K x M).  With the
    workspace the library asks for, few-tile problems are K-partitioned; without it they run unpartitioned."""
    M, K = A.shape
    N = B.shape[1]
    Mp, Np = (M + 3) // 4 * 4, (N + 3) // 4 * 4
    At = np.zeros((K, Mp), np.float32)
    At[:, :M] = A.T
    Bp = np.zeros((K, Np), np.float32)
    Bp[:, :N] = B
    return run_sgemm_f32_dev(lib, dev(At), dev(Bp), M, N, K, Mp, Np, workspace).cpu().numpy()


def run_sgemm_f32_dev(lib, dAt, dB, M, N, K, lda, ldb, workspace=True):
    dC = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda:0")
    wsb = lib.workspace_bytes(M, N, K) if workspace else 0
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda:0")
    lib.gemm(dAt.data_ptr(), dB.data_ptr(), dC.data_ptr(), M, N, K, lda, ldb, N, ws.data_ptr() if wsb else 0, wsb,
             torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return dC


def run_gemv_f32(lib, x, W):
    """x (M,K), W (K,N) f32 through a GEMV library (weights stored N x K)."""
    M, K = x.shape
    N = W.shape[1]
    Kp = (K + 3) // 4 * 4
    xp = np.zeros((M, Kp), np.float32)
    xp[:, :K] = x
    Wt = np.zeros((N, Kp), np.float32)
    Wt[:, :K] = W.T
    dx, dW = dev(xp), dev(Wt)
    dy = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda:0")
    wsb = lib.workspace_bytes(M, N, Kp)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda:0")
    lib.gemm(dx.data_ptr(), dW.data_ptr(), dy.data_ptr(), M, N, Kp, Kp, Kp, N, ws.data_ptr(), wsb)
    torch.cuda.synchronize()
    return dy.cpu().numpy()


def conv_out_hw(H, W, kH, kW, stride, pad):
    return (H + 2 * pad - kH) // stride + 1, (W + 2 * pad - kW) // stride + 1


def run_conv(lib, x, w, stride, pad, dtype):
    batch, H, W, IC = x.shape
    OC, kH, kW, _ = w.shape
    OH, OW = conv_out_hw(H, W, kH, kW, stride, pad)
    dx, dw = dev(x), dev(w)
    dy = torch.full((batch, OH, OW, OC), float("nan"), dtype=dtype, device="cuda:0")
    wsb = lib.conv_workspace_bytes(batch, H, W, IC, OC, kH, kW, stride, pad)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda:0")
    lib.conv2d(dx.data_ptr(), dw.data_ptr(), dy.data_ptr(), batch, H, W, IC, OC, kH, kW, stride, pad,
               ws.data_ptr() if wsb else 0, wsb, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return dy.cpu().numpy()


def sampled_gemm_error(C, A, Bt, rng, n=256, extra=()):
    """max |C[r, c] - <A[r], Bt[c]>| over n random entries (plus `extra` (r, c) pairs) and the scale of the
    sampled truths, both from float64 dot products.  A is M x K, Bt is N x K (host arrays)."""
    M, N = C.shape
    rows = np.concatenate([rng.integers(0, M, n), [0, M - 1], [r for r, _ in extra]]).astype(np.int64)
    cols = np.concatenate([rng.integers(0, N, n), [0, N - 1], [c for _, c in extra]]).astype(np.int64)
    want = np.einsum("ik,ik->i", A[rows].astype(np.float64), Bt[cols].astype(np.float64))
    got = np.asarray(C[rows, cols], dtype=np.float64)
    return float(np.max(np.abs(got - want))), float(np.max(np.abs(want)))


def sampled_conv_error(y, x, w, stride, pad, rng, n=40):
    """max error of n random output pixels (all channels) plus the corners against float64, and the scale."""
    batch, H, W, IC = x.shape
    OC, kH, kW, _ = w.shape
    OH, OW = conv_out_hw(H, W, kH, kW, stride, pad)
    assert y.shape == (batch, OH, OW, OC)
    xp = np.zeros((batch, H + 2 * pad, W + 2 * pad, IC), np.float64)
    xp[:, pad:pad + H, pad:pad + W] = x
    w64 = w.astype(np.float64)
    pts = [(0, 0, 0), (batch - 1, OH - 1, OW - 1), (batch - 1, 0, OW - 1), (0, OH - 1, 0)] + \
          [(int(rng.integers(batch)), int(rng.integers(OH)), int(rng.integers(OW))) for _ in range(n)]
    worst, scale = 0.0, 0.0
    for (b, oh, ow) in pts:
        patch = xp[b, oh * stride:oh * stride + kH, ow * stride:ow * stride + kW]
        want = np.einsum("hwc,ohwc->o", patch, w64)
        worst = max(worst, float(np.max(np.abs(y[b, oh, ow] - want))))
        scale = max(scale, float(np.max(np.abs(want))))
    return worst, scale


def ensure_profiles():
    """The cost-model dicts of both backends (profiling every built configuration takes a couple of seconds on
    the device); returns (prof16, prof32)."""
    from utils import helix_runtime
    from MI355X_FP16 import profile_MI355X_FP16 as p16
    from MI355X_FP32 import profile_MI355X_FP32 as p32
    if not os.path.exists(helix_runtime.prof_dict_path("MI355X_FP16")):
        p16.profile_Helix_MI355X_FP16_gemm_kernel()
    if not os.path.exists(helix_runtime.prof_dict_path("MI355X_FP32")):
        p32.profile_Helix_MI355X_FP32_gemm_kernel()
    return helix_runtime.read_prof_dict("MI355X_FP16"), helix_runtime.read_prof_dict("MI355X_FP32")
