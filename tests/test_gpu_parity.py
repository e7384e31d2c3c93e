"""GPU parity tests: every kernel family is called through the C ABI (ctypes -> helix_gemm / helix_conv2d)
and compared with the CPU oracle on the same seeded inputs.

Tolerances (normwise: |got - want| <= tol * max|want|, because the inputs are zero-mean and an elementwise
relative error is unbounded near zero):
    FP16 in / FP32 accumulate / FP16 out : 2e-2   (the stated bound; observed values are ~5e-4)
    FP32                                 : 1e-5
Integer-valued inputs make FP32 accumulation exact, so tile / edge / split-K mistakes show as exact
mismatches in those cases.
"""
import glob
import os

import numpy as np
import pytest
import torch

from oracle import oracle as O
from utils import seeded_inputs
from utils.helix_runtime import load
from utils.hip_ctypes import HelixError, HELIX_ERR_INVALID_VALUE, HELIX_ERR_UNSUPPORTED, HELIX_ERR_WORKSPACE
from MI355X_FP16 import build_MI355X_FP16 as b16
from MI355X_FP32 import build_MI355X_FP32 as b32
from MI355X_FP32 import MI355X_FP32_gemm as g32

pytestmark = pytest.mark.gpu

TOL16 = 2e-2
TOL32 = 1e-5
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


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
    dA, dB = dev(Ap), dev(Bt)
    dC = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda:0")
    Kk = (K + 7) // 8 * 8
    wsb = lib.workspace_bytes(M, N, Kk)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda:0")
    lib.gemm(dA.data_ptr(), dB.data_ptr(), dC.data_ptr(), M, N, Kk, Kp, Kp, N, ws.data_ptr(), wsb,
             torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return dC.cpu().numpy()


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
    dA, dB = dev(At), dev(Bp)
    dC = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda:0")
    wsb = lib.workspace_bytes(M, N, K) if workspace else 0
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda:0")
    lib.gemm(dA.data_ptr(), dB.data_ptr(), dC.data_ptr(), M, N, K, Mp, Np, N, ws.data_ptr() if wsb else 0, wsb,
             torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return dC.cpu().numpy()


FP16_CONFIGS = [(2, 256, 256, 128, 128, 64), (2, 256, 256, 64, 128, 64), (2, 128, 128, 64, 64, 128), (2, 64, 64, 32, 32, 64),
                (2, 32, 32, 32, 32, 128), (2, 256, 64, 64, 32, 64), (2, 64, 256, 32, 128, 128), (2, 128, 256, 128, 64, 64),
                (2, 128, 128, 64, 64, 64), (2, 256, 256, 128, 64, 64), (2, 64, 64, 32, 32, 128), (2, 32, 128, 32, 32, 64),
                # 48- and 96-column wave tiles (three and six MFMA tile columns per wave)
                (2, 256, 192, 128, 96, 64), (2, 128, 96, 64, 48, 128), (2, 32, 48, 32, 48, 64), (2, 128, 192, 32, 96, 128),
                (2, 256, 96, 64, 96, 64)]
# split-K libraries are built for wave tiles of up to 32 x 64
FP16_SPLITK_CONFIGS = [(2, 64, 64, 32, 32, 64), (2, 32, 32, 32, 32, 128), (2, 256, 64, 64, 32, 64), (2, 64, 256, 32, 64, 128),
                       (2, 128, 128, 32, 64, 64), (2, 128, 128, 64, 32, 128), (2, 32, 128, 32, 64, 64), (2, 64, 192, 32, 48, 64),
                       (2, 128, 96, 32, 48, 128), (2, 32, 48, 32, 48, 64), (2, 128, 64, 64, 32, 128)]


def test_parity_configs_are_built_points():
    assert set(FP16_CONFIGS) <= set(b16.iter_configs()) and set(FP16_SPLITK_CONFIGS) <= set(b16.iter_splitk_configs())


# ---------------------------------------------------------------------------------------------
# FP16 GEMM
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("splitk,cfg", [(0, c) for c in FP16_CONFIGS] + [(1, c) for c in FP16_SPLITK_CONFIGS])
def test_gemm_f16_vs_oracle(cfg, splitk):
    lib = load(b16.kernel_library("gemm_splitK" if splitk else "gemm", *cfg))
    for (M, N, K) in [(256, 256, 256), (300, 200, 136), (1, 7, 8), (513, 1025, 72), (1024, 1024, 1024), (130, 260, 4096),
                      (77, 90, 520), (64, 66, 2048)]:
        A, B = seeded_inputs.gemm_operands(M, N, K, np.float16)
        got = run_gemm_f16(lib, A, B)
        want = O.hgemm_f32acc(A, B)
        assert not np.isnan(got).any(), (cfg, M, N, K)
        assert normwise(got, want) < TOL16, (cfg, M, N, K)


@pytest.mark.parametrize("cfg,cfg_splitk", list(zip(FP16_CONFIGS[:4], FP16_SPLITK_CONFIGS[:4])))
def test_gemm_f16_integer_inputs_exact(cfg, cfg_splitk):
    """Small integers: products and FP32 sums are exact, and the sums are kept below 2048 in magnitude so
    the FP16 result is exact too -- any wrong tile, edge or split-K index is an exact mismatch."""
    rng = np.random.default_rng(3)
    for splitk in (0, 1):
        lib = load(b16.kernel_library("gemm_splitK", *cfg_splitk) if splitk else b16.kernel_library("gemm", *cfg))
        for (M, N, K) in [(257, 129, 200), (64, 500, 328)]:
            A = rng.integers(-2, 3, (M, K)).astype(np.float16)
            B = rng.integers(-2, 3, (K, N)).astype(np.float16)
            want = A.astype(np.int64) @ B.astype(np.int64)
            assert np.abs(want).max() < 2048
            got = run_gemm_f16(lib, A, B)
            assert np.array_equal(got.astype(np.int64), want), (cfg, splitk, M, N, K)
            assert np.array_equal(O.hgemm_f32acc(A, B).astype(np.int64), want)


def test_gemm_f16_closed_forms_and_layout():
    lib = load(b16.kernel_library("gemm", 2, 128, 128, 64, 64, 64))
    rng = np.random.default_rng(4)
    B = (rng.standard_normal((160, 96)) * 0.5).astype(np.float16)
    # identity picks B exactly; a unit vector e_i e_j^T moves row j of B to row i (transposed operands fail this)
    assert np.array_equal(run_gemm_f16(lib, np.eye(160, dtype=np.float16), B), B)
    E = np.zeros((40, 160), np.float16)
    E[7, 150] = 1
    want = np.zeros((40, 96), np.float16)
    want[7] = B[150]
    assert np.array_equal(run_gemm_f16(lib, E, B), want)
    # ones: C == K, exact up to 2048
    assert np.array_equal(run_gemm_f16(lib, np.ones((33, 2048), np.float16), np.ones((2048, 65), np.float16)),
                          np.full((33, 65), 2048, np.float16))
    # row strides larger than K (padded leading dimensions) do not leak into the result
    A = (rng.standard_normal((100, 160)) * 0.1).astype(np.float16)
    assert normwise(run_gemm_f16(lib, A, B, ldpad=24), O.hgemm_f32acc(A, B)) < TOL16


def test_gemm_f16_golden_vectors():
    lib = load(b16.kernel_library("gemm", 2, 64, 64, 32, 32, 64))
    files = sorted(glob.glob(os.path.join(GOLDEN, "gemm_f16_*.npz")))
    assert files
    for f in files:
        d = np.load(f)
        got = run_gemm_f16(lib, d["A"], d["B"])
        assert normwise(got, d["C64"]) < TOL16, f
        assert normwise(got, O.hgemm_f32acc(d["A"], d["B"])) < TOL16, f


# the 256 x 256-tile configurations the search's winner at 8192^3 has come from (register-staged and direct-to-LDS)
FULL_SIZE_KEYS = [(2, 256, 256, 64, 128, 0, 64), (2, 256, 256, 128, 64, 0, 64), (2, 256, 256, 128, 128, 0, 64),
                  (2, 256, 256, 64, 128, 0, 64, 1), (2, 256, 256, 128, 64, 0, 64, 1)]


@pytest.fixture(scope="module")
def full_size_operands():
    M = N = K = 8192
    A, B = seeded_inputs.gemm_operands(M, N, K, np.float16)
    Bt = np.ascontiguousarray(B.T)
    return A, Bt, dev(A), dev(Bt)


def test_full_size_keys_cover_the_benchmark_candidates():
    """The configurations bench.py knows counted traffic for (its winners so far) are the ones tested at full size."""
    import bench
    assert set(FULL_SIZE_KEYS) == set(bench.MEASURED_TRAFFIC)


@pytest.mark.parametrize("key", FULL_SIZE_KEYS, ids=lambda k: "_".join(map(str, k)))
def test_gemm_f16_full_size_properties(key, full_size_operands):
    """8192^3 (the benchmark size): too big for the CPU oracle in seconds, so check size-independent facts:
    a random sample of outputs against float64 dot products, and linearity in A."""
    M = N = K = 8192
    lib = load(b16.library_for_key(key))
    A, Bt, dA, dB = full_size_operands
    dC = torch.empty((M, N), dtype=torch.float16, device="cuda:0")
    lib.gemm(dA.data_ptr(), dB.data_ptr(), dC.data_ptr(), M, N, K, K, K, N)
    torch.cuda.synchronize()
    C = dC.cpu().numpy()
    rng = np.random.default_rng(5)
    rows, cols = rng.integers(0, M, 256), rng.integers(0, N, 256)
    want = np.einsum("ik,ik->i", A[rows].astype(np.float64), Bt[cols].astype(np.float64))
    scale = np.abs(want).max()
    assert np.max(np.abs(C[rows, cols].astype(np.float64) - want)) < TOL16 * scale
    # corners and tile seams
    for (r, c) in [(0, 0), (M - 1, N - 1), (255, 256), (256, 255), (4095, 4096), (8191, 0)]:
        w = float(A[r].astype(np.float64) @ Bt[c].astype(np.float64))
        assert abs(float(C[r, c]) - w) < TOL16 * scale
    # linearity: (2A) B == 2 (A B) exactly -- scaling by 2 is exact in FP16 and FP32 -- wherever the FP16
    # result is a normal number (a subnormal result rounds on a fixed grid, where round(2x) != 2 round(x))
    dA2 = dA * 2
    dC2 = torch.empty_like(dC)
    lib.gemm(dA2.data_ptr(), dB.data_ptr(), dC2.data_ptr(), M, N, K, K, K, N)
    torch.cuda.synchronize()
    normal = dC.abs() >= 2.0 ** -13
    assert normal.float().mean().item() > 0.999
    assert torch.equal(dC2[normal], (dC * 2)[normal])
    assert (dC2.float() - 2 * dC.float()).abs().max().item() <= 2.0 ** -23


SPLITK_PATH_SCRIPT = r"""
import sys, numpy as np, torch
sys.path.insert(0, sys.argv[2]); sys.path.insert(0, sys.argv[3]); sys.path.insert(0, sys.argv[4])
from utils import seeded_inputs
from utils.helix_runtime import load
from MI355X_FP16 import build_MI355X_FP16 as b16
from gpu_helpers import run_gemm_f16, run_conv
out = {}
for ci, cfg in enumerate([(2, 64, 64, 32, 32, 128), (2, 128, 128, 32, 64, 64), (2, 32, 128, 32, 32, 64)]):
    lib = load(b16.kernel_library("gemm_splitK", *cfg))
    for (M, N, K) in [(196, 512, 4608), (130, 260, 4096), (8, 4096, 1024), (1000, 72, 520)]:
        A, B = seeded_inputs.gemm_operands(M, N, K, np.float16)
        out[f"g{ci}_{M}_{N}_{K}"] = run_gemm_f16(lib, A, B)
    x, w = seeded_inputs.conv_operands(4, 256, 7, 7, 128, 3, 3)
    out[f"c{ci}"] = run_conv(lib, x, w, 1, 1, torch.float16)
from MI355X_FP32 import build_MI355X_FP32 as b32
from gpu_helpers import run_sgemm_f32
for ci, cfg in enumerate([(64, 64, 32, 32, 32), (128, 128, 16, 32, 64)]):
    lib = load(b32.sgemm_library(*cfg))
    for (M, N, K) in [(300, 200, 4096), (100, 96, 1000), (661, 768, 3072)]:
        assert lib.workspace_bytes(M, N, K) > 0
        A = seeded_inputs.uniform_pm1((M, K), seeded_inputs.SEED_A)
        B = seeded_inputs.uniform_pm1((K, N), seeded_inputs.SEED_B)
        out[f"s{ci}_{M}_{N}_{K}"] = run_sgemm_f32(lib, A, B)
np.savez(sys.argv[1], **out)
"""


def test_splitk_in_launch_sum_and_reduction_kernel_give_identical_bits(tmp_path):
    """Split-K libraries (FP16) and K-partitioned launches (FP32) add a tile's partitions inside the launch (the last workgroup of the tile to finish, all on
    one XCD) or, with HELIX_SPLITK_REDUCE=kernel, in a second kernel: same partials, same order of FP32 additions, so
    the FP16 results are bit-identical; both are within tolerance of the oracle."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    args = [os.path.join(root, "helix_amd", "scripts"), os.path.join(root, "tests"), root]
    outs = {}
    for mode in ("in_launch", "kernel"):
        env = dict(os.environ, HELIX_DEBUG="1")
        env.pop("HELIX_SPLITK_REDUCE", None)
        if mode == "kernel":
            env["HELIX_SPLITK_REDUCE"] = "kernel"
        path = str(tmp_path / f"{mode}.npz")
        run = subprocess.run([sys.executable, "-c", SPLITK_PATH_SCRIPT, path] + args, capture_output=True, text=True,
                             env=env, cwd=root, timeout=300)
        assert run.returncode == 0, run.stderr[-2000:]
        # the in-launch path announces the workgroup id -> XCC_ID deal it found; the kernel path never probes
        assert ("deals workgroup ids 0..7 to XCC_IDs" in run.stderr) == (mode == "in_launch"), run.stderr[-500:]
        outs[mode] = dict(np.load(path))
    assert outs["in_launch"].keys() == outs["kernel"].keys() and len(outs["kernel"]) == 15 + 6
    for name, got in outs["in_launch"].items():
        assert not np.isnan(got).any(), name
        bits = np.uint16 if got.dtype == np.float16 else np.uint32
        assert np.array_equal(got.view(bits), outs["kernel"][name].view(bits)), name
    A32 = seeded_inputs.uniform_pm1((300, 4096), seeded_inputs.SEED_A)
    B32 = seeded_inputs.uniform_pm1((4096, 200), seeded_inputs.SEED_B)
    assert normwise(outs["in_launch"]["s0_300_200_4096"], O.sgemm_seqk(A32, B32)) < TOL32
    A, B = seeded_inputs.gemm_operands(196, 512, 4608, np.float16)
    assert normwise(outs["in_launch"]["g0_196_512_4608"], O.hgemm_f32acc(A, B)) < TOL16
    x, w = seeded_inputs.conv_operands(4, 256, 7, 7, 128, 3, 3)
    assert normwise(outs["in_launch"]["c1"], O.conv2d_nhwc(x, w, 1, 1)) < TOL16


def test_gemm_f16_rejects_bad_arguments():
    lib = load(b16.kernel_library("gemm", 2, 128, 128, 64, 64, 64))
    A = torch.zeros((64, 64), dtype=torch.float16, device="cuda:0")
    C = torch.zeros((64, 64), dtype=torch.float16, device="cuda:0")
    p = A.data_ptr()
    assert lib.gemm(p, p, C.data_ptr(), 64, 64, 60, 64, 64, 64, check=False) == HELIX_ERR_INVALID_VALUE   # K % 8
    assert lib.gemm(p, p, C.data_ptr(), 64, 64, 64, 60, 64, 64, check=False) == HELIX_ERR_INVALID_VALUE   # lda % 8
    assert lib.gemm(p, p, C.data_ptr(), 64, 64, 64, 32, 64, 64, check=False) == HELIX_ERR_INVALID_VALUE   # lda < K
    assert lib.gemm(p + 2, p, C.data_ptr(), 32, 32, 32, 64, 64, 64, check=False) == HELIX_ERR_INVALID_VALUE  # alignment
    assert lib.gemm(0, p, C.data_ptr(), 64, 64, 64, 64, 64, 64, check=False) == HELIX_ERR_INVALID_VALUE
    assert lib.gemm(p, p, C.data_ptr(), 0, 64, 64, 64, 64, 64, check=False) == HELIX_ERR_INVALID_VALUE
    with pytest.raises(HelixError):
        lib.gemm(p, p, C.data_ptr(), 64, 64, 60, 64, 64, 64)
    sk = load(b16.kernel_library("gemm_splitK", 2, 128, 128, 32, 64, 64))
    assert sk.workspace_bytes(64, 64, 64) == 2 * 64 * 64 * 4           # one K tile: the minimum 2-way split
    assert sk.workspace_bytes(64, 64, 4096) == 8 * 64 * 64 * 4         # one output tile, long K: 8-way
    assert sk.gemm(p, p, C.data_ptr(), 64, 64, 64, 64, 64, 64, 0, 0, check=False) == HELIX_ERR_WORKSPACE


# ---------------------------------------------------------------------------------------------
# FP16 GEMV
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["gemv", "gemv_splitK"])
def test_gemv_f16_vs_oracle(name):
    lib = load(b16.kernel_library(name))
    for M in (1, 2, 3, 4, 5, 8, 9, 12, 16, 17, 33):
        for (N, K) in [(128, 512), (1000, 1032), (4096, 4096), (9001, 520), (20000, 8)]:
            x, W = seeded_inputs.gemv_operands(M, N, K)
            got = run_gemm_f16(lib, x, W)
            want = O.hgemm_f32acc(x, W)
            assert not np.isnan(got).any(), (M, N, K)
            assert normwise(got, want) < TOL16, (M, N, K)


def test_gemv_f16_integer_inputs_exact():
    rng = np.random.default_rng(6)
    for name in ("gemv", "gemv_splitK"):
        lib = load(b16.kernel_library(name))
        for (M, N, K) in [(1, 777, 1536), (4, 2050, 520), (16, 300, 1024), (7, 4100, 2056), (11, 1030, 776), (35, 257, 264)]:
            x = rng.integers(-2, 3, (M, K)).astype(np.float16)
            W = rng.integers(-1, 2, (K, N)).astype(np.float16)
            want = x.astype(np.int64) @ W.astype(np.int64)
            assert np.abs(want).max() < 2048
            assert np.array_equal(run_gemm_f16(lib, x, W).astype(np.int64), want), (name, M, N, K)
            # leading dimensions wider than K (rows 16 bytes apart from the packed layout)
            assert np.array_equal(run_gemm_f16(lib, x, W, ldpad=8).astype(np.int64), want), (name, M, N, K, "ld")


def test_gemv_f16_streamed_mfma_work_splits():
    """The two work splits of the LDS-streamed MFMA variant (9 or more activation rows): few weight rows and a long K
    (the waves of a workgroup split the columns and add their sums through LDS), many rows (a wave owns its row
    groups), with K ranges over grid z on top, ragged in every extent; integer-valued, so exact in any order."""
    rng = np.random.default_rng(66)
    for name in ("gemv", "gemv_splitK"):
        lib = load(b16.kernel_library(name))
        for (M, N, K) in [(16, 48, 8192), (9, 17, 5000), (13, 4096, 4096), (16, 30000, 264), (10, 130, 1032),
                          (16, 2000, 3080), (33, 64, 2048)]:
            x = rng.integers(-1, 2, (M, K)).astype(np.float16)
            W = rng.integers(-1, 2, (K, N)).astype(np.float16)
            want = x.astype(np.int64) @ W.astype(np.int64)
            assert np.abs(want).max() < 2048
            assert np.array_equal(run_gemm_f16(lib, x, W).astype(np.int64), want), (name, M, N, K)


def test_gemv_f16_baseline_shapes_sampled():
    """The decode shapes at full size: sampled outputs against float64 dot products."""
    lib = load(b16.kernel_library("gemv"))
    rng = np.random.default_rng(7)
    for (K, N) in [(4096, 11008), (8192, 28672)]:
        for M in (1, 16):
            x, W = seeded_inputs.gemv_operands(M, N, K)
            Wt = np.ascontiguousarray(W.T)
            dx, dW = dev(x), dev(Wt)
            dy = torch.empty((M, N), dtype=torch.float16, device="cuda:0")
            wsb = lib.workspace_bytes(M, N, K)   # wide activation tiles partition K and need FP32 scratch
            ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda:0")
            lib.gemm(dx.data_ptr(), dW.data_ptr(), dy.data_ptr(), M, N, K, K, K, N, ws.data_ptr(), wsb)
            torch.cuda.synchronize()
            y = dy.cpu().numpy()
            cols = np.concatenate([rng.integers(0, N, 200), [0, N - 1]])
            want = x.astype(np.float64) @ Wt[cols].astype(np.float64).T
            assert np.max(np.abs(y[:, cols] - want)) < TOL16 * np.abs(want).max()


def test_gemv_has_no_conv_entry():
    lib = load(b16.kernel_library("gemv"))
    t = torch.zeros(4096, dtype=torch.float16, device="cuda:0")
    assert lib.conv2d(t.data_ptr(), t.data_ptr(), t.data_ptr(), 1, 4, 4, 8, 8, 1, 1, 1, 0, check=False) == \
        HELIX_ERR_UNSUPPORTED


# ---------------------------------------------------------------------------------------------
# FP16 implicit-GEMM convolution
# ---------------------------------------------------------------------------------------------
def run_conv(lib, x, w, stride, pad, dtype):
    batch, H, W, IC = x.shape
    OC, kH, kW, _ = w.shape
    OH, OW = O.conv_out_hw(H, W, kH, kW, stride, pad)
    dx, dw = dev(x), dev(w)
    dy = torch.full((batch, OH, OW, OC), float("nan"), dtype=dtype, device="cuda:0")
    wsb = lib.conv_workspace_bytes(batch, H, W, IC, OC, kH, kW, stride, pad)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda:0")
    lib.conv2d(dx.data_ptr(), dw.data_ptr(), dy.data_ptr(), batch, H, W, IC, OC, kH, kW, stride, pad,
               ws.data_ptr() if wsb else 0, wsb, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return dy.cpu().numpy()


CONV_GEOMS = [(2, 14, 14, 16, 24, 3, 3, 1, 1), (2, 15, 13, 8, 8, 3, 3, 2, 1), (3, 8, 8, 32, 16, 1, 1, 2, 0),
              (1, 12, 12, 8, 40, 5, 5, 1, 2), (2, 9, 9, 64, 64, 3, 3, 1, 1), (1, 7, 7, 24, 16, 3, 3, 1, 0),
              (2, 6, 10, 72, 8, 1, 1, 1, 0)]
# channel counts that are not a multiple of the gather chunk: channel-padded copies in the workspace (IC = 3, 6,
# 25; 2 in FP32) or explicit im2col + GEMM through the workspace (IC = 1; 2 in FP16)
CONV_GEOMS_ODD = [(2, 20, 20, 3, 16, 7, 7, 2, 3), (1, 9, 11, 1, 8, 5, 5, 2, 0), (2, 8, 8, 25, 24, 5, 5, 1, 2),
                  (1, 10, 10, 6, 10, 3, 3, 1, 1), (3, 13, 13, 3, 96, 11, 11, 4, 0), (2, 7, 9, 2, 8, 3, 3, 1, 1)]


@pytest.mark.parametrize("cfg", [(2, 128, 128, 64, 64, 64), (2, 64, 64, 32, 32, 64), (2, 256, 64, 64, 32, 64),
                                 (2, 128, 64, 64, 32, 128), (2, 256, 256, 128, 64, 64), (2, 64, 128, 32, 32, 64),
                                 (2, 128, 96, 64, 48, 128), (2, 64, 192, 32, 48, 64)])
def test_conv_f16_vs_oracle(cfg):
    lib = load(b16.kernel_library("gemm", *cfg))
    for (batch, H, W, IC, OC, kH, kW, stride, pad) in CONV_GEOMS + CONV_GEOMS_ODD:
        x, w = seeded_inputs.conv_operands(batch, IC, H, W, OC, kH, kW)
        got = run_conv(lib, x, w, stride, pad, torch.float16)
        want = O.conv2d_nhwc(x, w, stride, pad)
        assert got.shape == want.shape
        assert not np.isnan(got).any(), (cfg, batch, H, W, IC, OC, kH, kW, stride, pad)
        assert normwise(got, want) < TOL16, (cfg, batch, H, W, IC, OC, kH, kW, stride, pad)


def test_conv_f16_golden_and_special_cases():
    lib = load(b16.kernel_library("gemm", 2, 64, 64, 32, 32, 64))
    for f in sorted(glob.glob(os.path.join(GOLDEN, "conv_f16_*.npz"))):
        d = np.load(f)
        got = run_conv(lib, d["x"], d["w"], int(d["stride"]), int(d["pad"]), torch.float16)
        assert normwise(got, d["y64"]) < TOL16, f
    # 1x1 stride 1 == GEMM on the reshaped tensors: bit-identical to the GEMM entry point of the same library
    x, w = seeded_inputs.conv_operands(2, 64, 12, 12, 48, 1, 1)
    y = run_conv(lib, x, w, 1, 0, torch.float16)
    g = run_gemm_f16(lib, x.reshape(-1, 64), np.ascontiguousarray(w.reshape(48, 64).T))
    assert np.array_equal(y.reshape(-1, 48), g)
    # integer-valued inputs: exact, padding taps contribute exactly zero
    rng = np.random.default_rng(8)
    xi = rng.integers(-2, 3, (2, 9, 8, 8)).astype(np.float16)
    wi = rng.integers(-2, 3, (16, 3, 3, 8)).astype(np.float16)
    want = O.conv2d_nhwc(xi.astype(np.float32), wi.astype(np.float32), 2, 1)
    assert np.array_equal(run_conv(lib, xi, wi, 2, 1, torch.float16).astype(np.float32), want)
    # IC = 3 runs on channel-padded copies, IC = 1 through the column buffer: exact on integers too, also through a
    # split-K library, and refused without the workspace rather than mis-computed
    xi3 = rng.integers(-2, 3, (2, 9, 8, 3)).astype(np.float16)
    wi3 = rng.integers(-2, 3, (16, 3, 3, 3)).astype(np.float16)
    want3 = O.conv2d_nhwc(xi3.astype(np.float32), wi3.astype(np.float32), 2, 1)
    assert np.array_equal(run_conv(lib, xi3, wi3, 2, 1, torch.float16).astype(np.float32), want3)
    libk = load(b16.kernel_library("gemm_splitK", 2, 64, 64, 32, 32, 64))
    assert np.array_equal(run_conv(libk, xi3, wi3, 2, 1, torch.float16).astype(np.float32), want3)
    xi1 = rng.integers(-2, 3, (2, 9, 8, 1)).astype(np.float16)
    wi1 = rng.integers(-2, 3, (16, 3, 3, 1)).astype(np.float16)
    want1 = O.conv2d_nhwc(xi1.astype(np.float32), wi1.astype(np.float32), 2, 1)
    for l in (lib, libk):
        assert np.array_equal(run_conv(l, xi1, wi1, 2, 1, torch.float16).astype(np.float32), want1)
    # padded copies: 64 pixels and 72 filter taps of 8 halves, each rounded up to 256 bytes
    assert lib.conv_workspace_bytes(1, 8, 8, 3, 8, 3, 3, 1, 1) == 64 * 8 * 2 + 1280
    # column buffer: 64 rows and 8 filters of K = 9 padded to 16 halves
    assert lib.conv_workspace_bytes(1, 8, 8, 1, 8, 3, 3, 1, 1) >= 64 * 16 * 2 + 8 * 16 * 2
    assert lib.conv_workspace_bytes(1, 8, 8, 8, 8, 3, 3, 1, 1) == 0
    t = torch.zeros(4096, dtype=torch.float16, device="cuda:0")
    for ic in (3, 1):
        assert lib.conv2d(t.data_ptr(), t.data_ptr(), t.data_ptr(), 1, 8, 8, ic, 8, 3, 3, 1, 1, check=False) == \
            HELIX_ERR_WORKSPACE


def test_conv_f16_baseline_layers_sampled():
    """The six ResNet-50-shaped layers at batch 32: sampled output pixels against float64."""
    from utils.get_benchmark_shape_list import get_baseline_conv_shape_list
    lib = load(b16.kernel_library("gemm", 2, 128, 64, 64, 32, 64))
    rng = np.random.default_rng(9)
    for (batch, IC, H, W, OC, kH, kW, stride, pad) in get_baseline_conv_shape_list():
        x, w = seeded_inputs.conv_operands(batch, IC, H, W, OC, kH, kW)
        y = run_conv(lib, x, w, stride, pad, torch.float16)
        OH, OW = O.conv_out_hw(H, W, kH, kW, stride, pad)
        assert y.shape == (batch, OH, OW, OC)
        xp = np.zeros((batch, H + 2 * pad, W + 2 * pad, IC), np.float64)
        xp[:, pad:pad + H, pad:pad + W] = x
        w64 = w.astype(np.float64)
        pts = [(0, 0, 0), (batch - 1, OH - 1, OW - 1), (batch - 1, 0, OW - 1)] + \
              [(int(rng.integers(batch)), int(rng.integers(OH)), int(rng.integers(OW))) for _ in range(40)]
        worst, scale = 0.0, 0.0
        for (b, oh, ow) in pts:
            patch = xp[b, oh * stride:oh * stride + kH, ow * stride:ow * stride + kW]
            want = np.einsum("hwc,ohwc->o", patch, w64)
            worst = max(worst, np.max(np.abs(y[b, oh, ow] - want)))
            scale = max(scale, np.max(np.abs(want)))
        assert worst < TOL16 * scale, (batch, IC, H, W, OC, kH, kW, stride, pad)


def _sampled_conv_check(y, x, w, stride, pad, tol, rng, n=40):
    batch, H, W, IC = x.shape
    OC, kH, kW, _ = w.shape
    OH, OW = O.conv_out_hw(H, W, kH, kW, stride, pad)
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
        worst = max(worst, np.max(np.abs(y[b, oh, ow] - want)))
        scale = max(scale, np.max(np.abs(want)))
    assert not np.isnan(y).any()
    assert worst < tol * scale, (x.shape, w.shape, stride, pad)


def test_gemm_random_shapes_vs_oracle():
    """Seeded random GEMM extents (ragged M and N, K from 1 to a few thousand so that K partitions of every
    size occur) on tile, split-K, K-group and GEMV libraries, FP16 and FP32, against the oracle."""
    rng = np.random.default_rng(44)
    lib16 = [load(b16.kernel_library("gemm", 2, 128, 96, 64, 48, 128)), load(b16.kernel_library("gemm_splitK", 2, 64, 64, 32, 32, 64)),
             load(b16.kernel_library("gemm_splitK", 2, 32, 128, 32, 32, 128))]
    lib32 = [load(b32.sgemm_library(128, 64, 32, 64, 32)), load(b32.sgemm_library(32, 32, 32, 32, 32, 4)),
             load(b32.sgemm_library(32, 32, 128, 32, 32, 8))]
    gemv16, gemv32 = load(b16.kernel_library("gemv")), load(b32.kernel_library("gemv_fp32"))
    for case in range(36):
        M, N = int(rng.integers(1, 400)), int(rng.integers(1, 400))
        K = int(rng.choice([1, 7, 33, 250, 1000, 2500])) + int(rng.integers(0, 40))
        A = seeded_inputs.uniform_pm1((M, K), seeded_inputs.SEED_A + case)
        B = seeded_inputs.uniform_pm1((K, N), seeded_inputs.SEED_B + case)
        A16, B16 = A.astype(np.float16), B.astype(np.float16)
        got = run_gemm_f16(lib16[case % 3], A16, B16)
        assert not np.isnan(got).any() and normwise(got, O.hgemm_f32acc(A16, B16)) < TOL16, (case, M, N, K)
        got = run_sgemm_f32(lib32[case % 3], A, B)
        assert not np.isnan(got).any() and normwise(got, O.sgemm_seqk(A, B)) < TOL32, (case, M, N, K)
        if M <= 16:
            got = run_gemm_f16(gemv16, A16, B16)
            assert not np.isnan(got).any() and normwise(got, O.hgemm_f32acc(A16, B16)) < TOL16, (case, M, N, K)


def test_conv_random_geometries_vs_oracle():
    """Seeded random small convolutions, channel counts 1 ... 20 (implicit gather, channel-padded copies and
    column-buffer paths all occur), strides 1 ... 3, padding up to the filter size, rectangular images and
    filters: FP16 and FP32 against the oracle."""
    rng = np.random.default_rng(33)
    lib16 = [load(b16.kernel_library("gemm", 2, 64, 64, 32, 32, 64)), load(b16.kernel_library("gemm_splitK", 2, 128, 64, 64, 32, 128))]
    lib32 = [load(b32.sgemm_library(64, 64, 16, 32, 32)), load(b32.sgemm_library(32, 64, 64, 32, 32, 4))]
    for case in range(40):
        IC = int(rng.integers(1, 21))
        kH, kW = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        stride, pad = int(rng.integers(1, 4)), int(rng.integers(0, max(kH, kW)))
        H, W = int(rng.integers(kH, kH + 12)), int(rng.integers(kW, kW + 12))
        batch, OC = int(rng.integers(1, 4)), int(rng.integers(1, 41))
        if (H + 2 * pad - kH) // stride + 1 < 1 or (W + 2 * pad - kW) // stride + 1 < 1:
            continue
        x, w = seeded_inputs.conv_operands(batch, IC, H, W, OC, kH, kW)
        want = O.conv2d_nhwc(x, w, stride, pad)
        geom = (case, batch, H, W, IC, OC, kH, kW, stride, pad)
        got = run_conv(lib16[case % 2], x, w, stride, pad, torch.float16)
        assert got.shape == want.shape and not np.isnan(got).any(), geom
        assert normwise(got, want) < TOL16, geom
        x32, w32 = x.astype(np.float32), w.astype(np.float32)
        got = run_conv(lib32[case % 2], x32, w32, stride, pad, torch.float32)
        assert got.shape == want.shape and not np.isnan(got).any(), geom
        assert normwise(got, O.conv2d_nhwc(x32, w32, stride, pad)) < TOL32, geom


def test_conv_first_layers_full_size_sampled():
    """The three-channel first layers of AlexNet, GoogleNet and a VGG-style stem at batch 32 and 224 x 224 (the
    channel-padded path at its real size, corners and image borders included): sampled output pixels against
    float64, FP16 and FP32."""
    rng = np.random.default_rng(12)
    lib16 = load(b16.kernel_library("gemm", 2, 128, 64, 32, 32, 64))
    lib32 = load(b32.sgemm_library(64, 64, 16, 32, 32))
    for (batch, IC, H, W, OC, kH, kW, stride, pad) in [(32, 3, 224, 224, 96, 11, 11, 4, 0), (32, 3, 224, 224, 64, 7, 7, 2, 3),
                                                       (32, 3, 224, 224, 64, 3, 3, 1, 1)]:
        x, w = seeded_inputs.conv_operands(batch, IC, H, W, OC, kH, kW)
        _sampled_conv_check(run_conv(lib16, x, w, stride, pad, torch.float16), x, w, stride, pad, TOL16, rng)
        x32, w32 = x.astype(np.float32), w.astype(np.float32)
        _sampled_conv_check(run_conv(lib32, x32, w32, stride, pad, torch.float32), x32, w32, stride, pad, TOL32, rng)


# ---------------------------------------------------------------------------------------------
# vendor comparator libraries (rocBLAS behind the same C ABI)
# ---------------------------------------------------------------------------------------------
def test_rocblas_comparators_vs_oracle():
    """The comparator libraries map the templates' operand layouts onto rocBLAS's column-major calls; a wrong
    transpose or leading dimension fails here, before any benchmark prints a vendor column."""
    lib16 = load(b16.kernel_library("rocblas_f16"))
    for (M, N, K) in [(64, 48, 40), (300, 200, 136), (1, 7, 8), (130, 260, 1024)]:
        A, B = seeded_inputs.gemm_operands(M, N, K, np.float16)
        assert normwise(run_gemm_f16(lib16, A, B), O.hgemm_f32acc(A, B)) < TOL16, (M, N, K)
    assert lib16.info()["family"] == "rocblas_f16"
    lib32 = load(b32.kernel_library("rocblas_f32"))
    for (M, N, K) in [(64, 48, 40), (152, 132, 97), (4, 8, 3), (260, 128, 1024)]:
        A, B = seeded_inputs.gemm_operands(M, N, K, np.float32)
        assert normwise(run_sgemm_f32(lib32, A, B), O.sgemm_seqk(A, B)) < TOL32, (M, N, K)
    mn, avg, mx = lib16.bench(512, 512, 512, warmup=2, iters=3)
    assert 0 < mn <= avg <= mx


def test_miopen_comparators_vs_oracle():
    """The MIOpen comparator libraries describe the templates' layouts (NHWC activations, [OC][kH][kW][IC] weights)
    to the vendor library; a wrong dimension order or layout fails here, before any benchmark prints a vendor
    column.  FP32 tolerance 1e-4: the vendor's algorithm (picked by its own search) may not sum in k order."""
    geoms = [(2, 14, 14, 16, 24, 3, 3, 1, 1), (2, 15, 13, 8, 8, 3, 3, 2, 1), (3, 8, 8, 32, 16, 1, 1, 2, 0),
             (2, 9, 9, 64, 64, 3, 3, 1, 1)]
    for lib, dtype, tol, cast in ((load(b16.kernel_library("miopen_f16")), torch.float16, TOL16, np.float16),
                                  (load(b32.kernel_library("miopen_f32")), torch.float32, 1e-4, np.float32)):
        assert lib.info()["family"] == "miopen"
        for (batch, H, W, IC, OC, kH, kW, stride, pad) in geoms:
            x, w = seeded_inputs.conv_operands(batch, IC, H, W, OC, kH, kW)
            x, w = x.astype(cast), w.astype(cast)
            got = run_conv(lib, x, w, stride, pad, dtype)
            want = O.conv2d_nhwc(x, w, stride, pad)
            assert got.shape == want.shape
            assert not np.isnan(got).any(), (dtype, batch, H, W, IC, OC, kH, kW, stride, pad)
            assert normwise(got, want) < tol, (dtype, batch, H, W, IC, OC, kH, kW, stride, pad)
        mn, avg, mx = lib.bench_conv(2, 16, 14, 14, 24, 3, 3, 1, 1, warmup=2, iters=3)
        assert 0 < mn <= avg <= mx


# ---------------------------------------------------------------------------------------------
# FP32
# ---------------------------------------------------------------------------------------------
def test_sgemm_f32_k_partitions():
    """Problems with few output tiles and a long K are partitioned along K when the caller passes the workspace
    `helix_workspace_bytes` asks for (partial sums + fixed-order reduction), and run unpartitioned otherwise:
    both agree with the oracle, and on integer-valued inputs both are exact."""
    rng = np.random.default_rng(21)
    for cfg in [(64, 64, 32, 32, 32), (128, 128, 16, 64, 64), (32, 32, 8, 32, 32), (32, 32, 64, 32, 32, 4)]:
        lib = load(b32.sgemm_library(*cfg))
        BM, BN, BK = cfg[:3]
        for (M, N, K) in [(100, 96, 2048), (257, 129, 1000), (64, 64, 8 * BK * 8), (300, 200, 137), (33, 500, 4096),
                          (1000, 640, 900), (1500, 768, 2304)]:
            # the host scripts mirror the library's partition rule; the two must agree for the workspace to fit
            want_splits = g32.split_factor(b32.config_key(*cfg), M, N, K)
            assert lib.workspace_bytes(M, N, K) == (want_splits * M * N * 4 if want_splits > 1 else 0), (cfg, M, N, K)
            A = seeded_inputs.uniform_pm1((M, K), seeded_inputs.SEED_A)
            B = seeded_inputs.uniform_pm1((K, N), seeded_inputs.SEED_B)
            want = O.sgemm_seqk(A, B)
            for workspace in (True, False):
                got = run_sgemm_f32(lib, A, B, workspace)
                assert not np.isnan(got).any(), (cfg, M, N, K, workspace)
                assert normwise(got, want) < TOL32, (cfg, M, N, K, workspace)
            Ai = rng.integers(-3, 4, (M, K)).astype(np.float32)
            Bi = rng.integers(-3, 4, (K, N)).astype(np.float32)
            exact = (Ai.astype(np.int64) @ Bi.astype(np.int64)).astype(np.float32)
            assert np.array_equal(run_sgemm_f32(lib, Ai, Bi, True), exact), (cfg, M, N, K)
            assert np.array_equal(run_sgemm_f32(lib, Ai, Bi, False), exact), (cfg, M, N, K)


# the last three are K-group configurations (2, 4 and 8 waves per 32 x 32 wave tile, partial tiles added in LDS)
FP32_CONFIGS = [(128, 128, 16, 64, 64), (256, 128, 16, 128, 64), (32, 32, 8, 32, 32), (64, 256, 32, 32, 128),
                (128, 64, 32, 64, 32), (64, 64, 32, 32, 32, 2), (32, 64, 64, 32, 32, 4), (32, 32, 128, 32, 32, 8)]


@pytest.mark.parametrize("cfg", FP32_CONFIGS)
def test_sgemm_f32_vs_oracle(cfg):
    lib = load(b32.sgemm_library(*cfg))
    for (M, N, K) in [(256, 256, 256), (300, 200, 137), (1, 7, 3), (513, 1025, 70), (1024, 1024, 1024)]:
        A = seeded_inputs.uniform_pm1((M, K), seeded_inputs.SEED_A)
        B = seeded_inputs.uniform_pm1((K, N), seeded_inputs.SEED_B)
        got = run_sgemm_f32(lib, A, B)
        want = O.sgemm_seqk(A, B)
        assert not np.isnan(got).any(), (cfg, M, N, K)
        assert normwise(got, want) < TOL32, (cfg, M, N, K)


def test_sgemm_f32_exact_and_closed_forms():
    lib = load(b32.sgemm_library(128, 128, 16, 64, 64))
    rng = np.random.default_rng(10)
    A = rng.integers(-8, 9, (257, 300)).astype(np.float32)
    B = rng.integers(-8, 9, (300, 129)).astype(np.float32)
    assert np.array_equal(run_sgemm_f32(lib, A, B), (A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32))
    Bf = rng.standard_normal((96, 77)).astype(np.float32)
    assert np.array_equal(run_sgemm_f32(lib, np.eye(96, dtype=np.float32), Bf), Bf)
    E = np.zeros((20, 96), np.float32)
    E[3, 90] = 1
    want = np.zeros((20, 77), np.float32)
    want[3] = Bf[90]
    assert np.array_equal(run_sgemm_f32(lib, E, Bf), want)
    for f in sorted(glob.glob(os.path.join(GOLDEN, "gemm_f32_*.npz"))):
        d = np.load(f)
        assert normwise(run_sgemm_f32(lib, d["A"], d["B"]), d["C64"]) < TOL32, f
    t = torch.zeros((64, 64), dtype=torch.float32, device="cuda:0")
    assert lib.gemm(t.data_ptr(), t.data_ptr(), t.data_ptr(), 62, 64, 64, 62, 64, 64, check=False) == \
        HELIX_ERR_INVALID_VALUE   # lda % 4


def test_sgemm_f32_config1_and_large_k():
    """config 1 (1024^3, U[-1,1)) against the x86 path's result, and K = 8192 where FP32 summation order
    matters most (sequential-k CPU vs MFMA order)."""
    lib = load(b32.sgemm_library(256, 128, 16, 128, 64))
    A = seeded_inputs.uniform_pm1((1024, 1024), seeded_inputs.SEED_A)
    B = seeded_inputs.uniform_pm1((1024, 1024), seeded_inputs.SEED_B)
    want = O.x86_sch_gemm(A, B, (4, 1, 8, 16, 3, 2, 4), nthreads=8)
    assert normwise(run_sgemm_f32(lib, A, B), want) < TOL32
    A = seeded_inputs.normal((64, 8192), 0.1, seeded_inputs.SEED_A)
    B = seeded_inputs.normal((8192, 96), 0.1, seeded_inputs.SEED_B)
    assert normwise(run_sgemm_f32(lib, A, B), O.sgemm_seqk(A, B)) < TOL32


def test_conv_f32_vs_oracle():
    for cfg in [(128, 128, 16, 64, 64), (32, 32, 8, 32, 32), (64, 64, 32, 32, 32), (64, 32, 64, 32, 32, 4)]:
        lib = load(b32.sgemm_library(*cfg))
        for (batch, H, W, IC, OC, kH, kW, stride, pad) in CONV_GEOMS + CONV_GEOMS_ODD + [(2, 8, 8, 4, 8, 3, 3, 1, 1)]:
            x, w = seeded_inputs.conv_operands(batch, IC, H, W, OC, kH, kW, dtype=np.float32)
            got = run_conv(lib, x, w, stride, pad, torch.float32)
            want = O.conv2d_nhwc(x, w, stride, pad)
            assert not np.isnan(got).any(), (cfg, batch, H, W, IC, OC, kH, kW, stride, pad)
            assert normwise(got, want) < TOL32, (cfg, batch, H, W, IC, OC, kH, kW, stride, pad)


@pytest.mark.parametrize("name", ["gemv_fp32", "gemv_fp32_splitK"])
def test_gemv_f32_vs_oracle(name):
    lib = load(b32.kernel_library(name))
    for M in (1, 3, 4, 16, 17):
        for (N, K) in [(128, 256), (1000, 1028), (4096, 2048), (9001, 4)]:
            x = seeded_inputs.normal((M, K), 1.0, seeded_inputs.SEED_A)
            W = seeded_inputs.normal((K, N), 0.02, seeded_inputs.SEED_B)
            dx, dW = dev(x), dev(W.T)
            dy = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda:0")
            wsb = lib.workspace_bytes(M, N, K)
            ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda:0")
            lib.gemm(dx.data_ptr(), dW.data_ptr(), dy.data_ptr(), M, N, K, K, K, N, ws.data_ptr(), wsb)
            torch.cuda.synchronize()
            got = dy.cpu().numpy()
            assert not np.isnan(got).any(), (M, N, K)
            assert normwise(got, O.sgemm_seqk(x, W)) < TOL32, (M, N, K)


# ---------------------------------------------------------------------------------------------
# timing entry points and the host loop
# ---------------------------------------------------------------------------------------------
def test_bench_entry_points_return_sane_times():
    lib = load(b16.kernel_library("gemm", 2, 128, 128, 64, 64, 64))
    mn, avg, mx = lib.bench(1024, 1024, 1024, warmup=2, iters=5, outer=2)
    assert 0 < mn <= avg <= mx < 1e-2
    mn, avg, mx = lib.bench_conv(2, 64, 14, 14, 64, 3, 3, 1, 1, warmup=2, iters=5, outer=1)
    assert 0 < mn <= avg <= mx < 1e-2
    gv = load(b16.kernel_library("gemv"))
    mn, avg, mx = gv.bench(4, 4096, 4096, warmup=2, iters=5, outer=1, rotate_bytes=256 << 20)
    assert 0 < mn < 1e-2
    A = torch.zeros((512, 512), dtype=torch.float16, device="cuda:0")
    t = lib.gemm_timed(A.data_ptr(), A.data_ptr(), A.data_ptr(), 512, 512, 512, 512, 512, 512, warmup=1, iters=3)
    assert 0 < t < 1e-2


def test_profile_select_run_loop(tmp_path, monkeypatch):
    """build -> profile -> cost-model select -> run, on a handful of configurations."""
    from utils import helix_runtime
    from MI355X_FP16 import profile_MI355X_FP16 as p16
    from MI355X_FP16 import MI355X_FP16_gemm as g16
    from MI355X_FP16 import MI355X_FP16_conv as c16
    keys = [(2, 256, 256, 128, 128, 0, 64), (2, 128, 128, 64, 64, 0, 64), (2, 64, 64, 32, 32, 1, 64),
            (0, 1, 128, 0, 0, 0, 0), (0, 16, 128, 0, 0, 0, 0)]
    prof = {k: p16.time_config(k, warmup=1, iters=3) for k in keys}
    assert all(0 < v < 1 for v in prof.values())
    cost, tflops = g16.get_MI355X_FP16_gemm_Helix_result(prof, 2048, 2048, 2048)
    assert cost > 0 and 10 < tflops < 2600
    big_or_gemv = {k: v for k, v in prof.items() if k[0] == 0 or k[1] == 256}
    assert g16.cost_model(big_or_gemv, 1, 28672, 8192)[0] == 0          # decode shape goes to the GEMV kernel
    assert g16.cost_model(prof, 8192, 8192, 8192) == (2, 256, 256, 128, 128, 0, 64)
    cost, tflops = c16.get_MI355X_FP16_conv_Helix_result(prof, 32, 64, 56, 56, 64, 3, 3, 1, 1)
    assert cost > 0 and tflops > 1
    ms, tf, key = g16.get_MI355X_FP16_gemm_Oracle_result(prof, 1024, 1024, 1024)
    assert key in prof and tf > 1
