"""GPU parity tests that widen the coverage of test_gpu_parity.py to everything the cost model and the
exhaustive search can pick:

  * every built tile configuration (FP16 plain and split-K, FP32 incl. the K-group ones) on integer-valued
    GEMMs and convolutions, where FP32 accumulation is exact and a wrong tile, edge, schedule slot or K
    partition is an exact mismatch (each configuration is its own instruction schedule, so each is run);
  * the BERT-base M = 4096 GEMM list and the irregular 4000 x 2300 x 770 shape, FP16 and FP32, through the cost
    model's pick and through the exhaustive search's pick;
  * the decode GEMV shapes at full size for every batch and both GEMV libraries, the FP32 squares up to 8192,
    the six batch-32 convolution layers through the cost model's picks;
  * the extreme members of the op-level shape tables (1.9 M-row GNN products, K = 8 / 29 / 66, N = 1 with
    K = 500 000, a one-channel 5 x 20 filter).

Everything goes through the C ABI (ctypes -> helix_gemm / helix_conv2d) and is compared with the CPU oracle
or, at sizes the oracle cannot finish in seconds, with float64 dot products of sampled outputs.
Tolerances: FP16 in / FP32 accumulate / FP16 out 2e-2, FP32 1e-5, normwise (|got - want| <= tol * max|want|).
"""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from utils import seeded_inputs
from utils.helix_runtime import load
from utils.hip_ctypes import HELIX_ERR_UNSUPPORTED
from utils import get_benchmark_shape_list as shapes
from MI355X_FP16 import build_MI355X_FP16 as b16
from MI355X_FP16 import profile_MI355X_FP16 as p16
from MI355X_FP16 import MI355X_FP16_gemm as g16
from MI355X_FP16 import MI355X_FP16_conv as c16
from MI355X_FP32 import build_MI355X_FP32 as b32
from MI355X_FP32 import profile_MI355X_FP32 as p32
from MI355X_FP32 import MI355X_FP32_gemm as g32

from gpu_helpers import (TOL16, TOL32, dev, normwise, run_gemm_f16, run_gemm_f16_dev, run_sgemm_f32, run_sgemm_f32_dev,
                         run_gemv_f32, run_conv, sampled_gemm_error, sampled_conv_error, ensure_profiles)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def profiles():
    return ensure_profiles()


# ---------------------------------------------------------------------------------------------
# every built configuration, integer-exact
# ---------------------------------------------------------------------------------------------
FP16_TILE_KEYS = [k for k in p16.all_keys() if k[0] != 0]
FP32_TILE_KEYS = [k for k in p32.all_keys() if k[2] != 0]
CHUNK = 40


def _chunks(keys):
    return [keys[i:i + CHUNK] for i in range(0, len(keys), CHUNK)]


def _int_gemm_cases(rng, dtype):
    """(A, B, exact) with small integers; |exact| stays below 2048 so an FP16 result is exact too."""
    out = []
    for (M, N, K) in [(257, 129, 200), (70, 300, 712)]:
        A = rng.integers(-2, 3, (M, K)).astype(dtype)
        B = rng.integers(-1, 2, (K, N)).astype(dtype)
        exact = A.astype(np.int64) @ B.astype(np.int64)
        assert np.abs(exact).max() < 2048
        out.append((A, B, exact))
    return out


def _int_conv_cases(rng, dtype, channel_counts):
    """(x, w, stride, pad, exact): one small convolution per channel count, values in {-1, 0, 1}."""
    out = []
    for IC in channel_counts:
        batch, H, W, OC, kH, kW, stride, pad = (2, 7, 6, 24, 3, 3, 1, 1) if IC >= 64 else (2, 9, 8, 40, 3, 3, 2, 1)
        x = rng.integers(-1, 2, (batch, H, W, IC)).astype(dtype)
        w = rng.integers(-1, 2, (OC, kH, kW, IC)).astype(dtype)
        exact = O.conv2d_nhwc(x.astype(np.float32), w.astype(np.float32), stride, pad)
        assert np.abs(exact).max() < 2048
        out.append((x, w, stride, pad, exact))
    # a 1 x 1 filter walked pixel by pixel (the FP16 libraries run it as the plain GEMM on the activations as they lie)
    x = rng.integers(-1, 2, (3, 5, 7, 72)).astype(dtype)
    w = rng.integers(-1, 2, (40, 1, 1, 72)).astype(dtype)
    out.append((x, w, 1, 0, O.conv2d_nhwc(x.astype(np.float32), w.astype(np.float32), 1, 0)))
    return out


@pytest.mark.parametrize("keys", _chunks(FP16_TILE_KEYS), ids=lambda ks: f"{ks[0]}..")
def test_every_fp16_library_integer_exact(keys):
    """Per configuration: two ragged GEMMs (a narrow first K tile, a split-K partition with a remainder) and five
    convolutions -- IC = 128 and 64 (a K tile inside one filter tap when IC is a multiple of BLOCK_K), IC = 8
    (the general gather), IC = 3 (channel-padded copies in the workspace), and a 1 x 1 stride-1 layer."""
    rng = np.random.default_rng(100)
    gemms = _int_gemm_cases(rng, np.float16)
    convs = _int_conv_cases(rng, np.float16, (128, 64, 8, 3))
    for key in keys:
        lib = load(b16.library_for_key(key))
        for (A, B, exact) in gemms:
            got = run_gemm_f16(lib, A, B)
            assert np.array_equal(got.astype(np.int64), exact), (key, A.shape, B.shape)
        if b16.is_dtl_key(key):      # the direct-to-LDS family has no convolution entry
            t = torch.zeros(4096, dtype=torch.float16, device="cuda:0")
            assert lib.conv2d(t.data_ptr(), t.data_ptr(), t.data_ptr(), 1, 4, 4, 8, 8, 1, 1, 1, 0, check=False) == \
                HELIX_ERR_UNSUPPORTED
            continue
        for (x, w, stride, pad, exact) in convs:
            got = run_conv(lib, x, w, stride, pad, torch.float16)
            assert np.array_equal(got.astype(np.float32), exact), (key, x.shape, w.shape)


def test_many_tile_grids_integer_exact():
    """An integer-valued 4096 x 4096 x 256 GEMM: a few thousand tiles, so that workgroups of the small tiles share
    compute units and their waves arrive in whatever placement the dispatcher produces.  Every direct-to-LDS
    configuration (its wave groups and copy quarters are dealt by placement, with a placement-independent deal as
    the fallback) and every eighth register-staged one; the whole result is compared on the device with the exact
    product, which a corner block ties to int64 arithmetic on the host."""
    M = N = 4096
    K = 256
    rng = np.random.default_rng(7)
    A = rng.integers(-2, 3, (M, K)).astype(np.float16)
    Bt = rng.integers(-1, 2, (N, K)).astype(np.float16)
    dA, dBt = dev(A), dev(Bt)
    want = (dA.float() @ dBt.float().T)          # integers below 2^24: exact in FP32 in any summation order
    assert float(want.abs().max()) <= 2 * K
    corner = A[:300].astype(np.int64) @ Bt[:300].astype(np.int64).T
    assert np.array_equal(want[:300, :300].cpu().numpy().astype(np.int64), corner)
    want16 = want.half()
    dtl = [k for k in FP16_TILE_KEYS if b16.is_dtl_key(k)]
    staged = [k for k in FP16_TILE_KEYS if not b16.is_dtl_key(k)][::8]
    assert len(dtl) >= 2 and len(staged) > 30
    for key in dtl + staged:
        lib = load(b16.library_for_key(key))
        for _ in range(2):                       # twice: placements differ from launch to launch
            got = run_gemm_f16_dev(lib, dA, dBt, M, N, K, K)
            assert torch.equal(got, want16), (key, int((got != want16).sum()))


@pytest.mark.parametrize("keys", _chunks(FP32_TILE_KEYS), ids=lambda ks: f"{ks[0]}..")
def test_every_fp32_library_integer_exact(keys):
    """Per configuration: the same GEMMs with and without the K-partition workspace, and convolutions with
    IC = 64, 8 (implicit gather), 3 (channel-padded copies) and 1 (column buffer)."""
    rng = np.random.default_rng(101)
    gemms = _int_gemm_cases(rng, np.float32)
    convs = _int_conv_cases(rng, np.float32, (64, 8, 3, 1))
    for key in keys:
        lib = load(b32.library_for_key(key))
        for (A, B, exact) in gemms:
            for workspace in (True, False):
                got = run_sgemm_f32(lib, A, B, workspace)
                assert np.array_equal(got, exact.astype(np.float32)), (key, A.shape, B.shape, workspace)
        for (x, w, stride, pad, exact) in convs:
            got = run_conv(lib, x, w, stride, pad, torch.float32)
            assert np.array_equal(got, exact), (key, x.shape, w.shape)


# ---------------------------------------------------------------------------------------------
# config 5: BERT-base list and the irregular shape, cost-model pick and exhaustive-search pick
# ---------------------------------------------------------------------------------------------
BERT_SHAPES = [(shapes.BASELINE_BERT_M, n, k) for (n, k) in shapes.BASELINE_BERT_LAYER_NK] + [shapes.BASELINE_IRREGULAR_MNK]
SLAB = 256   # rows compared in full against the oracle


def _check_f16(key, dA, dBt, A, Bt, M, N, K, ld, rng, slab_want):
    lib = load(b16.library_for_key(key))
    C = run_gemm_f16_dev(lib, dA, dBt, M, N, (K + 7) // 8 * 8, ld).cpu().numpy()
    assert not np.isnan(C).any(), key
    worst, scale = sampled_gemm_error(C, A, Bt, rng, extra=[(M - 1, 0), (0, N - 1), (M // 2, N // 2)])
    assert worst < TOL16 * scale, (key, M, N, K)
    assert normwise(C[-SLAB:], slab_want) < TOL16, (key, M, N, K)


@pytest.mark.parametrize("shape", BERT_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_bert_list_f16_vs_oracle(profiles, shape):
    prof16, _ = profiles
    M, N, K = shape
    rng = np.random.default_rng(7)
    A, B = seeded_inputs.gemm_operands(M, N, K, np.float16)
    ld = (K + 7) // 8 * 8
    Ap = np.zeros((M, ld), np.float16)
    Ap[:, :K] = A
    Bt = np.zeros((N, ld), np.float16)
    Bt[:, :K] = B.T
    dA, dBt = dev(Ap), dev(Bt)
    slab_want = O.hgemm_f32acc(A[-SLAB:], B)     # the last rows: the ragged bottom tile of M = 4000
    picks = {g16.cost_model(prof16, M, N, K), g16.get_MI355X_FP16_gemm_Oracle_result(prof16, M, N, K)[2]}
    assert all(k is not None and k[0] != 0 for k in picks), picks
    for key in picks:
        _check_f16(key, dA, dBt, Ap, Bt, M, N, K, ld, rng, slab_want)


@pytest.mark.parametrize("shape", BERT_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_bert_list_f32_vs_oracle(profiles, shape):
    _, prof32 = profiles
    M, N, K = shape
    rng = np.random.default_rng(8)
    A, B = seeded_inputs.gemm_operands(M, N, K, np.float32)
    Mp, Np = (M + 3) // 4 * 4, (N + 3) // 4 * 4
    At = np.zeros((K, Mp), np.float32)
    At[:, :M] = A.T
    Bp = np.zeros((K, Np), np.float32)
    Bp[:, :N] = B
    dAt, dB = dev(At), dev(Bp)
    slab_want = O.sgemm_seqk(A[-SLAB:], B)
    Bt = np.ascontiguousarray(B.T)
    picks = {g32.cost_model(prof32, M, N, K), g32.get_MI355X_FP32_gemm_Oracle_result(prof32, M, N, K)[2]}
    assert all(k is not None and k[2] != 0 for k in picks), picks
    for key in picks:
        lib = load(b32.library_for_key(key))
        C = run_sgemm_f32_dev(lib, dAt, dB, M, N, K, Mp, Np).cpu().numpy()
        assert not np.isnan(C).any(), key
        worst, scale = sampled_gemm_error(C, A, Bt, rng, extra=[(M - 1, 0), (0, N - 1)])
        assert worst < TOL32 * scale, (key, M, N, K)
        assert normwise(C[-SLAB:], slab_want) < TOL32, (key, M, N, K)


# ---------------------------------------------------------------------------------------------
# config 2: squares at full size -- the search winners (FP16) and the FP32 squares
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("size", [2048, 4096, 8192])
def test_sgemm_f32_squares_sampled(profiles, size):
    """FP32 squares through the cost model's pick and the largest tile: sampled outputs against float64."""
    _, prof32 = profiles
    M = N = K = size
    rng = np.random.default_rng(9)
    A, B = seeded_inputs.gemm_operands(M, N, K, np.float32)
    dAt, dB = dev(A.T), dev(B)
    Bt = np.ascontiguousarray(B.T)
    for key in {g32.cost_model(prof32, M, N, K), b32.config_key(256, 256, 8, 64, 128)}:
        lib = load(b32.library_for_key(key))
        C = run_sgemm_f32_dev(lib, dAt, dB, M, N, K, M, N).cpu().numpy()
        assert not np.isnan(C).any()
        worst, scale = sampled_gemm_error(C, A, Bt, rng, extra=[(255, 256), (256, 255), (size - 1, size // 2)])
        assert worst < TOL32 * scale, (key, size)


@pytest.mark.parametrize("size", [1024, 2048, 4096])
def test_gemm_f16_squares_search_winner_sampled(profiles, size):
    """FP16 squares below the benchmark size through the exhaustive search's winner and the cost model's pick."""
    prof16, _ = profiles
    M = N = K = size
    rng = np.random.default_rng(10)
    A, B = seeded_inputs.gemm_operands(M, N, K, np.float16)
    Bt = np.ascontiguousarray(B.T)
    dA, dBt = dev(A), dev(Bt)
    for key in {g16.cost_model(prof16, M, N, K), g16.get_MI355X_FP16_gemm_Oracle_result(prof16, M, N, K)[2]}:
        lib = load(b16.library_for_key(key))
        C = run_gemm_f16_dev(lib, dA, dBt, M, N, K, K).cpu().numpy()
        assert not np.isnan(C).any()
        worst, scale = sampled_gemm_error(C, A, Bt, rng)
        assert worst < TOL16 * scale, (key, size)


# ---------------------------------------------------------------------------------------------
# config 3: every decode shape x batch x GEMV library
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("kn", shapes.BASELINE_GEMV_KN, ids=lambda kn: f"{kn[0]}x{kn[1]}")
def test_gemv_f16_decode_shapes_all_batches(profiles, kn):
    """W (K x N) streamed once per launch: M = 1, 4, 16 through libgemv, libgemv_splitK and the tile
    configuration the cost model prefers for the shape; sampled columns against float64."""
    prof16, _ = profiles
    K, N = kn
    rng = np.random.default_rng(11)
    x16, W = seeded_inputs.gemv_operands(16, N, K)
    Wt = np.ascontiguousarray(W.T)
    dW = dev(Wt)
    cols = np.concatenate([rng.integers(0, N, 200), [0, N - 1]])
    for M in shapes.BASELINE_GEMV_BATCHES:
        x = x16[:M]
        dx = dev(x)
        want = x.astype(np.float64) @ Wt[cols].astype(np.float64).T
        scale = np.abs(want).max()
        tile_keys = {k: v for k, v in prof16.items() if k[0] != 0}
        libs = [b16.kernel_library("gemv"), b16.kernel_library("gemv_splitK"),
                b16.library_for_key(g16.cost_model(tile_keys, M, N, K))]
        for path in libs:
            y = run_gemm_f16_dev(load(path), dx, dW, M, N, K, K).cpu().numpy()
            assert not np.isnan(y).any(), (path, M)
            assert np.max(np.abs(y[:, cols] - want)) < TOL16 * scale, (path, M, K, N)


# ---------------------------------------------------------------------------------------------
# config 4: the six layers through the cost model's picks
# ---------------------------------------------------------------------------------------------
def test_conv_f16_baseline_layers_cost_model_picks(profiles):
    prof16, _ = profiles
    rng = np.random.default_rng(12)
    for (batch, IC, H, W, OC, kH, kW, stride, pad) in shapes.get_baseline_conv_shape_list():
        OH, OW = (H + 2 * pad - kH) // stride + 1, (W + 2 * pad - kW) // stride + 1
        key = c16.cost_model(prof16, batch * OH * OW, OC, IC * kH * kW, IC)
        x, w = seeded_inputs.conv_operands(batch, IC, H, W, OC, kH, kW)
        for k in {key, (2, 256, 256, 128, 64, 0, 64)}:
            y = run_conv(load(b16.library_for_key(k)), x, w, stride, pad, torch.float16)
            assert not np.isnan(y).any(), k
            worst, scale = sampled_conv_error(y, x, w, stride, pad, rng)
            assert worst < TOL16 * scale, (k, batch, IC, H, W, OC, kH, kW, stride, pad)


# ---------------------------------------------------------------------------------------------
# extreme members of the op-level shape tables
# ---------------------------------------------------------------------------------------------
def _run_key_f16(key, A, B):
    """C = A B through the library of `key`; the GEMV libraries stream their second operand, so a tall-skinny
    product is run transposed (the runner swaps the same way, MI355X_FP16_gemm.run_config)."""
    lib = load(b16.library_for_key(key))
    if key[0] == 0 and A.shape[0] > B.shape[1]:
        return run_gemm_f16(lib, np.ascontiguousarray(B.T), np.ascontiguousarray(A.T)).T
    return run_gemm_f16(lib, A, B)


def _run_key_f32(key, A, B):
    lib = load(b32.library_for_key(key))
    if key[2] == 0:
        if A.shape[0] > B.shape[1]:
            return run_gemv_f32(lib, np.ascontiguousarray(B.T), np.ascontiguousarray(A.T)).T
        return run_gemv_f32(lib, A, B)
    return run_sgemm_f32(lib, A, B)


EXTREME_GEMMS = [(1889542, 16, 66), (56944, 16, 50), (43466, 16, 29), (512, 1, 500000), (7680, 1, 2560), (19717, 3, 16),
                 (2, 15360, 5120), (1949, 12288, 4096), (128, 80, 10), (2708, 7, 8)]


@pytest.mark.parametrize("shape", EXTREME_GEMMS, ids=lambda s: "x".join(map(str, s)))
def test_extreme_list_members_vs_float64(profiles, shape):
    """Largest M, smallest and largest K, N = 1 and other shapes at the edges of the op-level tables
    (utils/get_benchmark_shape_list.py), through the cost model's pick and one fixed tile configuration."""
    prof16, prof32 = profiles
    M, N, K = shape
    rng = np.random.default_rng(13)
    A, B = seeded_inputs.gemm_operands(M, N, K, np.float32)
    Bt = np.ascontiguousarray(B.T)
    A16, B16 = A.astype(np.float16), B.astype(np.float16)
    Bt16 = np.ascontiguousarray(B16.T)
    for key in {g16.cost_model(prof16, M, N, K), (2, 128, 32, 32, 32, 0, 64), (2, 64, 64, 32, 32, 1, 64)}:
        C = _run_key_f16(key, A16, B16)
        assert C.shape == (M, N) and not np.isnan(C).any(), (key, shape)
        worst, scale = sampled_gemm_error(C, A16, Bt16, rng, n=512)
        assert worst < TOL16 * scale, (key, shape)
    for key in {g32.cost_model(prof32, M, N, K), b32.config_key(64, 64, 16, 32, 32)}:
        C = _run_key_f32(key, A, B)
        assert C.shape == (M, N) and not np.isnan(C).any(), (key, shape)
        worst, scale = sampled_gemm_error(C, A, Bt, rng, n=512)
        # K = 500 000 products summed in FP32 in a different order than float64: sqrt(K) * 2^-24 ~ 4e-5
        tol = TOL32 if K <= 16384 else 2e-4
        assert worst < tol * scale, (key, shape)


def test_extreme_conv_one_channel_wide_filter(profiles):
    """DeepBench speech layer: one input channel, 5 x 20 filter, stride 2 -- 100 taps through the column-buffer
    path, and the 32-channel 5 x 10 layer behind it (a K tile spanning several taps)."""
    prof16, _ = profiles
    for (batch, IC, H, W, OC, kH, kW, stride, pad) in [(1, 1, 161, 700, 32, 5, 20, 2, 0), (2, 32, 79, 341, 32, 5, 10, 2, 0)]:
        x, w = seeded_inputs.conv_operands(batch, IC, H, W, OC, kH, kW)
        want16 = O.conv2d_nhwc(x, w, stride, pad)
        OH, OW = want16.shape[1:3]
        Kc = c16.gather_channels(IC) * kH * kW
        key = c16.cost_model(prof16, batch * OH * OW, OC, Kc, c16.gather_channels(IC))
        for k in {key, (2, 64, 64, 32, 32, 0, 64), (2, 128, 32, 32, 32, 1, 128)}:
            got = run_conv(load(b16.library_for_key(k)), x, w, stride, pad, torch.float16)
            assert got.shape == want16.shape and not np.isnan(got).any(), k
            assert normwise(got, want16) < TOL16, (k, IC, kH, kW)
        x32, w32 = x.astype(np.float32), w.astype(np.float32)
        want32 = O.conv2d_nhwc(x32, w32, stride, pad)
        for cfg in [(64, 64, 16, 32, 32), (128, 32, 32, 32, 32)]:
            path = b32.sgemm_library(*cfg)
            got = run_conv(load(path), x32, w32, stride, pad, torch.float32)
            assert normwise(got, want32) < TOL32, (cfg, IC, kH, kW)
