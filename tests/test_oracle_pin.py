"""Pins the CPU oracle (oracle/helix_oracle.c) before anything is compared against it.

The reference has no tests, golden vectors or fixtures for this path, and its x86 path cannot run here
(it needs Apache TVM v0.12), so the oracle is pinned by what the mathematics fixes: float64 truth with
normwise bounds, closed forms (identity, all-ones, unit vectors), integer-valued inputs (exact in FP32),
pure-Python brute force on tiny cases, and library routines (numpy matmul, torch conv2d on CPU).
Each check is chosen so that a dropped term, a transposed operand or a wrong index fails it.
"""
import glob
import os

import numpy as np
import pytest
import torch

from oracle import oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
EPS32 = np.finfo(np.float32).eps


# ---------------------------------------------------------------------------------------------
# half <-> float
# ---------------------------------------------------------------------------------------------
def test_f16_to_f32_exhaustive():
    h = np.arange(65536, dtype=np.uint16).view(np.float16)
    got = O.f16_to_f32(h)
    want = h.astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_f32_to_f16_round_to_nearest_even():
    rng = np.random.default_rng(1)
    parts = [rng.standard_normal(200000).astype(np.float32) * s for s in (1e-8, 6e-8, 1e-5, 1e-3, 1.0, 100.0, 7e4)]
    # exact ties between neighbouring halves, and the subnormal / overflow boundaries
    h = np.arange(0, 0x7c00, dtype=np.uint16).view(np.float16).astype(np.float32)
    ties = (h[:-1] + h[1:]) / 2
    special = np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e30, -1e30, np.inf, -np.inf, 2.0 ** -24, 2.0 ** -25,
                        2.0 ** -25 * 1.0000001, 2.0 ** -14, 2.0 ** -14 * 0.9999], dtype=np.float32)
    x = np.concatenate(parts + [ties, -ties, special])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16)
    got = O.f32_to_f16(x)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


# ---------------------------------------------------------------------------------------------
# FP32 GEMM (sequential k)
# ---------------------------------------------------------------------------------------------
def _normwise_bound(A, B, K):
    # |fl(sum) - sum| <= K * eps * sum|a||b| for any summation order
    return K * EPS32 * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64))


@pytest.mark.parametrize("use_fma", [True, False])
@pytest.mark.parametrize("shape", [(64, 64, 64), (33, 47, 40), (1, 5, 300), (17, 1, 9)])
def test_sgemm_vs_float64(shape, use_fma):
    M, N, K = shape
    rng = np.random.default_rng(2)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    C = O.sgemm_seqk(A, B, use_fma=use_fma)
    C64 = A.astype(np.float64) @ B.astype(np.float64)
    assert np.all(np.abs(C - C64) <= _normwise_bound(A, B, K) + 1e-30)


def test_sgemm_golden_vectors():
    files = sorted(glob.glob(os.path.join(GOLDEN, "gemm_f32_*.npz")))
    assert files
    for f in files:
        d = np.load(f)
        C = O.sgemm_seqk(d["A"], d["B"])
        K = d["A"].shape[1]
        assert np.all(np.abs(C - d["C64"]) <= _normwise_bound(d["A"], d["B"], K) + 1e-30), f


def test_sgemm_closed_forms():
    rng = np.random.default_rng(3)
    B = rng.standard_normal((24, 31)).astype(np.float32)
    # identity: C == B exactly
    assert np.array_equal(O.sgemm_seqk(np.eye(24, dtype=np.float32), B), B)
    # ones @ ones == K exactly
    assert np.array_equal(O.sgemm_seqk(np.ones((5, 300), np.float32), np.ones((300, 7), np.float32)),
                          np.full((5, 7), 300, np.float32))
    # unit vector e_i e_j^T picks row j of B into row i (catches transposed operands / swapped indices)
    E = np.zeros((6, 24), np.float32)
    E[2, 17] = 1.0
    C = O.sgemm_seqk(E, B)
    want = np.zeros((6, 31), np.float32)
    want[2] = B[17]
    assert np.array_equal(C, want)
    # non-square, asymmetric integer matrices: exact in FP32, any index mix-up changes the result
    A = rng.integers(-8, 9, (13, 29)).astype(np.float32)
    Bi = rng.integers(-8, 9, (29, 11)).astype(np.float32)
    assert np.array_equal(O.sgemm_seqk(A, Bi), (A.astype(np.int64) @ Bi.astype(np.int64)).astype(np.float32))


def test_sgemm_is_sequential_k_bitwise():
    """Bit-level: the C loop equals a Python loop that adds products in ascending k with one rounding per
    step (no FMA) -- the order cpuSgemm (sgemm.cu:12-24) prescribes."""
    rng = np.random.default_rng(4)
    A = rng.uniform(-1, 1, (4, 37)).astype(np.float32)
    B = rng.uniform(-1, 1, (37, 5)).astype(np.float32)
    want = np.zeros((4, 5), np.float32)
    for m in range(4):
        for n in range(5):
            s = np.float32(0)
            for k in range(37):
                s = np.float32(s + np.float32(A[m, k] * B[k, n]))
            want[m, n] = s
    assert np.array_equal(O.sgemm_seqk(A, B, use_fma=False), want)
    # and the FMA flavour equals a loop with one rounding per multiply-add (emulated in float64: the
    # product of two floats is exact in float64, and one rounding of the float64 sum to float32 is an fma
    # except for double-rounding cases, which the chosen magnitudes keep out of reach)
    want_fma = np.zeros((4, 5), np.float32)
    for m in range(4):
        for n in range(5):
            s = np.float32(0)
            for k in range(37):
                s = np.float32(np.float64(A[m, k]) * np.float64(B[k, n]) + np.float64(s))
            want_fma[m, n] = s
    got = O.sgemm_seqk(A, B, use_fma=True)
    assert np.max(np.abs(got - want_fma)) <= EPS32  # at most one ulp-scale double-rounding difference
    assert np.mean(got == want_fma) > 0.9


# ---------------------------------------------------------------------------------------------
# FP16 in / FP32 accumulate / FP16 out
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("shape", [(64, 64, 64), (33, 47, 40), (1, 64, 520), (3, 2, 8)])
def test_hgemm_vs_numpy_and_float64(shape):
    M, N, K = shape
    rng = np.random.default_rng(5)
    A = (rng.standard_normal((M, K)) * 0.1).astype(np.float16)
    B = (rng.standard_normal((K, N)) * 0.1).astype(np.float16)
    C = O.hgemm_f32acc(A, B)
    C64 = A.astype(np.float64) @ B.astype(np.float64)
    # FP32 accumulation error + one FP16 rounding
    bound = _normwise_bound(A.astype(np.float32), B.astype(np.float32), K) + np.abs(C64) * 2.0 ** -11 + 2.0 ** -25
    assert np.all(np.abs(C.astype(np.float64) - C64) <= bound)
    # same semantic through numpy's own conversions and float32 matmul (different summation order)
    Cn = (A.astype(np.float32) @ B.astype(np.float32)).astype(np.float16)
    assert np.max(np.abs(C.astype(np.float32) - Cn.astype(np.float32))) <= np.max(np.abs(C64)) * 2.0 ** -10


def test_hgemm_golden_vectors():
    files = sorted(glob.glob(os.path.join(GOLDEN, "gemm_f16_*.npz")))
    assert files
    for f in files:
        d = np.load(f)
        C = O.hgemm_f32acc(d["A"], d["B"]).astype(np.float64)
        K = d["A"].shape[1]
        bound = (_normwise_bound(d["A"].astype(np.float32), d["B"].astype(np.float32), K)
                 + np.abs(d["C64"]) * 2.0 ** -11 + 2.0 ** -25)
        assert np.all(np.abs(C - d["C64"]) <= bound), f


def test_hgemm_closed_forms_and_accumulator_width():
    # ones @ ones == K: exact in FP16 up to 2048, and K = 4096 is still exact (power of two)
    for K in (8, 1024, 2048, 4096):
        C = O.hgemm_f32acc(np.ones((3, K), np.float16), np.ones((K, 2), np.float16))
        assert np.array_equal(C, np.full((3, 2), K, np.float16))
    # FP32 accumulation, not FP16: 2049 ones sum to 2049 in FP32 and round to 2048 only at the end, while an
    # FP16 accumulator would stall at 2048 and then adding 4 x 0.5 ... distinguishes them:
    A = np.concatenate([np.ones(2048), np.full(6, 0.5)]).astype(np.float16)[None, :]
    B = np.ones((2054, 1), np.float16)
    # exact sum 2051 -> nearest half (spacing 2 at this magnitude, tie to even) = 2052; an FP16 accumulator gives 2048
    assert O.hgemm_f32acc(A, B)[0, 0] == np.float16(2052)
    # unit vector picks a row; integer inputs are exact
    rng = np.random.default_rng(6)
    Bi = rng.integers(-4, 5, (24, 9)).astype(np.float16)
    E = np.zeros((5, 24), np.float16)
    E[3, 11] = 1
    want = np.zeros((5, 9), np.float16)
    want[3] = Bi[11]
    assert np.array_equal(O.hgemm_f32acc(E, Bi), want)
    Ai = rng.integers(-4, 5, (7, 24)).astype(np.float16)
    assert np.array_equal(O.hgemm_f32acc(Ai, Bi).astype(np.int64), Ai.astype(np.int64) @ Bi.astype(np.int64))


# ---------------------------------------------------------------------------------------------
# x86 schedules: every tiling gives the sequential-k result bit for bit
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("blk", [(1, 1, 16, 1, 1), (5, 1, 16, 3, 4), (9, 1, 64, 1, 6), (4, 1, 32, 1, 3), (3, 1, 16, 5, 2),
                                 (2, 2, 8, 2, 5)])
def test_x86_profile_kernel_equals_seqk(blk):
    m1, m2, n1, n2, k1 = blk
    rng = np.random.default_rng(7)
    M, N, K = 3 * m1 * m2, 2 * n1 * n2, 4 * k1
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    assert np.array_equal(O.x86_profile_kernel(A, B, m1, m2, n1, n2, k1), O.sgemm_seqk(A, B, use_fma=True))
    with pytest.raises(ValueError):
        O.x86_profile_kernel(A, B, M + 1, m2, n1, n2, k1)  # M is not a multiple of the block


@pytest.mark.parametrize("tiling", [(1, 1, 1, 16, 1, 1, 1), (5, 1, 4, 16, 3, 2, 7), (9, 1, 2, 64, 1, 2, 6),
                                    (4, 1, 8, 32, 1, 3, 3), (7, 1, 3, 16, 5, 1, 4), (3, 2, 2, 8, 2, 3, 5)])
@pytest.mark.parametrize("shape", [(100, 96, 70), (37, 200, 129), (1, 17, 5)])
def test_x86_sch_gemm_equals_seqk_with_padding(tiling, shape):
    M, N, K = shape
    rng = np.random.default_rng(8)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    got = O.x86_sch_gemm(A, B, tiling, nthreads=3)
    assert got.shape == (M, N)
    assert np.array_equal(got, O.sgemm_seqk(A, B, use_fma=True))


# ---------------------------------------------------------------------------------------------
# convolution
# ---------------------------------------------------------------------------------------------
def _conv_brute(x, w, stride, pad):
    B, H, W, IC = x.shape
    OC, kH, kW, _ = w.shape
    OH, OW = O.conv_out_hw(H, W, kH, kW, stride, pad)
    y = np.zeros((B, OH, OW, OC), np.float64)
    for b in range(B):
        for oh in range(OH):
            for ow in range(OW):
                for oc in range(OC):
                    s = 0.0
                    for kh in range(kH):
                        for kw in range(kW):
                            ih, iw = oh * stride - pad + kh, ow * stride - pad + kw
                            if 0 <= ih < H and 0 <= iw < W:
                                for c in range(IC):
                                    s += float(x[b, ih, iw, c]) * float(w[oc, kh, kw, c])
                    y[b, oh, ow, oc] = s
    return y


@pytest.mark.parametrize("geom", [(2, 5, 6, 3, 4, 3, 3, 1, 1), (1, 7, 5, 2, 3, 3, 2, 2, 1), (2, 4, 4, 5, 2, 1, 1, 2, 0),
                                  (1, 6, 7, 1, 2, 5, 3, 1, 2)])
def test_conv_brute_force_tiny(geom):
    B, H, W, IC, OC, kH, kW, stride, pad = geom
    rng = np.random.default_rng(9)
    x = rng.standard_normal((B, H, W, IC)).astype(np.float32)
    w = rng.standard_normal((OC, kH, kW, IC)).astype(np.float32)
    y = O.conv2d_nhwc(x, w, stride, pad)
    want = _conv_brute(x, w, stride, pad)
    assert y.shape == want.shape
    assert np.max(np.abs(y - want)) <= 1e-5 * max(1.0, np.max(np.abs(want)))


@pytest.mark.parametrize("geom", [(2, 14, 14, 16, 24, 3, 3, 1, 1), (2, 15, 13, 8, 8, 3, 3, 2, 1), (3, 8, 8, 32, 16, 1, 1, 2, 0),
                                  (1, 12, 12, 8, 8, 5, 5, 1, 2)])
def test_conv_vs_torch(geom):
    B, H, W, IC, OC, kH, kW, stride, pad = geom
    rng = np.random.default_rng(10)
    x = (rng.standard_normal((B, H, W, IC)) * 0.05).astype(np.float16)
    w = (rng.standard_normal((OC, kH, kW, IC)) * 0.05).astype(np.float16)
    y = O.conv2d_nhwc(x, w, stride, pad).astype(np.float32)
    xt = torch.from_numpy(x.astype(np.float32)).permute(0, 3, 1, 2)
    wt = torch.from_numpy(w.astype(np.float32)).permute(0, 3, 1, 2)
    want = torch.nn.functional.conv2d(xt, wt, stride=stride, padding=pad).permute(0, 2, 3, 1).numpy()
    assert y.shape == want.shape
    assert np.max(np.abs(y - want)) <= 2.0 ** -10 * np.max(np.abs(want)) + 1e-6


def test_conv_golden_vectors():
    files = sorted(glob.glob(os.path.join(GOLDEN, "conv_f16_*.npz")))
    assert files
    for f in files:
        d = np.load(f)
        y = O.conv2d_nhwc(d["x"], d["w"], int(d["stride"]), int(d["pad"])).astype(np.float64)
        assert y.shape == d["y64"].shape
        assert np.max(np.abs(y - d["y64"])) <= 2.0 ** -10 * np.max(np.abs(d["y64"])) + 1e-7, f


def test_conv_1x1_is_gemm():
    rng = np.random.default_rng(11)
    x = (rng.standard_normal((2, 6, 5, 16)) * 0.1).astype(np.float16)
    w = (rng.standard_normal((24, 1, 1, 16)) * 0.1).astype(np.float16)
    y = O.conv2d_nhwc(x, w, 1, 0)
    g = O.hgemm_f32acc(x.reshape(-1, 16), np.ascontiguousarray(w.reshape(24, 16).T))
    assert np.array_equal(y.reshape(-1, 24), g)


def test_im2col_index_map_and_composition():
    """im2col (NCHW, the reference's layout) followed by GEMM equals the direct NHWC convolution."""
    rng = np.random.default_rng(12)
    B, C, H, W, OC, k, stride, pad = 2, 3, 7, 6, 4, 3, 2, 1
    im = rng.integers(-3, 4, (B, C, H, W)).astype(np.float32)
    col = O.im2col_nchw(im, k, pad, stride)
    OH, OW = O.conv_out_hw(H, W, k, k, stride, pad)
    assert col.shape == (B, C * k * k, OH, OW)
    # brute-force index map
    for b in range(B):
        for c in range(C):
            for i in range(k):
                for j in range(k):
                    for oh in range(OH):
                        for ow in range(OW):
                            h, w_ = oh * stride - pad + i, ow * stride - pad + j
                            want = im[b, c, h, w_] if (0 <= h < H and 0 <= w_ < W) else 0.0
                            assert col[b, c * k * k + i * k + j, oh, ow] == want
    # composition: weights [OC][C][k][k] flattened over (c, i, j) times the column buffer
    wt = rng.integers(-3, 4, (OC, C, k, k)).astype(np.float32)
    y_gemm = np.stack([O.sgemm_seqk(wt.reshape(OC, -1), col[b].reshape(C * k * k, -1)) for b in range(B)])
    y_gemm = y_gemm.reshape(B, OC, OH, OW).transpose(0, 2, 3, 1)
    y_direct = O.conv2d_nhwc(np.ascontiguousarray(im.transpose(0, 2, 3, 1)),
                             np.ascontiguousarray(wt.transpose(0, 2, 3, 1)), stride, pad)
    assert np.array_equal(y_gemm, y_direct)  # integer-valued: exact in any order


# ---------------------------------------------------------------------------------------------
# x86 host logic (profile enumeration, cache-block extrapolation, tiling pick)
# ---------------------------------------------------------------------------------------------
def test_x86_register_block_enumeration():
    blocks = O.x86_register_blocks()
    assert len(blocks) == 270  # 9 * 5 * 6 (profile_x86_CPU.py:69-74)
    assert sorted({16 * n1 * n2 for (_, _, n1, n2, _) in blocks}) == [16, 32, 48, 64, 80]
    assert (1, 1, 1, 3, 1) in blocks and (9, 1, 1, 5, 6) in blocks


def test_x86_profile_with_injected_clock():
    # a clock under which every register block runs at exactly 100 GFLOP/s except M1 == 1 (50 GFLOP/s)
    def clock(M, N, K, m1, m2, n1, n2, k1):
        return 2 * M * N * K * 1e-9 / (50.0 if m1 == 1 else 100.0)

    reg, cache = O.x86_profile(peak_gflops=153, time_fn=clock)
    assert len(reg) == 8 * 5 * 6 and all(k[0] != 1 for k in reg)  # 100 > 0.6*153 > 50
    # extrapolated cache blocks: cost = t_reg / (20 * 16) * Mx * Nx (profile_x86_CPU.py:108).  The register
    # block was timed on 20 * M1 rows, so the true scaling is t_reg / 20 * Mx * Nx; the reference's extra
    # factor 16 is restated as it is (only ratios of these costs are ever used), hence 16 x 100 GFLOP/s here
    (key, cost, flops) = cache[(2 * 4, 32 * 3, 16 * 2)]
    assert abs(flops - 1600.0) < 1e-6
    # largest cache block is 256 x 256 wide at most
    assert max(k[0] for k in cache) <= 256 and max(k[1] for k in cache) <= 256


def test_x86_changed_profile_times_every_cache_block():
    # changed_profile_x86_CPU.py:101-127: each cache block is run with its register block's schedule and its own
    # extents.  A clock that charges 100 GFLOP/s to blocks narrower than 128 columns and 200 GFLOP/s from there
    # shows that the cache blocks are timed on their own (M, N, K) -- an extrapolated cost could not depend on N --
    # and that the register block's parameters are passed through.
    seen = []

    def clock(M, N, K, m1, m2, n1, n2, k1):
        seen.append((M, N, K, m1, m2, n1, n2, k1))
        return 2 * M * N * K * 1e-9 / (200.0 if N >= 128 else 100.0)

    reg, cache = O.x86_changed_profile(peak_gflops=153, time_fn=clock)
    assert len(reg) == 270                      # every register block runs at 100 > 0.6 * 153
    assert abs(cache[(8, 96, 32)][2] - 100.0) < 1e-9 and abs(cache[(8, 128, 32)][2] - 200.0) < 1e-9
    # the 48- and 80-wide register blocks are run as n1 = 16, n2 = 3 / 5 (changed_profile_x86_CPU.py:96-98)
    assert (2 * 4, 48 * 2, 16 * 3, 4, 1, 16, 3, 3) in seen and (9, 80, 16, 9, 1, 16, 5, 1) in seen
    # a cache block is K = 16 * K1 deep, a multiple of its register block in M and N, at most 256 x 256
    for (M, N, K), (key, cost, flops) in cache.items():
        assert M % key[0] == 0 and N % key[1] == 0 and K == 16 * key[2] and M <= 256 and N <= 256
    # where two register blocks give the same cache block, the cheaper one is kept (:121-125)
    def clock2(M, N, K, m1, m2, n1, n2, k1):
        return 2 * M * N * K * 1e-9 / (100.0 + m1)
    _, cache2 = O.x86_changed_profile(peak_gflops=153, time_fn=clock2)
    assert cache2[(8, 16, 16)][0] == (8, 16, 1)    # reachable from M1 = 1, 2, 4, 8: the fastest clock is M1 = 8


def test_x86_changed_profile_runs_the_real_kernel_on_cache_blocks():
    # without an injected clock the cache blocks go through the same timed kernel as the register blocks; keep the
    # run short: one repetition, and a peak so high that only the calibration path is exercised
    reg, cache = O.x86_changed_profile(peak_gflops=1e9, number=1)
    assert reg == {} and cache == {}


def test_x86_conv_is_timed_as_the_gemm_of_its_im2col_extents():
    # benchmark_x86_CPU_conv.py:123-125, checked on layers whose extents are known: ResNet-50 conv1 (7x7 s2 p3 on
    # 224^2 -> 112^2), a 3x3 s1 p1 layer (same size out), a 1x1 s2 layer (56 -> 28)
    assert O.x86_conv_gemm_extents(1, 3, 224, 224, 64, 7, 7, 2, 3) == (112 * 112, 64, 147)
    assert O.x86_conv_gemm_extents(32, 64, 56, 56, 64, 3, 3, 1, 1) == (32 * 56 * 56, 64, 576)
    assert O.x86_conv_gemm_extents(32, 256, 56, 56, 512, 1, 1, 2, 0) == (32 * 28 * 28, 512, 256)
    # and equals the extents of the NHWC convolution the oracle computes
    x = np.zeros((2, 9, 11, 4), np.float32)
    w = np.zeros((6, 3, 2, 4), np.float32)
    y = O.conv2d_nhwc(x, w, 2, 1)
    M, N, K = O.x86_conv_gemm_extents(2, 4, 9, 11, 6, 3, 2, 2, 1)
    assert (M, N, K) == (y.shape[0] * y.shape[1] * y.shape[2], y.shape[3], w[0].size)
    prof = {(64, 64, 32): ((4, 16, 2), 1.0, 100.0)}
    cost, gflops, padded, tiling, _ = O.x86_time_conv(prof, 1, 8, 10, 10, 24, 3, 3, 1, 1, num_thread=2, number=1)
    assert padded == (128, 64, 72) and tiling == (4, 1, 16, 16, 1, 4, 2)       # M = 100 -> 128, N = 24 -> 64, K = 72
    assert abs(gflops - 2 * 128 * 64 * 72 / 1e9 / cost) < 1e-6 * gflops          # GFLOP/s on the padded extents (:138)


def test_x86_model_cost_is_the_sum_over_the_list_with_repeats(monkeypatch):
    # benchmark_x86_CPU_model_level_LLM.py:187-193: one get_Helix_result per list entry, added up
    calls = []

    def fake(prof, M, N, K, num_thread=None, number=100, A=None, B=None):
        calls.append((M, N, K))
        return (M * 1e-3 + N * 1e-6, 0.0, (M, N, K), (), None)

    monkeypatch.setattr(O, "x86_time_gemm", fake)
    total = O.x86_time_model({}, [(2, 3, 4), (5, 6, 7), (2, 3, 4)])
    assert abs(total - (2 * (2e-3 + 3e-6) + (5e-3 + 6e-6))) < 1e-12
    assert sorted(calls) == [(2, 3, 4), (5, 6, 7)]


def test_x86_get_tiling_hand_cases():
    # two cache blocks; cost = t * ceil(M/Mc) * ceil(ceil(N/Nc)/threads) (benchmark_x86_CPU_gemm.py:52-54)
    prof = {(64, 64, 32): ((4, 16, 2), 1.0, 100.0), (128, 96, 48): ((8, 48, 3), 2.5, 110.0)}
    # M=N=256, 4 threads: first: 1.0*4*ceil(4/4)=4 ; second: 2.5*2*ceil(3/4)=5 -> first
    assert O.x86_get_tiling(prof, 256, 256, 256, num_thread=4) == (4, 1, 16, 16, 1, 4, 2)
    # 1 thread: first 1.0*4*4=16 ; second 2.5*2*3=15 -> second, and reg N 48 is rewritten to n1=16, n2=3
    assert O.x86_get_tiling(prof, 256, 256, 256, num_thread=1) == (8, 1, 16, 16, 3, 2, 3)
