"""GPU tests of the search-quality and crossover scripts (the counterparts of the reference's
benchmark_Ampere_FP16_performance_comparison.py, TensorCore_CUDACore_Adaptive.py and candidate_performance_curve.py),
of the comparison-only GEMV library without MFMA, and of the command-line shim that prints the reference's
result line.  The thresholds on measured ratios are loose (timings of a few microseconds are noisy): they catch a
cost model that routes a shape to a kernel family that is clearly slower, not a few per cent.
"""
import math
import os
import subprocess
import sys

import numpy as np
import pytest

from oracle import oracle as O
from utils import seeded_inputs
from utils.helix_runtime import load
from MI355X_FP16 import build_MI355X_FP16 as b16
from MI355X_FP16 import benchmark_MI355X_FP16_performance_comparison as cmp16
from MI355X_FP16 import MFMA_VectorCore_Adaptive as adaptive
from MI355X_FP16 import candidate_performance_curve as curve

from gpu_helpers import TOL16, normwise, run_gemm_f16, ensure_profiles

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def prof16():
    return ensure_profiles()[0]


def test_performance_comparison_default_close_to_oracle(prof16):
    """Oracle / Default / Static1 / Static2 on six shapes of the op-level list: the cost model's pick (Default)
    delivers most of what the exhaustive search finds, and the restricted searches run."""
    shapes = [(1024, 1024, 1024), (476, 4096, 1024), (1949, 11008, 4096), (128, 25088, 4096), (4096, 768, 3072),
              (5124, 700, 2048)]
    ratios = []
    for (M, N, K) in shapes:
        oracle = cmp16.get_Helix_Oracle_result(prof16, M, N, K)
        default = cmp16.get_Helix_Default_result(prof16, M, N, K)
        static1 = cmp16.get_Helix_Static1_result(prof16, M, N, K)
        static2 = cmp16.get_Helix_Static2_result(prof16, M, N, K)
        assert oracle > 0 and default > 0 and static1 > 0 and static2 > 0, (M, N, K)
        ratios.append(default / oracle)
        assert default / oracle > 0.6, (M, N, K, default, oracle)
    geomean = math.exp(sum(math.log(r) for r in ratios) / len(ratios))
    assert geomean > 0.85, ratios


def test_verified_selection_is_one_of_the_ranked_candidates_and_not_slower(prof16):
    """Verified mode (GEMM and convolution): the returned configuration is one of the cost model's first few, the
    first of which is the Default pick, and its time is not clearly worse than the Default pick's."""
    from MI355X_FP16 import MI355X_FP16_gemm as g16, MI355X_FP16_conv as c16
    for (M, N, K) in [(2048, 2048, 2048), (4096, 768, 3072), (1949, 11008, 4096)]:
        ranked = g16.ranked_configs(prof16, M, N, K)
        assert len(ranked) == g16.VERIFY_TOP and ranked[0] == g16.cost_model(prof16, M, N, K)
        ms, tflops, key = g16.get_MI355X_FP16_gemm_Verified_result(prof16, M, N, K)
        assert key in ranked and tflops > 0
        default_ms = min(g16.run_config(ranked[0], M, N, K) for _ in range(2)) * 1e3
        assert ms < 1.15 * default_ms, (M, N, K, key, ms, default_ms)
    layer = (32, 64, 56, 56, 256, 1, 1, 1, 0)
    b, ic, h, w, oc, kh, kw, st, pd = layer
    Mc = b * ((h + 2 * pd - kh) // st + 1) * ((w + 2 * pd - kw) // st + 1)
    ranked = c16.ranked_configs(prof16, Mc, oc, c16.gather_channels(ic) * kh * kw, c16.gather_channels(ic))
    assert ranked[0] == c16.cost_model(prof16, Mc, oc, c16.gather_channels(ic) * kh * kw, c16.gather_channels(ic))
    ms, tflops, key = c16.get_MI355X_FP16_conv_Verified_result(prof16, *layer)
    assert key in ranked and tflops > 0
    default_ms, _ = c16.get_MI355X_FP16_conv_Helix_result(prof16, *layer)
    assert ms < 1.15 * default_ms, (key, ms, default_ms)
    assert cmp16.get_Helix_Verified_result(prof16, 1024, 1024, 1024) > 0


def test_adaptive_dispatch_follows_the_faster_family(prof16):
    """M = 1 .. 16 activation rows against 4096 x 1024 and 28672 x 8192 weights: the pick over all libraries is not
    clearly slower than the better of {GEMV library, best-predicted MFMA tile}."""
    for (N, K) in [(4096, 1024), (28672, 8192)]:
        for M in (1, 4, 8, 10, 12, 16):
            helix = adaptive.get_Helix_result(prof16, M, N, K)
            gemv = adaptive.get_gemv_result(prof16, M, N, K)
            gemm = adaptive.get_gemm_result(prof16, M, N, K)
            assert helix > 0.8 * max(gemv, gemm), (M, N, K, helix, gemv, gemm)


def test_candidate_performance_curve(prof16, capsys):
    M, N, K = curve.CURVE_SHAPES[1]
    best_id, best_config, rows = curve.get_all_candidate_performance(prof16, M, N, K)
    assert len(rows) == len(prof16) and 1 <= best_id <= len(rows) and best_config in prof16
    measured = [t for (_, _, t) in rows if t is not None]
    assert len(measured) > 200 and max(measured) > 1.0
    picked = rows[best_id - 1][2]
    assert picked is not None and picked > 0.6 * max(measured), (picked, max(measured))
    out = capsys.readouterr().out
    assert out.startswith("Best candidate id:") and "candidate id: 1, flops = " in out


def test_gemv_without_mfma_vs_oracle():
    """The comparison-only library (vector dot products and a wave reduction for every batch up to 16 rows)."""
    lib = load(b16.kernel_library("gemv_nomfma"))
    for M in (1, 8, 9, 12, 16, 17):
        for (N, K) in [(1000, 1032), (4096, 2048)]:
            x, W = seeded_inputs.gemv_operands(M, N, K)
            got = run_gemm_f16(lib, x, W)
            assert not np.isnan(got).any() and normwise(got, O.hgemm_f32acc(x, W)) < TOL16, (M, N, K)


def test_helix_run_prints_the_reference_line():
    env = dict(os.environ, PYTHONPATH=os.path.join(ROOT, "helix_amd", "scripts"))
    lib = b16.kernel_library("gemm", 2, 128, 128, 64, 64, 64)
    run = subprocess.run([sys.executable, os.path.join(ROOT, "helix_amd", "scripts", "helix_run.py"), lib, "1024", "1024",
                          "1024", "2", "5"], capture_output=True, text=True, env=env, cwd=ROOT, timeout=120)
    assert run.returncode == 0, run.stderr[-2000:]
    line = run.stdout.strip().splitlines()[-1]
    assert line.startswith("M N K =   1024   1024   1024, Time =")
    avg = float(line.split()[-8])        # the token the reference's profilers parse
    assert 1e-6 < avg < 1e-2 and line.endswith("Tflops")


def test_mfma_probe_reports_a_plausible_ceiling():
    """The MFMA-only loop: a rate between a fifth of and the whole datasheet peak, and all-zero operands (no
    data-dependent power draw) not slower than seeded ones."""
    from utils.helix_runtime import probe_library
    from utils.hip_ctypes import mfma_probe
    path = probe_library("mfma_probe")
    seeded = max(mfma_probe(path, False, warmup=2, launches=10, loops=300)[1] for _ in range(3))
    zeros = max(mfma_probe(path, True, warmup=2, launches=10, loops=300)[1] for _ in range(3))
    assert 500.0 < seeded < 2516.6 * 1.02 and 500.0 < zeros < 2516.6 * 1.02, (seeded, zeros)
    assert zeros > 0.97 * seeded, (seeded, zeros)
