"""CPU-only tests of the host side: template-space enumeration, artifact naming, cost models, dict and
stdout formats, dispatcher tables, and that every built library exports the whole C ABI."""
import ctypes
import glob
import math
import json
import os
import re
import subprocess
import sys

import pytest

from utils import hip_ctypes, helix_runtime, roofline
from utils import get_benchmark_shape_list as shapes
from MI355X_FP16 import build_MI355X_FP16 as b16
from MI355X_FP16 import profile_MI355X_FP16 as p16
from MI355X_FP16 import MI355X_FP16_gemm as g16
from MI355X_FP16 import MI355X_FP16_conv as c16
from MI355X_FP16 import benchmark_MI355X_FP16_performance_comparison as cmp16
from MI355X_FP32 import build_MI355X_FP32 as b32
from MI355X_FP32 import profile_MI355X_FP32 as p32
from MI355X_FP32 import MI355X_FP32_gemm as g32
from MI355X_FP32 import MI355X_FP32_conv as c32

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
N_FP16_FIT = (159, 86, 68)   # points that fit the hardware: two-stage (each with a split-K twin), three-stage, direct-to-LDS
N_FP16_CONFIGS = 106   # two-stage points the measured pruning keeps (workgroups of two waves are left out)
N_FP16_STAGES3 = 81    # three-stage points kept (wave tiles of up to 64 rows)
N_FP16_SPLITK = 62     # split-K libraries (wave tiles of up to 32 x 64)
N_FP16_DTL = 2         # direct-to-LDS family: the 256 x 256 tile with two 64-column stages, both wave layouts


# ---- enumeration ----------------------------------------------------------------------------------
def test_fp16_reference_validity_rules():
    # the four rules of build_Ampere_FP16.py:30-39 keep their meaning
    assert not b16.is_valid_config(4, 4, 128, 128, 32, 32)            # 4x4 scale
    assert not b16.is_valid_config(4, 1, 512, 128, 128, 128)          # block > 256
    assert not b16.is_valid_config(1, 1, 16, 128, 16, 128)            # wave aspect 8x
    assert not b16.is_valid_config(1, 4, 16, 256, 16, 64)             # block aspect 16x
    assert b16.is_valid_config(2, 2, 256, 256, 128, 128, 64, 2)
    # gfx950 resource rules
    assert not b16.is_valid_config(2, 2, 256, 256, 128, 128, 128, 2)  # 2 x 512 x 128 x 2 B > 160 KiB of LDS
    assert not b16.is_valid_config(2, 2, 256, 256, 128, 128, 64, 3)   # no registers for a second staging set
    assert not b16.is_valid_config(2, 2, 256, 256, 128, 128, 64, 4)   # two or three stages only
    assert b16.is_valid_config(2, 2, 128, 128, 64, 64, 64, 3)         # four waves, 64 accumulator registers each
    assert b16.is_valid_config(2, 4, 256, 256, 128, 64, 64, 2)        # 8 waves x 256 registers
    # measured pruning on top of what fits: two-wave workgroups (two stages), 128-row wave tiles with three stages,
    # split-K beyond 32 x 64 wave tiles
    assert b16.fits_hardware(1, 2, 32, 128, 32, 64, 64, 2) and not b16.is_valid_config(1, 2, 32, 128, 32, 64, 64, 2)
    assert b16.is_valid_config(1, 2, 32, 128, 32, 64, 64, 2, 1) and b16.is_valid_config(1, 2, 32, 128, 32, 64, 64, 3)
    assert b16.fits_hardware(2, 2, 256, 64, 128, 32, 64, 3) and not b16.is_valid_config(2, 2, 256, 64, 128, 32, 64, 3)
    assert b16.is_valid_config(2, 2, 128, 128, 64, 64, 64, 2) and not b16.is_valid_config(2, 2, 128, 128, 64, 64, 64, 2, 1)
    assert b16.is_valid_config(2, 2, 128, 128, 32, 64, 64, 2, 1)
    assert b16.vgpr_estimate(256, 256, 128, 128, 64) == 256 + 80 + 64 + 16
    assert b16.vgpr_estimate(256, 256, 128, 64, 64) == 128 + 80 + 32 + 16      # exactly the 256 of two waves per SIMD
    assert b16.vgpr_estimate(128, 128, 64, 64, 64, 3) == 64 + 48 + 2 * 32 + 16   # two staging sets


def test_fp16_template_space():
    cfgs = list(b16.iter_configs())
    assert len(cfgs) == N_FP16_CONFIGS + N_FP16_STAGES3 and len(set(cfgs)) == len(cfgs)
    assert sum(1 for c in cfgs if c[0] == 2) == N_FP16_CONFIGS
    for (st, br, bc, wr, wc, bk) in cfgs:
        assert br % wr == 0 and bc % wc == 0 and br <= 256 and bc <= 256
        assert st in (2, 3) and bk in (64, 128) and 2 * (br + bc) * bk * 2 <= 160 * 1024
        threads = 64 * (br // wr) * (bc // wc)
        assert threads <= 512 and (br * bk // 8) % threads == 0 and (bc * bk // 8) % threads == 0
        assert b16.vgpr_estimate(br, bc, wr, wc, bk, st) <= 512 // ((threads // 64 + 3) // 4)
        if st == 3:      # every three-stage point is a two-stage point with room for the second staging set
            assert b16.fits_hardware(br // wr, bc // wc, br, bc, wr, wc, bk, 2) and wr <= 64
        else:
            assert (br // wr) * (bc // wc) != 2
    splitk = list(b16.iter_splitk_configs())
    assert len(splitk) == N_FP16_SPLITK and all(st == 2 and wr * wc <= 32 * 64 for (st, br, bc, wr, wc, bk) in splitk)
    # the space before pruning
    fit = [(st, rs, cs, wr, wc, bk) for st in (2, 3) for wr in b16.WAVE_TILE_LIST for wc in b16.WAVE_COLS_LIST
           for rs in b16.BLOCK_SCALE_LIST for cs in b16.BLOCK_SCALE_LIST for bk in b16.BLOCK_K_LIST
           if b16.fits_hardware(rs, cs, rs * wr, cs * wc, wr, wc, bk, st)]
    assert (sum(1 for c in fit if c[0] == 2), sum(1 for c in fit if c[0] == 3)) == N_FP16_FIT[:2]
    assert (2, 256, 256, 128, 128, 64) in cfgs and (3, 256, 128, 64, 64, 64) in cfgs
    assert (3, 256, 256, 64, 128, 64) not in cfgs and (3, 256, 192, 64, 96, 64) not in cfgs
    assert (2, 32, 128, 32, 64, 64) not in cfgs and (2, 32, 128, 32, 64, 64) in splitk
    keys = p16.all_keys()
    # a three-stage point whose GEMM kernel was recorded as spilling at build time is left out of the key list
    spilling3 = sum(1 for (st, br, bc, wr, wc, bk) in cfgs
                    if st == 3 and p16.gemm_kernel_scratch((st, br, bc, wr, wc, 0, bk)) > 0)
    assert len(keys) == N_FP16_CONFIGS + N_FP16_STAGES3 - spilling3 + N_FP16_SPLITK + N_FP16_DTL + 6
    assert not any(k[0] == 3 and k[5] == 1 and not b16.is_dtl_key(k) for k in keys)    # split-K is built for two stages
    # seven fields; the direct-to-LDS family carries a trailing eighth field 1
    assert all(len(k) == (8 if b16.is_dtl_key(k) else 7) for k in keys)
    assert sum(1 for k in keys if b16.is_dtl_key(k)) == N_FP16_DTL
    assert sum(1 for k in keys if k[0] == 0) == 6   # GEMV rows are tagged by a zero first field


def test_fp16_direct_to_lds_space():
    """The K_STAGES x DIRECT_TO_LDS axes: eight waves per workgroup, a ring of stages within the 160 KiB of LDS,
    accumulators plus one K tile of fragments within 256 registers; the build keeps the 256 x 256 tile with two
    64-column stages."""
    cfgs = list(b16.iter_dtl_configs())
    assert cfgs == [(2, 256, 256, 64, 128, 64), (2, 256, 256, 128, 64, 64)] and len(cfgs) == N_FP16_DTL
    for (st, br, bc, wr, wc, bk) in cfgs:
        assert (br // wr) * (bc // wc) == 8 and br <= 256 and bc <= 256
        assert (bk, st) in b16.DTL_BK_STAGES_LIST and st * (br + bc) * bk * 2 + 64 <= 160 * 1024
        rows_per_copy = {32: 16, 64: 8}[bk]     # matrix rows one 1 KiB copy instruction fills
        assert (br // 4) % rows_per_copy == 0 and (bc // 4) % rows_per_copy == 0
        assert (bk // 32) * (wr // 16 + wc // 16) * 4 + (wr // 16) * (wc // 16) * 4 <= 236
    assert not b16.is_valid_dtl_config(2, 4, 256, 256, 128, 64, 64, 3)    # three 64-column stages of that tile exceed the LDS
    assert not b16.is_valid_dtl_config(2, 4, 128, 256, 64, 64, 64, 2)     # other tiles: pruned
    assert b16.library_for_key((2, 256, 256, 128, 64, 0, 64, 1)).endswith("build/bin_fp16/libgemm_dtl_2_256_256_128_64_64.so")
    src, out, defines = b16.compile_job("gemm_dtl", 2, 256, 256, 128, 64, 64)
    assert src.endswith("src_template/MI355X_FP16/gemm_dtl.hip") and defines["K_STAGES"] == 2 and defines["BLOCK_K"] == 64
    # no convolution entry: the conv cost model never picks the family
    d = {(2, 256, 256, 128, 64, 0, 64, 1): 1e-9, (2, 128, 128, 64, 64, 0, 64): 1.0}
    assert c16.cost_model(d, 4096, 256, 576, 64) == (2, 128, 128, 64, 64, 0, 64)
    assert g16.cost_model(d, 4096, 4096, 4096) == (2, 256, 256, 128, 64, 0, 64, 1)


def test_fp16_library_names():
    assert b16.library_for_key((2, 256, 128, 64, 64, 0, 64)).endswith("build/bin_fp16/libgemm_2_256_128_64_64_64.so")
    assert b16.library_for_key((2, 256, 128, 64, 64, 1, 64)).endswith("build/bin_fp16/libgemm_splitK_2_256_128_64_64_64.so")
    assert b16.library_for_key((0, 1, 128, 0, 0, 0, 0)).endswith("build/bin_fp16/libgemv.so")
    assert b16.library_for_key((0, 16, 128, 0, 0, 1, 0)).endswith("build/bin_fp16/libgemv_splitK.so")
    src, out, defines = b16.compile_job("gemm_splitK", 2, 128, 64, 64, 32, 64)
    assert src.endswith("src_template/MI355X_FP16/gemm.hip")
    assert defines == {"SPLIT_K": 8, "K_STAGES": 2, "BLOCK_ROWS": 128, "BLOCK_COLS": 64, "WAVE_ROWS": 64,
                       "WAVE_COLS": 32, "BLOCK_K": 64}
    cmd = helix_runtime.compile_command(src, out, defines)
    assert "--offload-arch=gfx950" in cmd and "-DBLOCK_ROWS=128" in cmd and "-shared" in cmd
    assert "-packed-fp32-ops" in cmd


def test_fp32_template_space():
    cfgs = list(b32.iter_configs())
    assert len(cfgs) == 143 and len(set(cfgs)) == 143
    for (BM, BN, BK, WM, WN) in cfgs:
        assert BM % WM == 0 and BN % WN == 0 and 32 <= BM <= 256 and 32 <= BN <= 256
        assert 64 * (BM // WM) * (BN // WN) <= 512
    # K-group configurations: 32 x 32 wave tiles, K_GROUPS waves per tile, up to 1024 threads
    kg = list(b32.iter_kgroup_configs())
    assert len(kg) == 14 and len(set(kg)) == 14
    for (BM, BN, BK, WM, WN, KG) in kg:
        assert WM == WN == 32 and KG in (2, 4, 8) and (BK // 2) % KG == 0
        assert 64 * (BM // WM) * (BN // WN) * KG <= 1024 and (KG - 1) * BM * BN * 4 <= 160 * 1024
    keys = p32.all_keys()
    assert len(keys) == 143 + 14 + 6 and len(set(keys)) == len(keys) and all(len(k) == 8 for k in keys)
    assert b32.config_key(64, 64, 16, 32, 32) == (64, 64, 16, 32, 32, 2, 1, 4)
    assert b32.config_key(32, 32, 64, 32, 32, 4) == (32, 32, 64, 32, 32, 2, 4, 4)
    assert b32.library_for_key((128, 64, 16, 64, 32, 2, 1, 4)).endswith("build/bin_fp32/libsgemm_128_64_16_64_32.so")
    assert b32.library_for_key((64, 64, 64, 32, 32, 2, 4, 4)).endswith("build/bin_fp32/libsgemm_64_64_64_32_32_kg4.so")
    assert b32.library_for_key((4, 128, 0, 0, 0, 0, 4, 4)).endswith("build/bin_fp32/libgemv_fp32.so")
    assert b32.library_for_key((4, 128, 0, 0, 0, 1, 4, 4)).endswith("build/bin_fp32/libgemv_fp32_splitK.so")


# ---- cost model ---------------------------------------------------------------------------------------
def test_fp16_cost_model_hand_cases():
    K = p16.PROFILE_K
    # 4096^2 outputs: 128x128 tiles -> 1024 blocks -> 4 rounds x 1.0; 256x128 -> 512 blocks -> 2 rounds x 1.8
    d = {(2, 128, 128, 64, 64, 0, 64): 1.0, (2, 256, 128, 64, 64, 0, 64): 1.8}
    assert g16.config_cost((2, 128, 128, 64, 64, 0, 64), 1.0, 4096, 4096, K) == pytest.approx(4.0)
    assert g16.config_cost((2, 256, 128, 64, 64, 0, 64), 1.8, 4096, 4096, K) == pytest.approx(3.6)
    assert g16.cost_model(d, 4096, 4096, K) == (2, 256, 128, 64, 64, 0, 64)
    # the quantisation is what makes the small tile win on a small problem: 300x300 -> 9 vs 4 blocks, one round each
    assert g16.cost_model(d, 300, 300, K) == (2, 128, 128, 64, 64, 0, 64)
    # round time scales with K
    assert g16.config_cost((2, 128, 128, 64, 64, 0, 64), 1.0, 4096, 4096, K // 2) == pytest.approx(2.0)
    # split-K multiplies the blocks (reference: * (k[5] + 1); here 2..8 ways, as many as fill 256 CUs) and
    # divides the K walk
    assert g16.split_factor((2, 128, 128, 64, 64, 1, 64), 128, 128, 8192) == 8
    assert g16.split_factor((2, 128, 128, 64, 64, 1, 64), 1024, 1024, 8192) == 4
    assert g16.split_factor((2, 128, 128, 64, 64, 1, 64), 8192, 8192, 8192) == 2
    assert g16.split_factor((2, 128, 128, 64, 64, 1, 64), 128, 128, 192) == 2
    assert g16.split_factor((2, 128, 128, 64, 64, 0, 64), 128, 128, 8192) == 1
    c0 = g16.config_cost((2, 128, 128, 64, 64, 0, 64), 1.0, 128, 128, 8192)
    c1 = g16.config_cost((2, 128, 128, 64, 64, 1, 64), 1.0, 128, 128, 8192)
    assert c1 < c0
    assert g16.config_cost((2, 128, 128, 64, 64, 1, 64), 1.0, 4096 * 4, 4096, K) > \
        g16.config_cost((2, 128, 128, 64, 64, 0, 64), 1.0, 4096 * 4, 4096, K) * 0.99
    # GEMV rows: a row describes problems of up to its own row count; blocks = ceil(big / 128), a proportional share of
    # a 256-block round of the part of the profiled launch beyond one launch's fixed time (GEMV_LAUNCH_FLOOR_S)
    gemv = (0, 4, 128, 0, 0, 0, 0)
    fixed, stream = g16.GEMV_LAUNCH_FLOOR_S, 2.56e-3 - g16.GEMV_LAUNCH_FLOOR_S
    assert g16.resident_share(128 * 256 * K * 2) == 1.0            # 268 MB of weights: streamed from HBM
    assert g16.config_cost(gemv, 2.56e-3, 4, 128 * 256, K) == pytest.approx(2.56e-3)
    assert g16.config_cost(gemv, 2.56e-3, 128 * 256, 3, K) == pytest.approx(2.56e-3)      # operands swap
    assert g16.config_cost(gemv, 2.56e-3, 5, 128 * 256, K) == float("inf")                # the 16-row profile row's case
    assert g16.config_cost((0, 16, 128, 0, 0, 0, 0), 2.56e-3, 17, 128 * 256, K) == float("inf")
    # weights that stay in the memory-side cache between launches take a smaller share of the profiled stream
    half = 128 * 128 * K * 2
    share = g16.resident_share(half)
    assert g16.GEMV_RESIDENT_SHARE < share < 1.0
    assert share == pytest.approx(0.45 + 0.55 * (half - 32e6) / (200e6 - 32e6))
    assert g16.config_cost(gemv, 2.56e-3, 4, 128 * 128, K) == pytest.approx(fixed + share * stream / 2)
    assert g16.resident_share(1e6) == g16.GEMV_RESIDENT_SHARE
    # five to eight rows run the eight-row tile, which gains nothing from resident weights
    wide = (0, 16, 128, 0, 0, 0, 0)
    assert g16.config_cost(wide, 2.56e-3, 8, 128 * 128, K) == pytest.approx(fixed + stream / 2)
    assert g16.config_cost(wide, 2.56e-3, 9, 128 * 128, K) == pytest.approx(g16.GEMV_MFMA_FLOOR_S + share * stream / 2)
    assert g16.config_cost(gemv, 1e-9, 1, 128, 512) == pytest.approx(g16.GEMV_LAUNCH_FLOOR_S)  # never less than a launch
    # conv never selects a GEMV row
    d2 = dict(d)
    d2[gemv] = 1e-12
    assert c16.cost_model(d2, 4096, 4096, K)[0] != 0
    assert g16.cost_model(d2, 4, 4096, K) == gemv


def test_static_cost_models():
    d = {(2, 128, 128, 64, 64, 0, 64): 1.0, (2, 64, 64, 64, 64, 0, 64): 0.4, (2, 256, 128, 64, 64, 0, 64): 1.8,
         (0, 1, 128, 0, 0, 0, 0): 1e-9}
    # Verified mode ranks with the same costs: the Default pick first, then by predicted cost
    ranked = g16.ranked_configs(d, 4096, 4096, 4096, top=3)
    assert ranked[0] == g16.cost_model(d, 4096, 4096, 4096) and len(ranked) == 3
    costs = [g16.config_cost(k, d[k], 4096, 4096, 4096, g16.short_value(d, k)) for k in ranked]
    assert costs == sorted(costs) and max(costs) <= min(g16.config_cost(k, v, 4096, 4096, 4096, g16.short_value(d, k))
                                                        for k, v in d.items() if k not in ranked)
    assert cmp16.cost_model_static1(d, 4096, 4096, 4096) == (2, 64, 64, 64, 64, 0, 64)     # only block == wave tile
    assert cmp16.cost_model_static2(d, 64, 64, 64) == (2, 256, 128, 64, 64, 0, 64)         # best time per tile area


def test_verified_selection_reports_why_no_candidate_ran(monkeypatch):
    """When every ranked candidate fails, Verified mode raises an error that carries the last failure instead of
    min() over an empty list."""
    d16 = {(2, 128, 128, 64, 64, 0, 64): 1.0, (2, 64, 64, 64, 64, 0, 64): 0.4}
    d32 = {b32.config_key(64, 64, 16, 32, 32): 1.0}

    def failing(*a, **kw):
        raise hip_ctypes.HelixError("helix_bench", 100)

    monkeypatch.setattr(g16, "run_config", failing)
    monkeypatch.setattr(g32, "run_config", failing)
    for fn, d in ((g16.get_MI355X_FP16_gemm_Verified_result, d16), (g32.get_MI355X_FP32_gemm_Verified_result, d32)):
        with pytest.raises(RuntimeError, match="ranked configurations could run 64x64x64") as info:
            fn(d, 64, 64, 64)
        assert isinstance(info.value.__cause__, hip_ctypes.HelixError) and info.value.__cause__.code == 100

    class Failing:
        def bench_conv(self, *a, **kw):
            raise hip_ctypes.HelixError("helix_bench_conv", 100)

    monkeypatch.setattr(c16, "load", lambda path: Failing())
    monkeypatch.setattr(c32, "load", lambda path: Failing())
    for fn, d in ((c16.get_MI355X_FP16_conv_Verified_result, d16), (c32.get_MI355X_FP32_conv_Verified_result, d32)):
        with pytest.raises(RuntimeError, match="ranked configurations could run this layer") as info:
            fn(d, 1, 8, 8, 8, 8, 3, 3, 1, 1)
        assert isinstance(info.value.__cause__, hip_ctypes.HelixError)


def test_fp32_cost_model_hand_cases():
    K = p32.PROFILE_K
    d = {(128, 128, 16, 64, 64, 2, 1, 4): 1.0, (256, 128, 16, 128, 64, 2, 1, 4): 1.8}
    assert g32.cost_model(d, 4096, 4096, K) == (256, 128, 16, 128, 64, 2, 1, 4)
    assert g32.cost_model(d, 300, 300, K) == (128, 128, 16, 64, 64, 2, 1, 4)
    assert g32.config_cost((128, 128, 16, 64, 64, 2, 1, 4), 1.0, 4096, 4096, 2 * K) == pytest.approx(8.0)


def test_fp16_cost_model_two_point_profile():
    """With the short-K point a round costs the line through (K_short, v_short) and (K_profile, v); a further
    round of one launch saves ROUND_OVERLAP_S of the fixed part."""
    K, Ks = p16.PROFILE_K, p16.PROFILE_K_SHORT
    small, big = (2, 32, 64, 32, 32, 0, 64), (2, 128, 256, 64, 64, 0, 64)
    # per-K slopes favour the small tile (per tile area), fixed parts favour the big one
    d = helix_runtime.ProfDict({small: 17e-6, big: 60e-6})
    d.short = {small: 4e-6, big: 8e-6}
    assert g16.round_time(17e-6, 4e-6, Ks) == pytest.approx(4e-6)
    assert g16.round_time(17e-6, 4e-6, K) == pytest.approx(17e-6)
    assert g16.round_time(17e-6, 4e-6, (K + Ks) // 2) == pytest.approx(10.5e-6)
    assert g16.round_time(17e-6, None, K // 2) == pytest.approx(8.5e-6)                 # one point: proportional
    assert g16.round_time(17e-6, 4e-6, 64) >= 1e-6                                       # never below a quarter of the short point
    # 100352 x 256 x 64 (a 1x1 convolution as GEMM): 12544 small tiles = 49 rounds, 784 big tiles = 4 rounds
    c_small = g16.config_cost(small, d[small], 100352, 256, 64, d.short[small])
    c_big = g16.config_cost(big, d[big], 100352, 256, 64, d.short[big])
    r_small, r_big = g16.round_time(17e-6, 4e-6, 64), g16.round_time(60e-6, 8e-6, 64)
    assert c_small == pytest.approx(49 * r_small - 48 * g16.ROUND_OVERLAP_S)
    assert c_big == pytest.approx(max(4 * r_big - 3 * g16.ROUND_OVERLAP_S,
                                      roofline.gemm_bytes(100352, 256, 64, 2) / (g16.TILE_HBM_SUSTAINED_FRACTION * roofline.HBM_BYTES_PER_S)))
    assert g16.cost_model(d, 100352, 256, 64) == big
    # without the short point a round is taken to cost K / K_profile of the profiled one: 49 almost free rounds
    hbm_floor = roofline.gemm_bytes(100352, 256, 64, 2) / (g16.TILE_HBM_SUSTAINED_FRACTION * roofline.HBM_BYTES_PER_S)
    assert g16.config_cost(small, d[small], 100352, 256, 64) == pytest.approx(max(49 * 17e-6 * 64 / K, hbm_floor))
    assert 49 * 17e-6 * 64 / K < hbm_floor < 49 * 17e-6 * 128 / K          # the floor binds for this shape, not for twice its K
    assert g16.config_cost(small, d[small], 100352, 256, 128) == pytest.approx(49 * 17e-6 * 128 / K)
    # conv: every column of tiles gathers its rows again
    assert c16.conv_config_cost(big, 60e-6, 4096, 512, K, 8e-6) == \
        pytest.approx(g16.config_cost(big, 60e-6, 4096, 512, K, 8e-6) * (1 + 2 * c16.GATHER_COST_PER_TILE_COLUMN))
    # a K tile spanning several filter taps (IC not a multiple of BLOCK_K) pays the per-chunk tap decomposition
    assert c16.conv_config_cost(big, 60e-6, 4096, 512, K, 8e-6, IC=big[6]) == c16.conv_config_cost(big, 60e-6, 4096, 512, K, 8e-6)
    assert c16.conv_config_cost(big, 60e-6, 4096, 512, K, 8e-6, IC=8) == pytest.approx(
        c16.conv_config_cost(big, 60e-6, 4096, 512, K, 8e-6) * (1 + c16.GENERAL_GATHER_COST_PER_64_K * big[6] / 64)
        * (1 + c16.GENERAL_GATHER_COST_PER_128_ROWS * big[1] / 128))
    # few K tiles: the gather term halves and a workgroup alone on its compute unit pays for not overlapping its phases
    assert c16.resident_workgroups(big) == 1 and c16.resident_workgroups(small) == 6
    assert c16.resident_workgroups((2, 128, 128, 64, 32, 0, 64)) == 2 and c16.resident_workgroups((2, 64, 64, 32, 32, 0, 64)) == 4
    Kshort = c16.SHORT_K_TILES * big[6]
    assert c16.conv_config_cost(big, 60e-6, 4096, 512, Kshort, 8e-6) == pytest.approx(
        g16.config_cost(big, 60e-6, 4096, 512, Kshort, 8e-6) * (1 + 2 * c16.SHORT_K_GATHER_COST_PER_TILE_COLUMN)
        * (1 + c16.SHORT_K_ALONE_COST / 1))
    assert c16.conv_config_cost(big, 60e-6, 4096, 512, Kshort + big[6], 8e-6) == pytest.approx(
        g16.config_cost(big, 60e-6, 4096, 512, Kshort + big[6], 8e-6) * (1 + 2 * c16.GATHER_COST_PER_TILE_COLUMN))
    # channel counts off the gather chunk: padded when that is at most 8/3 of the real count, else left alone
    assert [c16.gather_channels(c) for c in (1, 2, 3, 6, 8, 25, 64)] == [1, 2, 8, 8, 8, 32, 64]
    assert [c32.gather_channels(c) for c in (1, 2, 3, 6, 8, 25, 64)] == [1, 4, 4, 8, 8, 28, 64]
    # GEMV rows: 9 or more activation rows run the K-partitioned MFMA variant (higher floor); the split-K
    # GEMV library pays its reduction
    assert g16.config_cost((0, 16, 128, 0, 0, 0, 0), 1e-9, 13, 128, 512) == g16.GEMV_MFMA_FLOOR_S
    assert g16.config_cost((0, 16, 128, 0, 0, 1, 0), 1e-9, 4, 128, 512) == \
        pytest.approx(g16.GEMV_LAUNCH_FLOOR_S + g16.GEMV_SPLITK_EXTRA_S)


def test_fp32_split_factor_rule():
    key = (128, 128, 16, 32, 64, 2, 1, 4)
    # few tiles: towards 768 workgroups, at most 8, at least 256 (64 up to 32 tiles) of K per partition
    assert g32.split_factor(key, 1024, 1024, 1024) == 4          # 64 tiles
    assert g32.split_factor(key, 256, 256, 4096) == 8            # 4 tiles
    assert g32.split_factor(key, 256, 256, 200) == 3
    # more than 128 tiles: rounds of 256 workgroups x K walk; 196 tiles go five ways (four rounds of 922 instead of
    # four of 1152), 256 tiles stay whole, 784 tiles go three ways
    assert g32.split_factor(key, 6272, 512, 4608) == 5
    assert g32.split_factor(key, 2048, 2048, 2048) == 1
    assert g32.split_factor(key, 25088, 512, 4608) == 3
    assert g32.split_factor((64, 64, 32, 32, 32, 2, 1, 4), 1024, 1024, 1024) == 1
    assert g32.split_factor((4, 128, 0, 0, 0, 0, 4, 4), 4, 4096, 4096) == 1    # GEMV rows never partition here


def test_fp32_cost_model_extra_points():
    K, Ks = p32.PROFILE_K, p32.PROFILE_K_SHORT
    key = (64, 64, 16, 32, 32, 2, 1, 4)
    d = helix_runtime.ProfDict({key: 30e-6})
    d.short, d.two_rounds, d.short_two_rounds = {key: 12e-6}, {key: 48e-6}, {key: 15e-6}
    pts = g32.extra_points(d, key)
    assert pts == (12e-6, 48e-6, 15e-6)
    assert g32.extra_points({key: 1.0}, key) is None
    # one round of 256 tiles: the one-round line; 1024 x 1024 outputs with 64 x 64 tiles
    assert g32.config_cost(key, 30e-6, 1024, 1024, K, pts) == pytest.approx(30e-6)
    assert g32.config_cost(key, 30e-6, 1024, 1024, Ks, pts) == pytest.approx(12e-6)
    # four rounds at the profile K: later rounds cost the two-round increment (18 us), which is above what the
    # matrix pipes need for a round (256 tiles x 64 x 64 x 1024 x 2 flop at 0.85 of 157.3 TFLOP/s = 16.1 us)
    pipes = lambda kk: 2.0 * 256 * 64 * 64 * kk / (g32.LATER_ROUND_MFMA_FRACTION * g32.FP32_MFMA_FLOPS)
    assert pipes(K) == pytest.approx(16.06e-6, rel=1e-3)
    assert g32.config_cost(key, 30e-6, 2048, 2048, K, pts) == pytest.approx(30e-6 + 3 * 18e-6)
    # at the short K the increment (3 us) is below the pipes' time for the round (4.0 us), which then applies
    assert g32.config_cost(key, 30e-6, 2048, 2048, Ks, pts) == pytest.approx(12e-6 + 3 * pipes(Ks))
    # BK = 32 over several rounds: 5 % on top
    key32 = (64, 64, 32, 32, 32, 2, 1, 4)
    assert g32.config_cost(key32, 30e-6, 2048, 2048, K, pts) == pytest.approx((30e-6 + 3 * 18e-6) * (1 + g32.BK32_MULTI_ROUND_COST))
    assert g32.config_cost(key32, 30e-6, 1024, 1024, K, pts) == pytest.approx(30e-6)
    # a long problem on small tiles is bound by the rate the compute units take operands in
    big = g32.config_cost(key, 20e-6, 8192, 8192, 8192, (12e-6, 30e-6, 15e-6))
    assert big == pytest.approx(4.0 * 8192 ** 3 * (2 / 64) / g32.OPERAND_BYTES_PER_S)
    # the K-partitioned GEMV library pays its reduction
    assert g32.config_cost((4, 128, 0, 0, 0, 1, 4, 4), 1e-9, 2, 128, 256) == \
        pytest.approx(g32.GEMV_LAUNCH_FLOOR_S + g32.GEMV_SPLITK_EXTRA_S)


def test_build_records_kernel_resources_and_conv_skips_spilling_gathers(monkeypatch):
    """hipcc's per-kernel resource remarks are parsed at build time; the conv cost model leaves out configurations
    whose gather kernel for the layer's channel count spills registers to scratch."""
    text = (
        "gemm.hip:144:1: remark: Function Name: _ZN12_GLOBAL__N_121helix_gemm_f16_kernelILi0ELi2ELi256ELi256ELi128ELi64ELi64ELi1EEEvNS_6ParamsE [-Rpass-analysis=kernel-resource-usage]\n"
        "gemm.hip:144:1: remark:     VGPRs: 256 [-Rpass-analysis=kernel-resource-usage]\n"
        "gemm.hip:144:1: remark:     AGPRs: 0 [-Rpass-analysis=kernel-resource-usage]\n"
        "gemm.hip:144:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]\n"
        "gemm.hip:144:1: remark:     Occupancy [waves/SIMD]: 2 [-Rpass-analysis=kernel-resource-usage]\n"
        "gemm.hip:144:1: remark: Function Name: _ZN12_GLOBAL__N_121helix_gemm_f16_kernelILi2ELi2ELi256ELi256ELi128ELi64ELi64ELi1EEEvNS_6ParamsE [-Rpass-analysis=kernel-resource-usage]\n"
        "gemm.hip:144:1: remark:     VGPRs: 256 [-Rpass-analysis=kernel-resource-usage]\n"
        "gemm.hip:144:1: remark:     ScratchSize [bytes/lane]: 52 [-Rpass-analysis=kernel-resource-usage]\n")
    usage = helix_runtime.parse_resource_usage(text)
    assert len(usage) == 2
    gemm_k, conv_k = sorted(usage)
    assert usage[gemm_k] == {"vgprs": 256, "agprs": 0, "scratch": 0, "occupancy": 2} and usage[conv_k]["scratch"] == 52
    big, small = (2, 256, 256, 128, 64, 0, 64), (2, 128, 128, 64, 64, 0, 64)
    d = {big: 1e-9, small: 1.0}
    monkeypatch.setattr(c16, "kernel_resources", lambda path: usage if "256_256" in path else {})
    assert c16.conv_kernel_scratch(big, 64) == 52 and c16.conv_kernel_scratch(big, 24) == 0   # mode 2 spills, mode 1 has no record
    assert c16.cost_model(d, 100352, 256, 64, 64) == small      # the cheaper prediction is skipped: its gather spills
    assert c16.cost_model(d, 100352, 256, 72, 24) == big


def test_spilling_library_is_rebuilt_without_the_scheduler(tmp_path, monkeypatch):
    """compile_many builds a library whose kernels spill once more without the compiler's scheduler and keeps that
    build when no kernel spills more in it and the sum is smaller; a library without spills is compiled once."""
    remark = "x.hip:1:1: remark: Function Name: k%d [-Rpass-analysis=kernel-resource-usage]\n" \
             "x.hip:1:1: remark:     ScratchSize [bytes/lane]: %d [-Rpass-analysis=kernel-resource-usage]\n"
    calls = []
    scratch = {("a.so", ""): (36, 48), ("a.so", helix_runtime.NO_SCHEDULER_OPTION): (0, 28),      # improves: kept
               ("b.so", ""): (20, 8), ("b.so", helix_runtime.NO_SCHEDULER_OPTION): (0, 16),        # one kernel worse: dropped
               ("c.so", ""): (0, 0)}                                                                # no spill: one build

    def fake_compile(src, out, defines, link="", extra=""):
        name = os.path.basename(out).replace(".nosched", "")
        calls.append((name, extra))
        with open(out, "w") as f:
            f.write(extra or "default")
        s0, s1 = scratch[(name, extra)]
        return True, remark % (0, s0) + remark % (1, s1)

    monkeypatch.setattr(helix_runtime, "compile_library", fake_compile)
    jobs = [("x.hip", str(tmp_path / n), {}) for n in ("a.so", "b.so", "c.so")]
    assert helix_runtime.compile_many(jobs, max_workers=2) == []
    assert sorted(calls) == sorted([("a.so", ""), ("a.so", helix_runtime.NO_SCHEDULER_OPTION), ("b.so", ""),
                                    ("b.so", helix_runtime.NO_SCHEDULER_OPTION), ("c.so", "")])
    assert open(tmp_path / "a.so").read() == helix_runtime.NO_SCHEDULER_OPTION
    assert open(tmp_path / "b.so").read() == "default" and open(tmp_path / "c.so").read() == "default"
    assert not list(tmp_path.glob("*.nosched"))
    usage = json.load(open(helix_runtime.resource_usage_path(str(tmp_path))))
    assert usage["a.so"] == {"k0": {"scratch": 0}, "k1": {"scratch": 28}} and usage["b.so"]["k1"] == {"scratch": 8}
    assert helix_runtime.spills_less({"k": {"scratch": 0}}, {"k": {"scratch": 4}})
    assert not helix_runtime.spills_less({"k": {"scratch": 4}}, {"k": {"scratch": 4}})
    assert not helix_runtime.spills_less({"k": {"scratch": 0}}, {"j": {"scratch": 4}})


def test_fastdiv_header_matches_integer_division(tmp_path):
    """The conv gathers divide by OW, OH, IC and kW with a multiply and a shift (common/helix_fastdiv.h); the
    host half of the header is compiled and swept against `/` here."""
    exe = str(tmp_path / "fastdiv_check")
    src = os.path.join(ROOT, "tests", "cpp", "fastdiv_check.cpp")
    inc = os.path.join(ROOT, "helix_amd", "src_template", "common")
    build = subprocess.run(["hipcc", "-O2", "-w", "--offload-arch=gfx950", f"-I{inc}", src, "-o", exe],
                           capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-2000:]
    run = subprocess.run([exe], capture_output=True, text=True)
    assert run.returncode == 0 and "mismatches 0" in run.stdout, run.stdout + run.stderr


def test_padded_k():
    assert g16.padded_k(770) == 776 and g16.padded_k(768) == 768 and g16.padded_k(1) == 8


# ---- formats --------------------------------------------------------------------------------------------
def test_reference_stdout_line_token():
    line = helix_runtime.reference_line(256, 128, 4096, 1.25e-5, 1.5e-5, 2.0e-5)
    assert float(line.split()[-8]) == pytest.approx(1.5e-5)      # what profile_Ampere_FP16.py:38 parses
    assert line.startswith("M N K =    256    128   4096, Time =")
    assert line.endswith("Tflops")


def test_prof_dict_roundtrip(tmp_path, monkeypatch):
    monkeypatch.setattr(helix_runtime, "root_path", str(tmp_path))
    d = {(2, 128, 128, 64, 64, 0, 64): 1.5e-5, (0, 1, 128, 0, 0, 0, 0): float("inf")}
    helix_runtime.write_prof_dict("MI355X_FP16", d)
    text = open(tmp_path / "build" / "prof_dict" / "MI355X_FP16_cost_model.dict").read()
    assert "\n" not in text and text.startswith("{(2, 128, 128, 64, 64, 0, 64): 1.5e-05")
    # `inf` is not a Python literal: the reader evaluates the line exactly as the reference does
    # (eval(lines[0]), benchmark_Ampere_FP16_gemm.py:10-12), with inf defined
    assert "inf" in text
    assert helix_runtime.read_prof_dict("MI355X_FP16") == d
    assert helix_runtime.read_prof_dict("MI355X_FP16").short == {}
    # extra profile points travel in files of their own beside the reference's dict
    pd = helix_runtime.ProfDict(d)
    pd.short = {(2, 128, 128, 64, 64, 0, 64): 4e-6}
    pd.two_rounds = {(2, 128, 128, 64, 64, 0, 64): 2.5e-5}
    helix_runtime.write_prof_dict("MI355X_FP16", pd)
    assert open(tmp_path / "build" / "prof_dict" / "MI355X_FP16_cost_model.dict").read() == text
    back = helix_runtime.read_prof_dict("MI355X_FP16")
    assert back == d and back.short == pd.short and back.two_rounds == pd.two_rounds and back.short_two_rounds == {}
    # a profile without them removes the stale files
    helix_runtime.write_prof_dict("MI355X_FP16", d)
    assert helix_runtime.read_prof_dict("MI355X_FP16").short == {}


def test_pointwise_layers_are_ranked_as_the_gemm_they_run_as():
    """1 x 1, stride 1, no padding, channels on the gather chunk: the FP16 library runs the layer through its GEMM
    entry, so the convolution model adds no gather term and does not look at the gather kernels' registers."""
    assert c16.is_pointwise(1, 1, 1, 0) and not c16.is_pointwise(1, 1, 2, 0) and not c16.is_pointwise(3, 3, 1, 1)
    assert not c16.is_pointwise(1, 1, 1, 1)
    k = (2, 128, 128, 64, 64, 0, 64)
    assert c16.conv_config_cost(k, 60e-6, 100352, 256, 64, 8e-6, 64, pointwise=True) == \
        g16.config_cost(k, 60e-6, 100352, 256, 64, 8e-6)
    assert c16.conv_config_cost(k, 60e-6, 100352, 256, 64, 8e-6, 64) > g16.config_cost(k, 60e-6, 100352, 256, 64, 8e-6)
    d = {(2, 128, 128, 64, 64, 0, 64): 600e-6, (2, 64, 64, 32, 32, 0, 64): 220e-6, (0, 1, 128, 0, 0, 0, 0): 1e-9,
         (2, 256, 256, 64, 128, 0, 64, 1): 1e-9}    # values large enough that no floor of the model binds
    layer = (32, 64, 56, 56, 256, 1, 1, 1, 0)
    M = 32 * 56 * 56
    pick = c16.layer_cost_model(d, *layer)
    assert pick == c16.cost_model(d, M, 256, 64, 64, pointwise=True) and pick[0] != 0 and not b16.is_dtl_key(pick)
    assert pick == min((k for k in d if k[0] and not b16.is_dtl_key(k)), key=lambda k: g16.config_cost(k, d[k], M, 256, 64))
    assert c16.ranked_configs(d, M, 256, 64, 64, 12, pointwise=True)[0] == pick
    # stride 2 or channels off the chunk: the gather model
    assert c16.layer_cost_model(d, 32, 64, 56, 56, 256, 1, 1, 2, 0) == c16.cost_model(d, 32 * 28 * 28, 256, 64, 64)
    assert c16.layer_cost_model(d, 32, 3, 56, 56, 256, 1, 1, 1, 0) == c16.cost_model(d, M, 256, 8, 8)
    assert c32.layer_cost_model({b32.config_key(64, 64, 16, 32, 32): 1.0}, *layer) == b32.config_key(64, 64, 16, 32, 32)


def test_fastest_of_times_the_leaders_again():
    """First pass 2 + 5 launches each; the candidates within 10 % of its fastest (at most four) are timed again, two
    rounds of 5 + 20 in turn, and the smallest of those means decides; a candidate that cannot run is skipped."""
    calls = []
    first = {"a": 1.00, "b": 0.97, "c": 2.0, "e": 1.05, "f": 1.06, "g": 1.065}
    second = {"a": [0.95, 0.99], "b": [1.0, 0.96], "e": [1.2, 1.2], "f": [1.3, 1.3]}

    def time_config(k, warmup, iters):
        calls.append((k, warmup, iters))
        if k == "d":
            raise RuntimeError("cannot run")
        if iters == 5:
            return first[k]
        return second[k].pop(0)

    assert helix_runtime.fastest_of(["a", "b", "c", "d", "e", "f", "g"], time_config, "p") == "a"
    assert calls[:7] == [(k, 2, 5) for k in "abcdefg"]
    # b, a, e, f in first-pass order, twice round; c (beyond 10 %), g (fifth) and d (failed) are not timed again
    assert calls[7:] == [(k, 5, 20) for k in "baef"] * 2
    calls.clear()
    assert helix_runtime.fastest_of(["c", "a"], time_config, "p") == "a" and calls == [("c", 2, 5), ("a", 2, 5)]
    with pytest.raises(RuntimeError, match="none of the 1 ranked configurations could run p") as err:
        helix_runtime.fastest_of(["d"], time_config, "p")
    assert "cannot run" in str(err.value.__cause__)


def test_winner_cache_and_selection_modes(tmp_path, monkeypatch):
    """tuned_config: first meeting of a problem verifies and records, later ones read the record (also from a fresh
    process: the file), records are kept per profile (by its contents), a record the profile does not hold is verified
    again, a new profile file discards the winners file, and HELIX_SELECTION=model asks the cost model alone."""
    monkeypatch.setattr(helix_runtime, "root_path", str(tmp_path))
    monkeypatch.setattr(helix_runtime, "_winners", {})
    monkeypatch.delenv("HELIX_SELECTION", raising=False)
    a, b, c = (2, 128, 128, 64, 64, 0, 64), (2, 64, 64, 64, 64, 0, 64), (3, 128, 128, 64, 64, 0, 64)
    prof = {a: 1.0, b: 0.4}
    calls = []

    def verify(key):
        def run():
            calls.append(key)
            return key
        return run

    problem = ("gemm", 512, 512, 512)
    tag = {helix_runtime.PROFILE_TAG: helix_runtime.profile_fingerprint(prof)}
    assert helix_runtime.tuned_config("MI355X_FP16", problem, prof, lambda: a, verify(b)) == b and calls == [b]
    assert helix_runtime.tuned_config("MI355X_FP16", problem, prof, lambda: a, verify(a)) == b and calls == [b]
    text = open(helix_runtime.winners_path("MI355X_FP16")).read()
    assert text == str({**tag, problem: b}) and "\n" not in text
    monkeypatch.setattr(helix_runtime, "_winners", {})                     # a fresh process reads the file
    assert helix_runtime.tuned_config("MI355X_FP16", problem, prof, lambda: a, verify(a)) == b and calls == [b]
    assert set(helix_runtime.read_winners("MI355X_FP32", prof)) == {helix_runtime.PROFILE_TAG}      # per backend
    # winners belong to the profile they were timed under: another profile (other values, other keys) starts afresh,
    # in this process and from the file
    other = {a: 1.0, b: 0.5}
    assert helix_runtime.profile_fingerprint(other) != helix_runtime.profile_fingerprint(prof)
    assert helix_runtime.profile_fingerprint(dict(reversed(list(prof.items())))) == helix_runtime.profile_fingerprint(prof)
    assert helix_runtime.tuned_config("MI355X_FP16", problem, other, lambda: a, verify(a)) == a and calls == [b, a]
    assert problem in helix_runtime.read_winners("MI355X_FP16", other)
    monkeypatch.setattr(helix_runtime, "_winners", {})
    assert helix_runtime.tuned_config("MI355X_FP16", problem, prof, lambda: a, verify(b)) == b and calls == [b, a, b]
    # the recorded configuration is not in the profile (a hand-edited file): verified again, record replaced
    helix_runtime.read_winners("MI355X_FP16", prof)[problem] = c
    assert helix_runtime.tuned_config("MI355X_FP16", problem, prof, lambda: a, verify(a)) == a
    assert calls == [b, a, b, a] and helix_runtime.read_winners("MI355X_FP16", prof)[problem] == a
    # the cost model alone
    monkeypatch.setenv("HELIX_SELECTION", "model")
    assert helix_runtime.tuned_config("MI355X_FP16", problem, prof, lambda: b, verify(c)) == b and calls == [b, a, b, a]
    monkeypatch.setenv("HELIX_SELECTION", "fastest")
    with pytest.raises(ValueError):
        helix_runtime.selection_mode()
    monkeypatch.delenv("HELIX_SELECTION")
    # a new profile discards the winners
    helix_runtime.write_prof_dict("MI355X_FP16", prof)
    assert not os.path.exists(helix_runtime.winners_path("MI355X_FP16"))
    assert set(helix_runtime.read_winners("MI355X_FP16", prof)) == {helix_runtime.PROFILE_TAG}
    # the dispatchers' select_config goes through it: problem keys per family, candidates from the model's ranking
    monkeypatch.setattr(g16, "verified_config", lambda prof_dict, M, N, K, top=6: g16.ranked_configs(prof_dict, M, N, K, 2)[1])
    picked = g16.select_config(prof, 4096, 4096, 4096)
    assert picked == g16.ranked_configs(prof, 4096, 4096, 4096, 2)[1] != g16.cost_model(prof, 4096, 4096, 4096)
    assert helix_runtime.read_winners("MI355X_FP16", prof) == {**tag, ("gemm", 4096, 4096, 4096): picked}
    monkeypatch.setattr(c16, "verified_config", lambda prof_dict, *layer, top=6: b)
    layer = (2, 64, 14, 14, 64, 3, 3, 1, 1)
    assert c16.select_config(prof, *layer) == b
    assert helix_runtime.read_winners("MI355X_FP16", prof)[("conv",) + layer] == b
    d32 = {b32.config_key(64, 64, 16, 32, 32): 1.0, b32.config_key(128, 64, 16, 32, 32): 1.7}
    monkeypatch.setattr(g32, "verified_config", lambda prof_dict, M, N, K, top=6: b32.config_key(128, 64, 16, 32, 32))
    assert g32.select_config(d32, 1024, 1024, 1024) == b32.config_key(128, 64, 16, 32, 32)
    monkeypatch.setattr(c32, "verified_config", lambda prof_dict, *layer, top=6: b32.config_key(64, 64, 16, 32, 32))
    assert c32.select_config(d32, *layer) == b32.config_key(64, 64, 16, 32, 32)
    assert set(helix_runtime.read_winners("MI355X_FP32", d32)) == {helix_runtime.PROFILE_TAG, ("gemm", 1024, 1024, 1024),
                                                                    ("conv",) + layer}


def test_shape_lists():
    g = shapes.get_gemm_op_MNKList()
    # transformer projections x token counts, CNN fully-connected x batches, DeepBench, two-layer GCNs on 15 graphs
    assert len(g) == 60 * 16 + 8 * 10 + 84 + 5 * 2 * 15 and g[0] == (2, 1024, 1024) and g[15] == (2, 4096, 11008)
    assert g[-1] == (1888584, 2, 128) and g[60 * 16 + 8 * 10] == (5124, 700, 2048)
    assert (2708, 16, 1433) in g and (2708, 7, 16) in g and max(m for (m, _, _) in g) == 1889542
    conv_all = shapes.get_conv_op_shape_list()
    assert len(conv_all) == 17 * (5 + 56 + 16 + 20) + 107 and conv_all[0] == (1, 3, 224, 224, 96, 11, 11, 4, 0)
    alex, res, goog = shapes.get_cnn_opset_shape_List()
    assert (len(alex), len(res), len(goog)) == (17 * 5, 17 * 20, 17 * 56)
    assert all(len(s) == 9 and min(s) >= 0 for s in conv_all)
    bert, llama, gpt2 = shapes.get_llm_opset_MNKList()
    assert len(bert) == 60 * 73 and len(llama) == 60 * 4 and len(gpt2) == 60 * 96
    bb = shapes.get_baseline_bert_MNKList()
    assert len(bb) == 49 and bb[-1] == (4000, 2300, 770) and bb[0] == (4096, 2304, 768)
    flops = sum(2 * m * n * k for (m, n, k) in bb)
    assert flops == pytest.approx(695.8e9 + 14.17e9, rel=1e-3)
    conv = shapes.get_baseline_conv_shape_list()
    assert len(conv) == 6 and conv[0] == (32, 64, 56, 56, 64, 3, 3, 1, 1)
    want = [7.40, 3.29, 7.40, 7.40, 7.40, 6.58]
    for s, w in zip(conv, want):
        assert roofline.conv_flops(*s) / 1e9 == pytest.approx(w, abs=0.01)


def test_roofline_constants():
    assert roofline.FP16_MFMA_FLOPS == 2516.6e12 and roofline.FP32_MFMA_FLOPS == 157.3e12
    assert roofline.HBM_BYTES_PER_S == 8.0e12 and roofline.NUM_CU == 256
    assert roofline.gemm_bytes(1, 4096, 4096, 2) / 1e6 == pytest.approx(33.6, abs=0.05)
    assert roofline.gemm_bytes(1, 28672, 8192, 2) / 1e6 == pytest.approx(469.8, abs=0.1)
    assert roofline.gemm_flops(8192, 8192, 8192) / roofline.FP16_MFMA_FLOPS * 1e6 == pytest.approx(436.9, abs=0.1)


# ---- dispatchers --------------------------------------------------------------------------------------------
def test_dispatch_tables_resolve():
    import _dispatch
    import build_template, profile_template, changed_profile, runtime_cost, benchmark_op_level_eval, \
        benchmark_model_level_eval
    for rows in build_template.func_dict.values():
        for row in rows:
            assert callable(_dispatch.resolve(row))
    for table in (profile_template.func_dict, changed_profile.func_dict, runtime_cost.func_dict,
                  benchmark_op_level_eval.func_dict, benchmark_model_level_eval.func_dict):
        for row in table.values():
            assert callable(_dispatch.resolve(row))


def test_baseline_config_script_resolves_backend_functions():
    import benchmark_baseline_configs as bc
    for name, fp32 in (("MI355X_FP16", False), ("MI355X_FP32", True)):
        be = bc.Backend(name)
        assert be.fp32 == fp32 and be.elem_bytes == (4 if fp32 else 2)
        assert be.peak == (roofline.FP32_MFMA_FLOPS if fp32 else roofline.FP16_MFMA_FLOPS)
        assert callable(be.gemm_result) and callable(be.gemm_oracle) and callable(be.conv_result)
    be16, be32 = bc.Backend("MI355X_FP16"), bc.Backend("MI355X_FP32")
    assert be16.is_gemv_key((0, 4, 128, 0, 0, 0, 0)) and not be16.is_gemv_key((2, 32, 64, 32, 32, 0, 128))
    assert be32.is_gemv_key((4, 128, 0, 0, 0, 0, 4, 4)) and not be32.is_gemv_key((32, 64, 16, 32, 32, 2, 1, 4))
    assert be16.block_rows((2, 32, 64, 32, 32, 0, 128)) == 32 and be32.block_rows((32, 64, 16, 32, 32, 2, 1, 4)) == 32
    assert set(bc.SECTIONS) == {"square", "gemv", "conv", "bert"}
    out = subprocess.run([sys.executable, os.path.join(ROOT, "helix_amd", "scripts", "benchmark_baseline_configs.py"),
                          "-c", "nothing"], capture_output=True, text=True,
                         env=dict(os.environ, PYTHONPATH=os.path.join(ROOT, "helix_amd", "scripts")))
    assert out.returncode == 2 and "invalid choice" in out.stderr


def test_cli_unsupported_combination_message():
    env = dict(os.environ, PYTHONPATH=os.path.join(ROOT, "helix_amd", "scripts"))
    out = subprocess.run([sys.executable, os.path.join(ROOT, "helix_amd", "scripts", "benchmark_op_level_eval.py"), "-o",
                          "Conv", "-b", "MI355X_FP16", "-s", "rocblas"], capture_output=True, text=True, env=env, cwd=ROOT)
    assert out.returncode == 0 and out.stdout.strip() == "Conv MI355X_FP16 rocblas is not supported"


# ---- C ABI ------------------------------------------------------------------------------------------------------
def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "helix_abi.h")).read()
    return sorted(set(re.findall(r"^HELIX_API\s+(?:int|size_t)\s+(helix_\w+)\s*\(", text, flags=re.M)))


def test_header_matches_binding():
    assert _declared_symbols() == sorted(hip_ctypes.ABI_SYMBOLS)


def _built_libraries():
    return sorted(glob.glob(os.path.join(ROOT, "build", "bin_fp16", "*.so")) +
                  glob.glob(os.path.join(ROOT, "build", "bin_fp32", "*.so")))


def test_every_built_library_exports_the_whole_abi():
    libs = _built_libraries()
    if not libs:
        pytest.skip("kernel libraries are not built (run __graft_entry__.build())")
    want = set(_declared_symbols())
    # dlopen + dlsym only; no compute without a GPU.  A sample keeps this fast: every family, every 7th gemm
    sample = [p for p in libs if "gemv" in p or "rocblas" in p or "miopen" in p] + [p for p in libs if "_kg" in p][::5] + libs[::7]
    for path in sample:
        assert set(hip_ctypes.exported_symbols(path)) == want, path
        info = hip_ctypes.HelixLib(path).info()
        assert info["arch"] == "gfx950" and info["family"] in ("gemm_f16", "gemv_f16", "sgemm_f32", "gemv_f32", "rocblas_f16", "rocblas_f32",
                                                           "miopen")


def test_libraries_export_only_the_abi():
    """Every library carries its own copy of the tile code (same C++ names, different constants): nothing but the
    helix_* entry points may be visible to the dynamic linker, or a process holding two configurations could bind
    one library's entry points to the other's tile code."""
    libs = _built_libraries()
    if not libs:
        pytest.skip("kernel libraries are not built (run __graft_entry__.build())")
    want = set(_declared_symbols())
    for path in libs:
        out = subprocess.run(["nm", "-D", "--defined-only", path], capture_output=True, text=True, check=True).stdout
        names = {line.split()[-1] for line in out.splitlines() if line.strip()}
        # __hip_cuid_<hash>: the compilation-unit id hipcc emits; _ZSt19piecewise_construct: an empty libstdc++ tag object
        extra = {n for n in names - want if not n.startswith("__hip_cuid_") and n != "_ZSt19piecewise_construct"}
        assert not extra, (path, sorted(extra)[:5])
        assert want <= names, path


def test_probe_library_exports_what_its_header_declares():
    text = open(os.path.join(ROOT, "include", "helix_probe.h")).read()
    declared = sorted(set(re.findall(r"^HELIX_PROBE_API\s+int\s+(helix_\w+)\s*\(", text, flags=re.M)))
    assert declared == sorted(hip_ctypes.PROBE_SYMBOLS)
    path = helix_runtime.probe_library("mfma_probe")
    assert path.endswith("build/bin_probe/libmfma_probe.so")
    if not os.path.exists(path):
        pytest.skip("probe library is not built (run __graft_entry__.build())")
    out = subprocess.run(["nm", "-D", "--defined-only", path], capture_output=True, text=True, check=True).stdout
    names = {line.split()[-1] for line in out.splitlines() if line.strip()}
    assert set(declared) <= names
    assert not {n for n in names - set(declared) if not n.startswith("__hip_cuid_") and n != "_ZSt19piecewise_construct"}
    with pytest.raises(FileNotFoundError):
        hip_ctypes.mfma_probe(path + ".missing")


def test_all_expected_libraries_are_built():
    if not _built_libraries():
        pytest.skip("kernel libraries are not built (run __graft_entry__.build())")
    missing = [job[1] for job in b16.build_jobs() + b32.build_jobs() if not os.path.exists(job[1])]
    assert not missing, missing[:5]


def test_missing_library_fails_loudly(tmp_path):
    with pytest.raises(FileNotFoundError):
        hip_ctypes.HelixLib(str(tmp_path / "libgemm_nope.so"))


def test_info_matches_file_name():
    path = b16.kernel_library("gemm", 2, 256, 128, 64, 64, 64)
    if not os.path.exists(path):
        pytest.skip("kernel libraries are not built")
    info = hip_ctypes.HelixLib(path).info()
    assert (info["k_stages"], info["block_rows"], info["block_cols"], info["wave_rows"], info["wave_cols"],
            info["block_k"], info["split_k"]) == (2, 256, 128, 64, 64, 64, 1)
    assert info["threads"] == 64 * 4 * 2 and info["lds_bytes"] == 2 * (256 + 128) * 64 * 2
    # a K-group configuration: 4 waves on the one 32 x 32 wave tile
    info = hip_ctypes.HelixLib(b32.sgemm_library(32, 32, 64, 32, 32, 4)).info()
    assert (info["block_rows"], info["block_cols"], info["block_k"], info["k_groups"], info["threads"]) == (32, 32, 64, 4, 256)
    assert hip_ctypes.HelixLib(b32.sgemm_library(64, 64, 16, 32, 32)).info()["k_groups"] == 1
