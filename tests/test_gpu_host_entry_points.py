"""GPU tests of the host entry points the reference exposes around the kernels, run on the device through the same
functions the command-line dispatchers resolve: the cheap profile (scripts/Ampere_FP16/changed_profile_Ampere_FP16.py:17-70,
scripts/Ampere_FP32/changed_profile_Ampere_FP32.py:16-48), the selection-overhead report
(Ampere_FP16_runtime_cost.py:31-40), and the op-level and model-level wrappers, whose printed lines are the reference's
(benchmark_Ampere_FP16_gemm.py:17,23, benchmark_Ampere_FP16_conv.py:17,23, benchmark_Ampere_FP16_model_level_LLM.py:27,43,
benchmark_Ampere_FP16_model_level_CNN.py:27).  The wrappers run on short shape lists patched into their modules: the
full tables hold thousands of shapes.
"""
import importlib
import math
import os
import re
import shutil

import pytest

from utils import helix_runtime
from gpu_helpers import ensure_profiles

pytestmark = pytest.mark.gpu

BACKENDS = ["MI355X_FP16", "MI355X_FP32"]
NUMBER = r"(\d+\.\d\d)"
GEMM_SHAPES = [(512, 768, 1024), (1949, 1000, 520), (8, 4096, 4096)]
CONV_SHAPES = [(2, 64, 28, 28, 64, 3, 3, 1, 1), (4, 32, 14, 14, 48, 1, 1, 1, 0), (1, 3, 32, 32, 16, 5, 5, 2, 2)]


def module(backend, name):
    return importlib.import_module(f"{backend}.{name}")


@pytest.fixture(scope="module")
def profiles():
    prof16, prof32 = ensure_profiles()
    return {"MI355X_FP16": prof16, "MI355X_FP32": prof32}


@pytest.fixture
def saved_prof_dicts():
    """The cheap profile writes the same dict file as the full one (as in the reference): keep the full profile's
    files aside and put them back afterwards."""
    directory = os.path.dirname(helix_runtime.prof_dict_path("MI355X_FP16"))
    backup = directory + ".saved_by_test"
    if os.path.exists(backup):
        shutil.rmtree(backup)
    shutil.copytree(directory, backup)
    yield directory
    shutil.rmtree(directory)
    shutil.move(backup, directory)
    helix_runtime._winners.clear()      # winners recorded against the cheap profile are gone with its files


def is_gemv_key(backend, k):
    return k[0] == 0 if backend == "MI355X_FP16" else k[2] == 0


def scale_of(backend, k):
    """Block tile / wave tile of a key: the factor the cheap profile multiplies the base tile's time by."""
    if backend == "MI355X_FP16":
        return (k[1] // k[3]) * (k[2] // k[4])
    return (k[0] // k[3]) * (k[1] // k[4])


@pytest.mark.parametrize("backend", BACKENDS)
def test_changed_profile_against_full_profile(backend, profiles, saved_prof_dicts, capsys):
    full = profiles[backend]
    changed = module(backend, f"changed_profile_{backend}")
    got = getattr(changed, f"profile_Helix_{backend}_gemm_kernel")()
    out = capsys.readouterr().out
    assert out.startswith(f"Start profiling {backend.replace('_', ' ')} GEMM kernel ...") and "Profile finished." in out
    # the dict file on disk is the reference's one-line literal and reads back as what was returned
    with open(helix_runtime.prof_dict_path(backend)) as f:
        lines = f.readlines()
    assert len(lines) == 1
    on_disk = helix_runtime.read_prof_dict(backend)
    assert dict(on_disk) == dict(got) and len(got) > 100
    # every GEMV row is timed directly; every MFMA row is a timed base tile times its block scale
    base_ratios, scaled_ratios = [], []
    for k, v in got.items():
        assert k in full or scale_of(backend, k) >= 1, k
        if k not in full or not math.isfinite(full[k]):
            continue
        assert math.isfinite(v) and v > 0, (k, v)
        if is_gemv_key(backend, k) or scale_of(backend, k) == 1:
            base_ratios.append(v / full[k])
        else:
            scaled_ratios.append(v / full[k])
    assert len(base_ratios) >= 8 and len(scaled_ratios) > 50
    # a base tile is the same measurement in both profiles
    assert all(0.4 < r < 2.5 for r in base_ratios), sorted(base_ratios)[::max(1, len(base_ratios) // 10)]
    # a scaled value over-predicts (a tile of four wave tiles does not take four times a round of one-wave tiles) but
    # stays within the scale factor of the measurement
    srt = sorted(scaled_ratios)
    assert 0.5 < srt[len(srt) // 2] < 8.0 and srt[0] > 0.25 and srt[-1] < 20.0, (srt[0], srt[len(srt) // 2], srt[-1])
    # and the dict drives the cost model and a launch like the full one
    gemm = module(backend, f"{backend}_gemm")
    key = gemm.cost_model(on_disk, 1024, 1024, 1024)
    assert key in got
    cost, tflops = getattr(gemm, f"get_{backend}_gemm_Helix_result")(on_disk, 1024, 1024, 1024)
    assert cost > 0 and tflops > 1


@pytest.mark.parametrize("backend", BACKENDS)
def test_runtime_cost_lines(backend, profiles, capsys):
    rc = module(backend, f"{backend}_runtime_cost")
    getattr(rc, f"{backend}_runtime_cost")()
    lines = capsys.readouterr().out.strip().splitlines()
    sizes = [64, 128, 256, 512, 1024, 2048, 4096]
    assert len(lines) == len(sizes)
    for s, line in zip(sizes, lines):
        m = re.fullmatch(rf"The runtime cost of {s}x{s}x{s} is (\S+) ms, and the op cost is (\S+) ms\.", line)
        assert m, line
        lookup_ms, op_ms = float(m.group(1)), float(m.group(2))
        assert 0 < lookup_ms < 100.0, line            # one pass over a few hundred dict rows
        assert 1e-4 < op_ms < 50.0, line
    # the op cost grows with the problem: 4096^3 is 64^3 times the work of 64^3
    first = float(lines[0].split()[-2])
    last = float(lines[-1].split()[-2])
    assert last > 3 * first
    # get_Helix_runtime_cost returns (lookup ms, op ms) of the configuration the cost model picks
    lookup_ms, op_ms = rc.get_Helix_runtime_cost(profiles[backend], 512, 512, 512)
    assert 0 < lookup_ms < 100.0 and 1e-4 < op_ms < 10.0


def tflops_of(cost_ms, flops):
    return flops / 1e9 / cost_ms


@pytest.mark.parametrize("backend", BACKENDS)
def test_op_level_gemm_wrappers_print_the_reference_lines(backend, profiles, monkeypatch, capsys):
    bench = module(backend, f"benchmark_{backend}_gemm")
    monkeypatch.setattr(bench, "get_gemm_op_MNKList", lambda: list(GEMM_SHAPES))
    seen = []
    real = getattr(bench, f"get_{backend}_gemm_Helix_result")

    def recording(prof_dict, M, N, K, backend_name="hip"):
        cost, tflops = real(prof_dict, M, N, K, backend_name)
        seen.append(((M, N, K), cost, tflops))
        return cost, tflops

    monkeypatch.setattr(bench, f"get_{backend}_gemm_Helix_result", recording)
    getattr(bench, f"{backend}_Helix_op_level_GEMM_benchmark")(backend="hip")
    lines = capsys.readouterr().out.strip().splitlines()
    assert len(lines) == len(GEMM_SHAPES) == len(seen)
    for (M, N, K), line, (shape, cost, tflops) in zip(GEMM_SHAPES, lines, seen):
        assert shape == (M, N, K)
        assert line == f"{M}x{N}x{K}: Helix: {tflops:.2f} TFLOPS", line
        assert re.fullmatch(rf"{M}x{N}x{K}: Helix: {NUMBER} TFLOPS", line)
        # the runner's two return values describe the same launch: TFLOPS from the unpadded extents and the cost in ms
        assert tflops == pytest.approx(tflops_of(cost, 2.0 * M * N * K), rel=1e-9) and cost > 0
    getattr(bench, f"{backend}_rocblas_op_level_GEMM_benchmark")()
    lines = capsys.readouterr().out.strip().splitlines()
    assert len(lines) == len(GEMM_SHAPES)
    for (M, N, K), line in zip(GEMM_SHAPES, lines):
        m = re.fullmatch(rf"{M}x{N}x{K}: rocblas: {NUMBER} TFLOPS", line)
        assert m and float(m.group(1)) > 0, line
    with pytest.raises(ValueError):
        getattr(bench, f"{backend}_Helix_op_level_GEMM_benchmark")(backend="tvm")   # the only backend value is "hip"


@pytest.mark.parametrize("backend", BACKENDS)
def test_op_level_conv_wrappers_print_the_reference_lines(backend, profiles, monkeypatch, capsys):
    bench = module(backend, f"benchmark_{backend}_conv")
    monkeypatch.setattr(bench, "get_conv_op_shape_list", lambda: list(CONV_SHAPES))
    seen = []
    real = getattr(bench, f"get_{backend}_conv_Helix_result")

    def recording(prof_dict, *shape_and_backend):
        cost, tflops = real(prof_dict, *shape_and_backend)
        seen.append((tuple(shape_and_backend[:9]), cost, tflops))
        return cost, tflops

    monkeypatch.setattr(bench, f"get_{backend}_conv_Helix_result", recording)
    getattr(bench, f"{backend}_Helix_op_level_Conv_benchmark")(backend="hip")
    lines = capsys.readouterr().out.strip().splitlines()
    assert len(lines) == len(CONV_SHAPES) == len(seen)
    for shape, line, (got_shape, cost, tflops) in zip(CONV_SHAPES, lines, seen):
        assert got_shape == shape
        assert line == f"Helix: {tflops:.2f} TFLOPS" and re.fullmatch(rf"Helix: {NUMBER} TFLOPS", line), line
        batch, IC, H, W, OC, kH, kW, stride, pad = shape
        M = batch * ((H + 2 * pad - kH) // stride + 1) * ((W + 2 * pad - kW) // stride + 1)
        assert tflops == pytest.approx(tflops_of(cost, 2.0 * M * OC * IC * kH * kW), rel=1e-9) and cost > 0
    getattr(bench, f"{backend}_miopen_op_level_Conv_benchmark")()
    lines = capsys.readouterr().out.strip().splitlines()
    assert len(lines) == len(CONV_SHAPES)
    for line in lines:
        m = re.fullmatch(rf"miopen: {NUMBER} TFLOPS", line)
        assert m, line


@pytest.mark.parametrize("backend", BACKENDS)
def test_model_level_llm_wrapper_sums_the_per_shape_costs(backend, profiles, monkeypatch, capsys):
    bench = module(backend, f"benchmark_{backend}_model_level_LLM")
    bert = [(512, 768, 768)] * 3 + [(512, 3072, 768)]
    llama = [(16, 4096, 4096), (16, 11008, 4096)]
    gpt2 = [(1024, 1600, 1600), (512, 768, 768)]
    monkeypatch.setattr(bench, "get_llm_opset_MNKList", lambda: (bert, llama, gpt2))
    costs = {}
    real = getattr(bench, f"get_{backend}_gemm_Helix_result")

    def recording(prof_dict, M, N, K, backend_name="hip"):
        cost, tflops = real(prof_dict, M, N, K, backend_name)
        costs.setdefault((M, N, K), []).append(cost)
        return cost, tflops

    monkeypatch.setattr(bench, f"get_{backend}_gemm_Helix_result", recording)
    getattr(bench, f"{backend}_Helix_model_level_LLM_benchmark")(backend="hip")
    line = capsys.readouterr().out.strip().splitlines()[-1]
    m = re.fullmatch(rf"Bert: {NUMBER} ms, LLAMA2: {NUMBER} ms, GPT2: {NUMBER} ms", line)
    assert m, line
    # a shape is measured once per op-set and its cost added once per occurrence
    assert len(costs[(512, 768, 768)]) == 2 and len(costs[(512, 3072, 768)]) == 1
    want_bert = 3 * costs[(512, 768, 768)][0] + costs[(512, 3072, 768)][0]
    want_llama = costs[(16, 4096, 4096)][0] + costs[(16, 11008, 4096)][0]
    want_gpt2 = costs[(1024, 1600, 1600)][0] + costs[(512, 768, 768)][1]
    assert [m.group(1), m.group(2), m.group(3)] == [f"{want_bert:.2f}", f"{want_llama:.2f}", f"{want_gpt2:.2f}"]
    assert want_bert > 0 and want_llama > 0 and want_gpt2 > 0
    # vendor column: same line
    getattr(bench, f"{backend}_rocblas_model_level_LLM_benchmark")()
    line = capsys.readouterr().out.strip().splitlines()[-1]
    assert re.fullmatch(rf"Bert: {NUMBER} ms, LLAMA2: {NUMBER} ms, GPT2: {NUMBER} ms", line), line
    # the BERT-base list of the measured configurations: 12 layers of four GEMMs plus the irregular one
    monkeypatch.setattr(bench, "get_baseline_bert_MNKList", lambda: [(4096, 768, 768)] * 2 + [(4000, 2300, 770)])
    total = getattr(bench, f"{backend}_Helix_baseline_bert_benchmark")()
    line = capsys.readouterr().out.strip().splitlines()[-1]
    assert line == f"Bert-base (M=4096, 12 layers + 4000x2300x770): {total:.3f} ms"
    assert total == pytest.approx(2 * costs[(4096, 768, 768)][0] + costs[(4000, 2300, 770)][0], rel=1e-12)


@pytest.mark.parametrize("backend", BACKENDS)
def test_model_level_cnn_wrapper_sums_the_per_layer_costs(backend, profiles, monkeypatch, capsys):
    bench = module(backend, f"benchmark_{backend}_model_level_CNN")
    alexnet = [CONV_SHAPES[2], CONV_SHAPES[0]]
    resnet = [CONV_SHAPES[0], CONV_SHAPES[1], CONV_SHAPES[0]]
    googlenet = [CONV_SHAPES[1]]
    monkeypatch.setattr(bench, "get_cnn_opset_shape_List", lambda: (alexnet, resnet, googlenet))
    calls = []
    real = getattr(bench, f"get_{backend}_conv_Helix_result")

    def recording(prof_dict, *shape_and_backend):
        cost, tflops = real(prof_dict, *shape_and_backend)
        calls.append((tuple(shape_and_backend[:9]), cost))
        return cost, tflops

    monkeypatch.setattr(bench, f"get_{backend}_conv_Helix_result", recording)
    getattr(bench, f"{backend}_Helix_model_level_CNN_benchmark")(backend="hip")
    line = capsys.readouterr().out.strip().splitlines()[-1]
    m = re.fullmatch(rf"AlexNet: {NUMBER} ms, ResNet: {NUMBER} ms, GoogleNet: {NUMBER} ms", line)
    assert m, line
    # one call per layer, in list order, and the printed sums are the sums of those calls
    assert [s for s, _ in calls] == alexnet + resnet + googlenet
    sums = [sum(c for _, c in calls[0:2]), sum(c for _, c in calls[2:5]), sum(c for _, c in calls[5:6])]
    assert [m.group(1), m.group(2), m.group(3)] == [f"{s:.2f}" for s in sums]
    assert all(s > 0 for s in sums)
    getattr(bench, f"{backend}_miopen_model_level_CNN_benchmark")()
    line = capsys.readouterr().out.strip().splitlines()[-1]
    assert re.fullmatch(rf"AlexNet: {NUMBER} ms, ResNet: {NUMBER} ms, GoogleNet: {NUMBER} ms", line), line
