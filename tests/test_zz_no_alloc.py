"""helix_gemm_static_scratch: the entry point that allocates nothing (K-partition partial sums in a fixed device
array inside the library) against helix_gemm with a caller-provided workspace -- same kernels, so the results
must be bit-identical.  Two calls in a row per library, the second on a smaller problem (the array keeps the
first call's partial sums), then the size limit and the comparator libraries' refusal."""
import numpy as np
import pytest
import torch

from utils.helix_runtime import load
from utils.hip_ctypes import HELIX_ERR_UNSUPPORTED, HELIX_ERR_WORKSPACE, STATIC_SCRATCH_BYTES
from utils import seeded_inputs
from MI355X_FP16 import build_MI355X_FP16 as b16
from MI355X_FP32 import build_MI355X_FP32 as b32

pytestmark = pytest.mark.gpu


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")


def _both_f16(lib, M, N, K):
    """(result through helix_gemm + workspace, result through helix_gemm_static_scratch, workspace bytes)."""
    A, B = seeded_inputs.gemm_operands(M, N, K, np.float16)
    dA, dBt = _dev(A), _dev(B.T)
    wsb = lib.workspace_bytes(M, N, K)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda:0")
    want = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda:0")
    got = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    lib.gemm(dA.data_ptr(), dBt.data_ptr(), want.data_ptr(), M, N, K, K, K, N, ws.data_ptr(), wsb, stream)
    lib.gemm_static_scratch(dA.data_ptr(), dBt.data_ptr(), got.data_ptr(), M, N, K, K, K, N, stream)
    torch.cuda.synchronize()
    return want, got, wsb


def _both_f32(lib, M, N, K):
    A = seeded_inputs.uniform_pm1((M, K), seeded_inputs.SEED_A)
    B = seeded_inputs.uniform_pm1((K, N), seeded_inputs.SEED_B)
    dAt, dB = _dev(A.T), _dev(B)
    wsb = lib.workspace_bytes(M, N, K)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda:0")
    want = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda:0")
    got = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    lib.gemm(dAt.data_ptr(), dB.data_ptr(), want.data_ptr(), M, N, K, M, N, N, ws.data_ptr(), wsb, stream)
    lib.gemm_static_scratch(dAt.data_ptr(), dB.data_ptr(), got.data_ptr(), M, N, K, M, N, N, stream)
    torch.cuda.synchronize()
    return want, got, wsb


def test_static_scratch_matches_workspace_path_two_calls():
    # FP16 split-K tile library, the K-partitioned FP16 GEMV, an FP32 tile library (K partitions on few-tile
    # problems): first call large, second call smaller, both bit-identical to the workspace path
    cases = [
        (load(b16.kernel_library("gemm_splitK", 2, 64, 64, 32, 32, 64)), _both_f16, [(320, 448, 4096), (130, 72, 520)]),
        (load(b16.kernel_library("gemv_splitK")), _both_f16, [(16, 4096, 8192), (3, 1000, 1032)]),
        (load(b32.sgemm_library(64, 64, 32, 32, 32)), _both_f32, [(300, 200, 4096), (100, 96, 1000)]),
    ]
    for lib, run, shapes in cases:
        used = []
        for (M, N, K) in shapes:
            want, got, wsb = run(lib, M, N, K)
            used.append(wsb)
            assert not torch.isnan(want).any() and not torch.isnan(got).any(), (lib.path, M, N, K)
            assert torch.equal(want, got), (lib.path, M, N, K)
        assert used[0] > used[1] > 0, (lib.path, used)   # the calls did go through the scratch array, second one smaller
    # a library that needs no scratch at all runs through the same entry point
    plain = load(b16.kernel_library("gemm", 2, 128, 128, 64, 64, 64))
    want, got, wsb = _both_f16(plain, 300, 200, 136)
    assert wsb == 0 and torch.equal(want, got)


def test_static_scratch_limit_and_refusals():
    lib = load(b16.kernel_library("gemm_splitK", 2, 64, 64, 32, 32, 64))
    M = N = 2048    # 1024 tiles -> the minimum two K partitions: 2 * 2048 * 2048 * 4 bytes = 32 MiB > 16 MiB
    K = 256
    assert lib.workspace_bytes(M, N, K) > STATIC_SCRATCH_BYTES
    A = torch.zeros((M, K), dtype=torch.float16, device="cuda:0")
    C = torch.full((M, N), 7.0, dtype=torch.float16, device="cuda:0")
    rc = lib.gemm_static_scratch(A.data_ptr(), A.data_ptr(), C.data_ptr(), M, N, K, K, K, N, check=False)
    torch.cuda.synchronize()
    assert rc == HELIX_ERR_WORKSPACE
    assert bool((C == 7.0).all())                      # nothing was launched
    assert lib.gemm_static_scratch(0, A.data_ptr(), C.data_ptr(), M, N, K, K, K, N, check=False) == 1
    for path in (b16.kernel_library("rocblas_f16"), b32.kernel_library("rocblas_f32")):
        assert load(path).gemm_static_scratch(A.data_ptr(), A.data_ptr(), C.data_ptr(), 64, 64, 64, K, K, N,
                                              check=False) == HELIX_ERR_UNSUPPORTED


def test_static_scratch_call_allocates_no_device_memory():
    """The property the entry point exists for: after a warm-up call (the first launch of a library loads its code
    object, scratch array included), further calls leave the device's free memory unchanged."""
    lib = load(b16.kernel_library("gemm_splitK", 2, 64, 64, 32, 32, 64))
    M, N, K = 320, 448, 4096
    A = torch.ones((M, K), dtype=torch.float16, device="cuda:0")
    B = torch.ones((N, K), dtype=torch.float16, device="cuda:0")
    C = torch.empty((M, N), dtype=torch.float16, device="cuda:0")
    assert 0 < lib.workspace_bytes(M, N, K) <= STATIC_SCRATCH_BYTES
    stream = torch.cuda.current_stream().cuda_stream
    lib.gemm_static_scratch(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, K, N, stream)   # warm-up
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for (m, n) in [(M, N), (130, 72), (M, N), (64, 448)]:
        lib.gemm_static_scratch(A.data_ptr(), B.data_ptr(), C.data_ptr(), m, n, K, K, K, N, stream)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, (free_before, free_after)
    assert bool((C[:64, :448] == K).all())
