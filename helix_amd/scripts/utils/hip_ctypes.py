"""ctypes binding of the C ABI in include/helix_abi.h.

One `HelixLib` wraps one kernel-template shared library (one instantiated configuration), the
counterpart of one executable of the reference (`os.popen(f"{exe} {M} {N} {K}")`,
scripts/Ampere_FP16/profile_Ampere_FP16.py:36-38).  Loading a library that does not exist raises
FileNotFoundError: there is no CPU fallback.
"""
import ctypes
import json
import os

HELIX_OK = 0
HELIX_ERR_INVALID_VALUE = 1
HELIX_ERR_UNSUPPORTED = 801
HELIX_ERR_WORKSPACE = 2001
STATIC_SCRATCH_BYTES = 16 << 20      # HELIX_STATIC_SCRATCH_BYTES of include/helix_abi.h

ABI_SYMBOLS = (
    "helix_info",
    "helix_workspace_bytes",
    "helix_conv_workspace_bytes",
    "helix_gemm",
    "helix_gemm_static_scratch",
    "helix_conv2d",
    "helix_gemm_timed",
    "helix_conv2d_timed",
    "helix_bench",
    "helix_bench_conv",
)

_vp = ctypes.c_void_p
_i = ctypes.c_int
_sz = ctypes.c_size_t
_dp = ctypes.POINTER(ctypes.c_double)


class HelixError(RuntimeError):
    def __init__(self, fn, code):
        super().__init__(f"{fn} failed with code {code}")
        self.code = code


class HelixLib:
    def __init__(self, path):
        if not os.path.exists(path):
            raise FileNotFoundError(
                f"kernel library {path} is not built; run build_template.py (or __graft_entry__.build()) first")
        self.path = path
        L = ctypes.CDLL(path)
        L.helix_info.argtypes = [ctypes.c_char_p, _i]
        L.helix_info.restype = _i
        L.helix_workspace_bytes.argtypes = [_i, _i, _i]
        L.helix_workspace_bytes.restype = _sz
        L.helix_conv_workspace_bytes.argtypes = [_i] * 9
        L.helix_conv_workspace_bytes.restype = _sz
        L.helix_gemm.argtypes = [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp]
        L.helix_gemm.restype = _i
        L.helix_gemm_static_scratch.argtypes = [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp]
        L.helix_gemm_static_scratch.restype = _i
        L.helix_conv2d.argtypes = [_vp, _vp, _vp] + [_i] * 9 + [_vp, _sz, _vp]
        L.helix_conv2d.restype = _i
        L.helix_gemm_timed.argtypes = [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp, _i, _i, _dp]
        L.helix_gemm_timed.restype = _i
        L.helix_conv2d_timed.argtypes = [_vp, _vp, _vp] + [_i] * 9 + [_vp, _sz, _vp, _i, _i, _dp]
        L.helix_conv2d_timed.restype = _i
        L.helix_bench.argtypes = [_i, _i, _i, _i, _i, _i, _sz, _dp, _dp, _dp]
        L.helix_bench.restype = _i
        L.helix_bench_conv.argtypes = [_i] * 12 + [_dp, _dp, _dp]
        L.helix_bench_conv.restype = _i
        self._lib = L
        self._info = None

    # -- metadata ---------------------------------------------------------------------------------
    def info(self):
        if self._info is None:
            need = self._lib.helix_info(None, 0)
            buf = ctypes.create_string_buffer(need)
            self._lib.helix_info(buf, need)
            self._info = json.loads(buf.value.decode())
        return self._info

    def workspace_bytes(self, M, N, K):
        return int(self._lib.helix_workspace_bytes(M, N, K))

    def conv_workspace_bytes(self, batch, H, W, IC, OC, kH, kW, stride, pad):
        return int(self._lib.helix_conv_workspace_bytes(batch, H, W, IC, OC, kH, kW, stride, pad))

    # -- launches (raw device pointers as ints) -------------------------------------------------------
    def gemm(self, A, B, C, M, N, K, lda, ldb, ldc, ws=0, ws_bytes=0, stream=0, check=True):
        rc = self._lib.helix_gemm(A, B, C, M, N, K, lda, ldb, ldc, ws or None, ws_bytes, stream or None)
        if check and rc != 0:
            raise HelixError("helix_gemm", rc)
        return rc

    def gemm_static_scratch(self, A, B, C, M, N, K, lda, ldb, ldc, stream=0, check=True):
        """helix_gemm without a workspace argument and without any allocation: K-partition partial sums go to
        the library's own fixed device array (STATIC_SCRATCH_BYTES); larger needs return HELIX_ERR_WORKSPACE."""
        rc = self._lib.helix_gemm_static_scratch(A, B, C, M, N, K, lda, ldb, ldc, stream or None)
        if check and rc != 0:
            raise HelixError("helix_gemm_static_scratch", rc)
        return rc

    def conv2d(self, x, w, y, batch, H, W, IC, OC, kH, kW, stride, pad, ws=0, ws_bytes=0, stream=0, check=True):
        rc = self._lib.helix_conv2d(x, w, y, batch, H, W, IC, OC, kH, kW, stride, pad, ws or None, ws_bytes,
                                    stream or None)
        if check and rc != 0:
            raise HelixError("helix_conv2d", rc)
        return rc

    def gemm_timed(self, A, B, C, M, N, K, lda, ldb, ldc, ws=0, ws_bytes=0, stream=0, warmup=10, iters=10):
        avg = ctypes.c_double(0.0)
        rc = self._lib.helix_gemm_timed(A, B, C, M, N, K, lda, ldb, ldc, ws or None, ws_bytes, stream or None,
                                        warmup, iters, ctypes.byref(avg))
        if rc != 0:
            raise HelixError("helix_gemm_timed", rc)
        return avg.value

    def conv2d_timed(self, x, w, y, batch, H, W, IC, OC, kH, kW, stride, pad, ws=0, ws_bytes=0, stream=0,
                     warmup=10, iters=10):
        avg = ctypes.c_double(0.0)
        rc = self._lib.helix_conv2d_timed(x, w, y, batch, H, W, IC, OC, kH, kW, stride, pad, ws or None, ws_bytes,
                                          stream or None, warmup, iters, ctypes.byref(avg))
        if rc != 0:
            raise HelixError("helix_conv2d_timed", rc)
        return avg.value

    # -- self-contained measurements: (min_s, avg_s, max_s) per launch -------------------------------
    def bench(self, M, N, K, warmup=10, iters=10, outer=1, rotate_bytes=0):
        mn, av, mx = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
        rc = self._lib.helix_bench(M, N, K, warmup, iters, outer, rotate_bytes, ctypes.byref(mn), ctypes.byref(av),
                                   ctypes.byref(mx))
        if rc != 0:
            raise HelixError("helix_bench", rc)
        return mn.value, av.value, mx.value

    def bench_conv(self, batch, IC, H, W, OC, kH, kW, stride, pad, warmup=10, iters=10, outer=1):
        mn, av, mx = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
        rc = self._lib.helix_bench_conv(batch, IC, H, W, OC, kH, kW, stride, pad, warmup, iters, outer,
                                        ctypes.byref(mn), ctypes.byref(av), ctypes.byref(mx))
        if rc != 0:
            raise HelixError("helix_bench_conv", rc)
        return mn.value, av.value, mx.value


PROBE_SYMBOLS = ("helix_mfma_probe",)


def mfma_probe(path, zero_operands=False, warmup=2, launches=10, loops=500):
    """(seconds per launch, TFLOP/s) of the MFMA-only loop of include/helix_probe.h: what the matrix pipes sustain
    with nothing else running, on seeded or on all-zero operands."""
    if not os.path.exists(path):
        raise FileNotFoundError(f"probe library {path} is not built; run __graft_entry__.build() first")
    L = ctypes.CDLL(path)
    L.helix_mfma_probe.argtypes = [_i, _i, _i, _i, _dp, _dp]
    L.helix_mfma_probe.restype = _i
    sec, flop = ctypes.c_double(), ctypes.c_double()
    rc = L.helix_mfma_probe(1 if zero_operands else 0, warmup, launches, loops, ctypes.byref(sec), ctypes.byref(flop))
    if rc != 0:
        raise HelixError("helix_mfma_probe", rc)
    return sec.value, flop.value / sec.value / 1e12


def exported_symbols(path):
    """Names from ABI_SYMBOLS that `path` exports (no device needed: dlopen + dlsym only)."""
    L = ctypes.CDLL(path)
    return [s for s in ABI_SYMBOLS if hasattr(L, s)]
