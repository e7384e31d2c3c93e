"""python3 benchmark_baseline_configs.py -c {square,gemv,conv,bert,all} -b <backend> [--oracle] [--no-tiles] [--no-verified] [--vendor] [--json]

The measured configurations of this backend, each against the roofline that bounds it:
  square  M = N = K in {1024, 2048, 4096, 8192}                              (MFMA peak)
  gemv    decode shapes, M in {1, 4, 16} activation rows, weights cold       (HBM peak)
  conv    batch-32 NHWC ResNet-50-shaped layers, implicit GEMM               (MFMA peak and HBM peak)
  bert    BERT-base encoder GEMMs at 4096 tokens x 12 layers + 4000x2300x770 (MFMA peak)
Every row is run through the runner's selection, as the reference's benchmark wrappers do
(scripts/Ampere_FP16/benchmark_Ampere_FP16_gemm.py:9-30): the cost model's ranking settled on the device and
remembered per problem (select_config), with the cost model's first choice alone beside it (model_config, model_us)
where the two differ; --no-verified runs the cost model's first choice only.  --oracle adds the exhaustive per-shape
search (benchmark_Ampere_FP16_performance_comparison.py:56-69).  Needs build_template.py to have run; profiles
first when no cost-model dict is on disk.
"""
import argparse
import importlib
import json
import os

from _dispatch import MI355X_BACKENDS
from utils import roofline as R
from utils import get_benchmark_shape_list as S
from utils.helix_runtime import load, read_prof_dict, prof_dict_path


class Backend:
    """The per-backend functions this script needs, looked up by the reference's naming scheme."""

    def __init__(self, name):
        self.name = name
        self.fp32 = name.endswith("FP32")
        self.elem_bytes = 4 if self.fp32 else 2
        self.peak = R.FP32_MFMA_FLOPS if self.fp32 else R.FP16_MFMA_FLOPS
        mod = lambda m: importlib.import_module(f"{name}.{m}")
        self.gemm, self.conv, self.build, self.profile = (mod(f"{name}_gemm"), mod(f"{name}_conv"),
                                                         mod(f"build_{name}"), mod(f"profile_{name}"))
        self.gemm_result = getattr(self.gemm, f"get_{name}_gemm_Helix_result")
        self.gemm_oracle = getattr(self.gemm, f"get_{name}_gemm_Oracle_result")
        self.conv_result = getattr(self.conv, f"get_{name}_conv_Helix_result")
        self.gemm_vendor = getattr(self.gemm, f"get_{name}_gemm_rocblas_result")

    def prof_dict(self):
        if not os.path.exists(prof_dict_path(self.name)):
            getattr(self.profile, f"profile_Helix_{self.name}_gemm_kernel")()
        return read_prof_dict(self.name)

    def is_gemv_key(self, k):
        return (k[2] == 0) if self.fp32 else (k[0] == 0)

    def block_rows(self, k):
        return k[0] if self.fp32 else k[1]


def steady_gemm(be, key, M, N, K):
    """(ms, TFLOP/s) of configuration `key`, timed the same way for every column of a row: three repetitions of
    10 warm-up + 10 timed launches, the fastest mean.  A single short measurement right behind a smaller problem
    runs while the engine clock is still ramping (a cost-model pick timed that way read 15 % slower than the same
    library a few seconds later), and the search's own minimum over hundreds of short timings is biased low."""
    t = min(be.gemm.run_config(key, M, N, K, warmup=10, iters=10) for _ in range(3))
    return t * 1e3, 2.0 * M * N * K / t / 1e12


def steady_oracle(be, prof_dict, dkey, dms, M, N, K):
    """(ms, TFLOP/s, key) of the exhaustive search's pick, timed like the Default column.  The Default configuration
    is one of the candidates, so when the search returns it again, or a configuration that the steadier timing shows
    to be slower, the row's Oracle column is the Default measurement itself."""
    _, _, okey = be.gemm_oracle(prof_dict, M, N, K)
    if tuple(okey) != tuple(dkey):
        oms, otf = steady_gemm(be, okey, M, N, K)
        if oms < dms:
            return oms, otf, okey
    return dms, 2.0 * M * N * K / (dms * 1e-3) / 1e12, dkey


def selected_and_model(be, prof_dict, M, N, K, verified):
    """(key the runner launches, the cost model's first choice): the same key when verified is False."""
    mkey = be.gemm.cost_model(prof_dict, M, N, K)
    return (be.gemm.select_config(prof_dict, M, N, K) if verified else mkey), mkey


def steady_vendor(be, M, N, K):
    lib = load(be.build.kernel_library("rocblas_f32" if be.fp32 else "rocblas_f16"))
    mn, _, _ = lib.bench(M, N, K, warmup=10, iters=10, outer=3, rotate_bytes=0)
    return mn * 1e3, 2.0 * M * N * K / mn / 1e12


def square_rows(be, prof_dict, oracle=False, vendor=False, verified=True):
    """Per size: the runner's selection (and the cost model's first choice where it differs); oracle=True adds the
    exhaustive per-shape search, vendor=True rocBLAS on the same operand layouts."""
    rows = []
    for s in S.BASELINE_SQUARE_SIZES:
        key, mkey = selected_and_model(be, prof_dict, s, s, s, verified)
        ms, tflops = steady_gemm(be, key, s, s, s)
        row = {"M": s, "N": s, "K": s, "config": list(key), "us": round(ms * 1e3, 2), "TFLOP/s": round(tflops, 2),
               "frac_mfma_peak": round(tflops * 1e12 / be.peak, 4)}
        if tuple(mkey) != tuple(key):
            row.update({"model_config": list(mkey), "model_us": round(steady_gemm(be, mkey, s, s, s)[0] * 1e3, 2)})
        if oracle:
            oms, otf, okey = steady_oracle(be, prof_dict, key, ms, s, s, s)
            row.update({"oracle_config": list(okey), "oracle_us": round(oms * 1e3, 2), "oracle_TFLOP/s": round(otf, 2),
                        "oracle_frac_mfma_peak": round(otf * 1e12 / be.peak, 4)})
        if vendor:
            vms, vtf = steady_vendor(be, s, s, s)
            row.update({"rocblas_us": round(vms * 1e3, 2), "rocblas_TFLOP/s": round(vtf, 2)})
        rows.append(row)
    return rows


def gemv_rows(be, prof_dict, rotate_bytes=1 << 30, tiles=True):
    """Weights rotated through >= 1 GiB so the 256 MB last-level cache cannot hold them.  Per shape: the GEMV
    library, and (tiles=True) the fastest of the 32-row MFMA tile libraries, the other family the cost model
    chooses from for skinny shapes."""
    lib = load(be.build.kernel_library("gemv_fp32" if be.fp32 else "gemv"))
    # FP16: the same template with the MFMA variant switched off (vector dot products and a wave reduction for
    # every batch), reported beside the MFMA variant where the two differ (9 or more activation rows)
    nomfma = None if be.fp32 else load(be.build.kernel_library("gemv_nomfma"))
    tile_keys = [k for k in prof_dict if not be.is_gemv_key(k) and be.block_rows(k) == 32] if tiles else []
    rows = []
    # what one launch costs when the kernel has next to nothing to do (same library, same back-to-back event timing,
    # a 64 x 512 weight matrix): the part of every row's time that is launch and drain rather than streaming
    floor = lib.bench(1, 64, 512, warmup=5, iters=50, outer=3, rotate_bytes=0)[0]
    for (K, N) in S.BASELINE_GEMV_KN:
        for M in S.BASELINE_GEMV_BATCHES:
            mn, _, _ = lib.bench(M, N, K, warmup=5, iters=50, outer=3, rotate_bytes=rotate_bytes)
            nbytes = R.gemm_bytes(M, N, K, be.elem_bytes)
            row = {"M": M, "K": K, "N": N, "us": round(mn * 1e6, 2), "GB/s": round(nbytes / mn / 1e9, 1),
                   "frac_hbm_peak": round(nbytes / mn / R.HBM_BYTES_PER_S, 4),
                   "launch_floor_us": round(floor * 1e6, 2),
                   "GB/s_above_floor": round(nbytes / max(mn - floor, 1e-9) / 1e9, 1)}
            if nomfma is not None and M >= 9:
                mn_v = nomfma.bench(M, N, K, warmup=5, iters=50, outer=3, rotate_bytes=rotate_bytes)[0]
                row["no_mfma_GB/s"] = round(nbytes / mn_v / 1e9, 1)
            best_t, best_k = float("inf"), None
            for k in tile_keys:
                try:
                    t = load(be.build.library_for_key(k)).bench(M, N, K, warmup=2, iters=10, outer=1,
                                                               rotate_bytes=rotate_bytes)[1]
                except Exception:
                    continue
                if t < best_t:
                    best_t, best_k = t, k
            if best_k is not None:
                mn_t = load(be.build.library_for_key(best_k)).bench(M, N, K, warmup=5, iters=50, outer=3,
                                                                   rotate_bytes=rotate_bytes)[0]
                row["tile_GB/s"] = round(nbytes / mn_t / 1e9, 1)
                row["tile_config"] = list(best_k)
                # what the search over both families delivers for the shape
                row["best_GB/s"] = max(row["GB/s"], row["tile_GB/s"])
                row["best_frac_hbm_peak"] = round(row["best_GB/s"] * 1e9 / R.HBM_BYTES_PER_S, 4)
            rows.append(row)
    return rows


def conv_rows(be, prof_dict, vendor=False, oracle=False, verified=True):
    """vendor=True adds MIOpen's time on the same layer (the comparator library); oracle=True the exhaustive
    per-layer search over every configuration with a conv entry (FP16 backend)."""
    miopen = load(be.build.kernel_library("miopen_f32" if be.fp32 else "miopen_f16")) if vendor else None
    conv_oracle = getattr(be.conv, f"get_{be.name}_conv_Oracle_result", None) if oracle else None
    rows = []
    for shp in S.get_baseline_conv_shape_list():
        b, ic, h, w, oc, kh, kw, st, pd = shp
        M = b * ((h + 2 * pd - kh) // st + 1) * ((w + 2 * pd - kw) // st + 1)
        mkey = be.conv.layer_cost_model(prof_dict, *shp)
        key = be.conv.select_config(prof_dict, *shp) if verified else mkey
        ms = min(load(be.build.library_for_key(key)).bench_conv(*shp, warmup=10, iters=10)[1] for _ in range(3)) * 1e3
        tflops = R.conv_flops(*shp) / (ms * 1e-3) / 1e12
        nbytes = R.conv_bytes(*shp, be.elem_bytes)
        rows.append({"shape": list(shp), "gemm_MNK": [M, oc, ic * kh * kw], "config": list(key), "us": round(ms * 1e3, 2),
                     "TFLOP/s": round(tflops, 2), "frac_mfma_peak": round(tflops * 1e12 / be.peak, 4),
                     "GB/s": round(nbytes / (ms * 1e-3) / 1e9, 1),
                     "frac_hbm_peak": round(nbytes / (ms * 1e-3) / R.HBM_BYTES_PER_S, 4)})
        if tuple(mkey) != tuple(key):
            mms = min(load(be.build.library_for_key(mkey)).bench_conv(*shp, warmup=10, iters=10)[1] for _ in range(3)) * 1e3
            rows[-1].update({"model_config": list(mkey), "model_us": round(mms * 1e3, 2)})
        if conv_oracle is not None:
            oms, otf, okey = conv_oracle(prof_dict, *shp)
            if oms >= ms:   # the Default configuration is one of the candidates
                oms, otf, okey = ms, tflops, key
            rows[-1].update({"oracle_config": list(okey), "oracle_us": round(oms * 1e3, 2),
                             "oracle_frac_mfma_peak": round(otf * 1e12 / be.peak, 4),
                             "oracle_frac_hbm_peak": round(nbytes / (oms * 1e-3) / R.HBM_BYTES_PER_S, 4)})
        if miopen is not None:
            rows[-1]["miopen_us"] = round(miopen.bench_conv(*shp, warmup=10, iters=10)[1] * 1e6, 2)
    return rows


def bert_rows(be, prof_dict, oracle=False, vendor=False, verified=True):
    """Per distinct GEMM of the encoder, then the whole list (12 layers + the irregular shape) as one row: summed
    latency, as the reference sums per-GEMM costs (benchmark_Ampere_FP16_model_level_LLM.py:16-27).  oracle=True adds
    the exhaustive per-shape search ("per-shape autotune"), vendor=True rocBLAS."""
    memo, rows = {}, []
    totals = {"default": 0.0, "model": 0.0, "oracle": 0.0, "rocblas": 0.0}
    total_flops = 0.0
    for (M, N, K) in S.get_baseline_bert_MNKList():
        if (M, N, K) not in memo:
            dkey, mkey = selected_and_model(be, prof_dict, M, N, K, verified)
            ms, tflops = steady_gemm(be, dkey, M, N, K)
            row = {"M": M, "N": N, "K": K, "config": list(dkey),
                   "us": round(ms * 1e3, 2), "TFLOP/s": round(tflops, 2),
                   "frac_mfma_peak": round(tflops * 1e12 / be.peak, 4)}
            times = {"default": ms, "model": ms}
            if tuple(mkey) != tuple(dkey):
                times["model"] = steady_gemm(be, mkey, M, N, K)[0]
                row.update({"model_config": list(mkey), "model_us": round(times["model"] * 1e3, 2)})
            if oracle:
                oms, otf, okey = steady_oracle(be, prof_dict, dkey, ms, M, N, K)
                row.update({"oracle_config": list(okey), "oracle_us": round(oms * 1e3, 2), "oracle_TFLOP/s": round(otf, 2)})
                times["oracle"] = oms
            if vendor:
                vms, vtf = steady_vendor(be, M, N, K)
                row.update({"rocblas_us": round(vms * 1e3, 2), "rocblas_TFLOP/s": round(vtf, 2)})
                times["rocblas"] = vms
            memo[(M, N, K)] = times
            rows.append(row)
        for name, ms in memo[(M, N, K)].items():
            totals[name] += ms
        total_flops += 2.0 * M * N * K
    tf = total_flops / (totals["default"] * 1e-3) / 1e12
    total = {"total_ms": round(totals["default"], 4), "TFLOP/s": round(tf, 2), "frac_mfma_peak": round(tf * 1e12 / be.peak, 4)}
    if verified:
        mtf = total_flops / (totals["model"] * 1e-3) / 1e12
        total.update({"model_total_ms": round(totals["model"], 4), "model_TFLOP/s": round(mtf, 2)})
    if oracle:
        otf = total_flops / (totals["oracle"] * 1e-3) / 1e12
        total.update({"oracle_total_ms": round(totals["oracle"], 4), "oracle_TFLOP/s": round(otf, 2),
                      "oracle_frac_mfma_peak": round(otf * 1e12 / be.peak, 4)})
    if vendor:
        total.update({"rocblas_total_ms": round(totals["rocblas"], 4),
                      "rocblas_TFLOP/s": round(total_flops / (totals["rocblas"] * 1e-3) / 1e12, 2)})
    rows.append(total)
    return rows


SECTIONS = {"square": square_rows, "gemv": gemv_rows, "conv": conv_rows, "bert": bert_rows}


def run(backend, configs, oracle=False, tiles=True, vendor=False, verified=True):
    be = Backend(backend)
    prof_dict = be.prof_dict()
    out = {}
    for name in configs:
        if name == "square":
            out[name] = square_rows(be, prof_dict, oracle, vendor, verified)
        elif name == "bert":
            out[name] = bert_rows(be, prof_dict, oracle, vendor, verified)
        elif name == "gemv":
            out[name] = gemv_rows(be, prof_dict, tiles=tiles)
        elif name == "conv":
            out[name] = conv_rows(be, prof_dict, vendor=vendor, oracle=oracle, verified=verified)
        else:
            out[name] = SECTIONS[name](be, prof_dict)
    return out


if __name__ == "__main__":
    parser = argparse.ArgumentParser(description="Benchmark the measured configurations against their rooflines")
    parser.add_argument("-c", "--config", type=str, choices=list(SECTIONS) + ["all"], default="all")
    parser.add_argument("-b", "--backend", type=str, choices=MI355X_BACKENDS, default="MI355X_FP16")
    parser.add_argument("--oracle", action="store_true", help="square, bert, conv: also run the exhaustive per-shape search")
    parser.add_argument("--no-tiles", action="store_true", help="gemv: time the GEMV library only")
    parser.add_argument("--no-verified", action="store_true", help="square, bert, conv: run the cost model's first choice only (no candidates timed, no winners kept)")
    parser.add_argument("--vendor", action="store_true", help="conv: add MIOpen's time per layer; square, bert: add rocBLAS's")
    parser.add_argument("--json", action="store_true", help="one JSON object instead of the table")
    args = parser.parse_args()

    result = run(args.backend, list(SECTIONS) if args.config == "all" else [args.config], args.oracle,
                 tiles=not args.no_tiles, vendor=args.vendor, verified=not args.no_verified)
    if args.json:
        print(json.dumps(result))
    else:
        for name, rows in result.items():
            print(f"== {name} ({args.backend})")
            for row in rows:
                print("  " + ", ".join(f"{k}: {v}" for k, v in row.items()))
