#!/usr/bin/env python3
"""Headline benchmark: autotuned FP16 GEMM (FP16 in, FP32 accumulate, FP16 out) at M=N=K=8192 on one
MI355X, reported as TFLOP/s and as a fraction of the FP16 MFMA peak, with the decode-GEMV HBM rate,
the autotune wall time and the CPU baseline (the restated x86_CPU path on the host cores) beside it.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one GEMM launch through the C ABI (helix_gemm) on operands already resident in HBM.  Prints
one JSON line.
"""
import argparse
import contextlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "helix_amd", "scripts"))
os.chdir(ROOT)

SIZE = 8192
# HBM-side bytes per 8192^3 launch (FETCH_SIZE + WRITE_SIZE from rocprofv3 --pmc runs, scaled by what the same
# counters read for a 1 GiB device copy), per configuration that has been counted, with the summary that holds
# the counter values.  A configuration without a counted run reports null: the figure cannot be measured from
# inside this process.
MEASURED_TRAFFIC = {
    (2, 256, 256, 64, 128, 0, 64): (1.748e9, "profiles/gemm_f16_8192_pmc.md"),
    (2, 256, 256, 128, 64, 0, 64): (1.745e9, "profiles/gemm_f16_8192_pmc.md"),
    (2, 256, 256, 128, 128, 0, 64): (1.745e9, "profiles/gemm_f16_8192_pmc.md"),
    (2, 256, 256, 64, 128, 0, 64, 1): (1.745e9, "profiles/gemm_f16_8192_pmc.md"),
    (2, 256, 256, 128, 64, 0, 64, 1): (1.745e9, "profiles/gemm_f16_8192_pmc.md"),
}


def autotune(prof_keys, M, N, K, finalists=6):
    """Full template search for one shape: run every MFMA configuration once (short timing), then time the fastest
    few again with more launches and keep the best of those."""
    from MI355X_FP16.MI355X_FP16_gemm import run_config
    timed = []
    for k in prof_keys:
        if k[0] == 0:
            continue
        try:
            timed.append((run_config(k, M, N, K, warmup=1, iters=3), k))
        except Exception:
            continue
    if not timed:
        raise RuntimeError("no MI355X_FP16 kernel library could run; build them with __graft_entry__.build()")
    timed.sort()
    best, best_t = None, float("inf")
    for _, k in timed[:finalists]:
        t = run_config(k, M, N, K, warmup=3, iters=10, outer=2)
        if t < best_t:
            best, best_t = k, t
    return best, best_t, len(timed)


def other_configs():
    """The other measured configurations, each against its roofline: decode GEMV (cold, HBM), FP16 and FP32 squares,
    the batch-32 ResNet-50 conv layers and the BERT-base GEMM list.  Squares and the BERT list are run three ways:
    the cost model's pick (Default), the exhaustive per-shape search (Oracle: "full template search per shape",
    "per-shape autotune") and the vendor library (rocBLAS; MIOpen for the conv layers).  Both backends are profiled
    here, timed: that is the autotune cost a user pays once per machine.  Rows as printed by
    helix_amd/scripts/benchmark_baseline_configs.py."""
    import benchmark_baseline_configs as bc
    from utils.helix_runtime import read_prof_dict
    out = {}
    profile_s = {}
    dicts = {}
    for name in ("MI355X_FP16", "MI355X_FP32"):
        be = bc.Backend(name)
        t0 = time.perf_counter()
        with contextlib.redirect_stdout(sys.stderr):     # the profile scripts' progress lines; stdout carries the one JSON line
            getattr(be.profile, f"profile_Helix_{name}_gemm_kernel")()
        profile_s[name] = round(time.perf_counter() - t0, 2)
        dicts[name] = (be, read_prof_dict(name))
    out["profile_wall_s"] = profile_s
    be16, d16 = dicts["MI355X_FP16"]
    out["gemv_hbm"] = bc.gemv_rows(be16, d16)
    out["gemm_f16_squares"] = bc.square_rows(be16, d16, oracle=True, vendor=True)
    out["conv_f16"] = bc.conv_rows(be16, d16, vendor=True, oracle=True)
    out["bert_f16"] = bc.bert_rows(be16, d16, oracle=True, vendor=True)[-1]
    be32, d32 = dicts["MI355X_FP32"]
    out["sgemm_f32"] = bc.square_rows(be32, d32, oracle=True, vendor=True)
    out["bert_f32"] = bc.bert_rows(be32, d32, oracle=True, vendor=True)[-1]
    return out


def build_times():
    """Seconds the last __graft_entry__.build() spent compiling each backend's libraries (written next to them)."""
    path = os.path.join(ROOT, "build", "build_times.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        return json.load(f)


def engine_clock_mhz(run_for_s, work):
    """(median engine clock in MHz the driver reports while `work()` is called in a loop for about run_for_s
    seconds -- None where the clock file is not readable --, seconds per call of work() over that loop)."""
    import glob
    import statistics
    import threading
    files = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))
    samples, stop = [], threading.Event()

    def sample():
        while files and not stop.is_set():
            try:
                for line in open(files[0]).read().splitlines():
                    if line.strip().endswith("*"):
                        samples.append(int(line.split(":")[1].strip().lower().split("mhz")[0]))
            except Exception:
                return
            time.sleep(0.02)

    th = threading.Thread(target=sample, daemon=True)
    th.start()
    t0 = time.perf_counter()
    calls = 0
    while time.perf_counter() - t0 < run_for_s:
        work()
        calls += 1
    per_call = (time.perf_counter() - t0) / calls
    stop.set()
    th.join(timeout=1.0)
    return (int(statistics.median(samples)) if samples else None), per_call


def mfma_ceiling():
    """The matrix pipes with nothing else running (the MFMA-only loop of include/helix_probe.h, same instruction,
    accumulators and waves per compute unit as the 256 x 256 x 64 GEMM tile), on seeded and on all-zero operands:
    rate over about half a second each and the engine clock the driver reports meanwhile.  On seeded operands the
    part runs against its power limit; this is the ceiling the GEMM rates above stand under."""
    from utils.helix_runtime import probe_library
    from utils.hip_ctypes import mfma_probe
    path = probe_library("mfma_probe")
    out = {}
    for name, zeros in (("seeded", False), ("zeros", True)):
        rates = []
        clk, _ = engine_clock_mhz(0.5, lambda: rates.append(mfma_probe(path, zeros, warmup=1, launches=8, loops=500)[1]))
        settled = rates[len(rates) // 2:]
        out[name] = {"tflops": round(sum(settled) / len(settled), 1), "engine_clock_mhz": clk,
                     "frac_datasheet_peak": round(sum(settled) / len(settled) * 1e12 / 2516.6e12, 4)}
    out["how"] = ("MFMA-only loop (v_mfma_f32_16x16x32_f16, 8 waves per compute unit, operands in registers), "
                  "second half of 0.5 s of launches each")
    return out


def cpu_baseline(budget_s=24.0):
    """The reference's x86_CPU path (restated in oracle/) on this machine's host cores: two-phase
    profile, tiling pick, then the packed / n-parallel schedule.  The headline sample is FP32 2048^3 (the
    largest square the host finishes a few times within the budget); three more samples cover configuration 1
    (FP32 1024^3), one convolution layer of configuration 4 and one BERT-base GEMM of configuration 5."""
    import numpy as np
    from oracle import oracle as O
    cores = os.cpu_count() or 1
    t0 = time.perf_counter()
    _, cache = O.x86_profile(peak_gflops=None, number=200)
    prof_s = time.perf_counter() - t0

    def sample(M, N, K, share):
        cost, gflops, padded, tiling, _ = O.x86_time_gemm(cache, M, N, K, num_thread=cores, number=1)
        number = max(1, min(100, int(share / max(cost, 1e-3))))
        cost, gflops, padded, tiling, _ = O.x86_time_gemm(cache, M, N, K, num_thread=cores, number=number)
        return cost, gflops, padded, tiling, number

    left = max(budget_s - prof_s, 6.0)
    s = 2048
    cost, gflops, padded, tiling, number = sample(s, s, s, 0.5 * left)
    extra = []
    # the reference's x86 path times a convolution as the GEMM of its im2col extents (restated in the oracle)
    conv_layer = (32, 128, 28, 28, 128, 3, 3, 1, 1)
    for (label, (M, N, K)) in (("config 1: FP32 GEMM 1024^3", (1024, 1024, 1024)),
                               ("config 4: conv 28x28x128 3x3 batch 32 as its im2col GEMM, FP32",
                                O.x86_conv_gemm_extents(*conv_layer)),
                               ("config 5: BERT-base FFN-out GEMM 4096x768x3072, FP32", (4096, 768, 3072))):
        c, g, pd, tl, n = sample(M, N, K, 0.15 * left)
        extra.append({"sample": f"{label} (padded to {pd[0]}x{pd[1]}x{pd[2]}), tiling {tl}, mean of {n} runs",
                      "value": round(g / 1e3, 4), "unit": "TFLOP/s", "ms": round(c * 1e3, 3)})
    return {"value": round(gflops / 1e3, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"FP32 GEMM {s}^3 (padded to {padded[0]}x{padded[1]}x{padded[2]}), restated x86_CPU schedule "
                      f"tiling {tiling}, mean of {number} runs; x86 profile took {prof_s:.1f} s",
            "isa": O.isa(), "more_samples": extra}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-gemv", action="store_true",
                    help="skip the other configurations (decode GEMV, FP32 squares, conv layers, BERT list)")
    ap.add_argument("--kernel-config", type=str, default=None,
                    help="skip the template search and time this configuration, e.g. 2,256,256,64,128,0,64")
    ap.add_argument("--operands", choices=["seeded", "zeros"], default="seeded",
                    help="zeros: all-zero operands (no data-dependent power draw; the kernel's structural rate)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch one 1 GiB device copy (a reference point for HBM traffic counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (every GPU box has one GPU); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from utils import seeded_inputs
    from utils.helix_runtime import load
    from utils.roofline import FP16_MFMA_FLOPS, gemm_flops
    from MI355X_FP16.build_MI355X_FP16 import library_for_key, is_dtl_key
    from MI355X_FP16.profile_MI355X_FP16 import all_keys

    if not torch.cuda.is_available():
        raise RuntimeError("bench.py needs an MI355X; there is no CPU fallback for the HIP path")
    dev = torch.device("cuda:0")
    M = N = K = SIZE

    # ---- seeded operands, resident in HBM before the timed region (generated first: the host-side generation
    # takes seconds, during which the GPU would fall back to its idle clocks right in front of the timed steps) --------------------------------------
    if args.operands == "zeros":
        A = torch.zeros((M, K), dtype=torch.float16, device=dev)
        Bt = torch.zeros((N, K), dtype=torch.float16, device=dev)
    else:
        A_h, B_h = seeded_inputs.gemm_operands(M, N, K, np.float16)      # A (M,K), B (K,N)
        A = torch.from_numpy(A_h).to(dev)
        Bt = torch.from_numpy(np.ascontiguousarray(B_h.T)).to(dev)       # device layout: N x K
    # ---- autotune: full template search on this shape ------------------------------------------------
    t0 = time.perf_counter()
    if args.kernel_config:
        best, tried = tuple(int(x) for x in args.kernel_config.split(",")), 0
    else:
        best, best_t, tried = autotune(all_keys(), M, N, K)
    autotune_s = time.perf_counter() - t0
    lib = load(library_for_key(best))

    C = torch.empty((M, N), dtype=torch.float16, device=dev)
    wsb = lib.workspace_bytes(M, N, K)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    def step():
        lib.gemm(A.data_ptr(), Bt.data_ptr(), C.data_ptr(), M, N, K, K, K, N, ws.data_ptr(), wsb, stream)

    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    flops = gemm_flops(M, N, K)
    value = flops / (elapsed / args.steps) / 1e12

    # ---- dominant kernel, HIP events on the launch stream -----------------------------------------------
    kern_s = lib.gemm_timed(A.data_ptr(), Bt.data_ptr(), C.data_ptr(), M, N, K, K, K, N, ws.data_ptr(), wsb, stream,
                            warmup=2, iters=args.steps)
    achieved = flops / kern_s / 1e12
    traffic, traffic_source = MEASURED_TRAFFIC.get(tuple(best), (None, None))
    if is_dtl_key(best):
        kernel = "helix_gemm_f16_dtl_kernel<%d, %d, %d, %d, %d, %d, 1>" % (best[0], best[1], best[2], best[3], best[4], best[6])
    else:
        kernel = "helix_gemm_f16_kernel<0, %d, %d, %d, %d, %d, %d, 1>" % (best[0], best[1], best[2], best[3], best[4], best[6])
    roofline = {"bound": "mfma", "achieved": round(achieved, 2), "peak": FP16_MFMA_FLOPS / 1e12, "unit": "TFLOP/s",
                "frac": round(achieved * 1e12 / FP16_MFMA_FLOPS, 4), "traffic": traffic, "traffic_source": traffic_source,
                "kernel": kernel, "kernel_avg_us": round(kern_s * 1e6, 2)}

    # ---- spot check of the timed result against torch's FP32 matmul on a slice ------------------------------
    ref = A[:256].float() @ Bt[:256].float().t()
    err = (C[:256, :256].float() - ref).abs().max().item() / max(ref.abs().max().item(), 1e-30)
    if not err < 2e-2:
        raise RuntimeError(f"timed GEMM result is wrong: normwise error {err}")

    out = {
        "metric": "FP16 GEMM TFLOP/s (autotuned, FP16 in / FP32 accumulate / FP16 out)",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 (f32 accumulate)", "data": "synthetic",
        "config": {"workload": f"FP16 GEMM M=N=K={SIZE}, A,B ~ N(0,0.1^2) seeded, full template search",
                   "kernel_config": list(best), "library": os.path.basename(library_for_key(best))},
        "pct_mfma_peak": round(100.0 * value * 1e12 / FP16_MFMA_FLOPS, 2),
        "autotune_wall_s": round(autotune_s, 2), "autotune_candidates": tried,
        "roofline": roofline,
    }
    if args.operands != "seeded":
        out["config"]["workload"] = f"FP16 GEMM M=N=K={SIZE}, all-zero operands"
    # the vendor library (hipBLASLt through torch.matmul) on the same operands and layout (A row-major, B stored
    # N x K), wall clock, same warm-up and step counts; and the engine clock the driver reports under each of the two
    C2 = torch.empty_like(C)

    def vendor_step():
        torch.matmul(A, Bt.t(), out=C2)

    for _ in range(args.warmup):
        vendor_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        vendor_step()
    torch.cuda.synchronize()
    out["vendor_tflops"] = round(flops / ((time.perf_counter() - t0) / args.steps) / 1e12, 2)
    out["vendor"] = "torch.matmul (hipBLASLt), same operands, wall clock"
    # half a second of back-to-back launches of each (batches of 16 between synchronizations): the engine clock the
    # driver reports meanwhile, and the rate once the part has settled into the load (the timed steps above start
    # right behind other work and run at another power state than a long run does)
    batch = 16
    clk_h, per_h = engine_clock_mhz(0.5, lambda: ([step() for _ in range(batch)], torch.cuda.synchronize()))
    clk_v, per_v = engine_clock_mhz(0.5, lambda: ([vendor_step() for _ in range(batch)], torch.cuda.synchronize()))
    out["engine_clock_mhz"] = {"helix": clk_h, "vendor": clk_v, "datasheet_peak": 2400}
    out["sustained_tflops"] = {"helix": round(flops / (per_h / batch) / 1e12, 2),
                               "vendor": round(flops / (per_v / batch) / 1e12, 2),
                               "how": "0.5 s of back-to-back launches each, wall clock"}
    del C2
    out["mfma_only"] = mfma_ceiling()
    out["build_wall_s"] = build_times()
    if not args.no_gemv:
        out.update(other_configs())
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
