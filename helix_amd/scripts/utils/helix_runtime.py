"""Shared host plumbing of the MI355X backends: hipcc invocation, artifact paths, library cache.

The reference shells out once per configuration (`os.system("nvcc ... -o build/bin_fp16/gemm_...")`,
scripts/Ampere_FP16/build_Ampere_FP16.py:7-28) and once per measurement (`os.popen(exe M N K)`,
scripts/Ampere_FP16/profile_Ampere_FP16.py:36-38).  Here a configuration is a shared library that is
compiled once, loaded once per process and called through ctypes.
"""
import json
import os
import re
import subprocess
import time
from concurrent.futures import ThreadPoolExecutor

from utils.hip_ctypes import HelixLib

root_path = os.getcwd()

_SCRIPTS_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC_ROOT = os.path.normpath(os.path.join(_SCRIPTS_DIR, "..", "src_template"))


def _find_include_dir():
    for cand in (os.path.join(_SCRIPTS_DIR, "..", "..", "include"), os.path.join(_SCRIPTS_DIR, "..", "include")):
        if os.path.exists(os.path.join(cand, "helix_abi.h")):
            return os.path.normpath(cand)
    raise FileNotFoundError("include/helix_abi.h not found next to the scripts tree")


HIPCC = os.environ.get("HIPCC", "hipcc")
# -packed-fp32-ops is switched off on purpose: the compiler must not form packed FP32 VALU ops here.
# Hidden visibility + -Bsymbolic: a library exports the helix_* entry points of include/helix_abi.h and nothing
# else, and its own calls bind inside it, so several configurations can share a process however they are opened.
# -Rpass-analysis=kernel-resource-usage: hipcc reports registers, scratch and LDS of every kernel on stderr;
# compile_many keeps the figures in <bin dir>/resource_usage.json (see kernel_resources).
COMPILE_OPTIONS = ("-O3 -std=c++17 --offload-arch=gfx950 -shared -fPIC -w -fvisibility=hidden -Wl,-Bsymbolic "
                   "-Xclang -target-feature -Xclang -packed-fp32-ops -Rpass-analysis=kernel-resource-usage")


def bin_dir(precision):
    return f"{root_path}/build/bin_{precision}"


def probe_library(name="mfma_probe"):
    """Path of a measurement aid (include/helix_probe.h), built beside the template libraries."""
    return f"{root_path}/build/bin_probe/lib{name}.so"


def build_probes():
    """Compiles the measurement aids of src_template/probe; returns the list of failures like compile_many."""
    return compile_many([(os.path.join(SRC_ROOT, "probe", "mfma_probe.hip"), probe_library("mfma_probe"), {})])


def prof_dict_path(backend):
    return f"{root_path}/build/prof_dict/{backend}_cost_model.dict"


# The tile kernels fix their own instruction order (a scheduling fence behind every MFMA slot), but the compiler's
# scheduler in front of the register allocator still decides the register pressure.  Where a default build leaves a
# kernel spilling, compile_many builds the library once more with this option and keeps that build when no kernel in
# it spills more and the sum over the kernels is smaller.
NO_SCHEDULER_OPTION = "-mllvm -enable-misched=0"


def compile_command(src, out, defines, link="", extra=""):
    """hipcc line of one library; `link` holds extra linker flags (the vendor comparators' -lrocblas), `extra`
    further compiler options."""
    inc = _find_include_dir()
    cmd = f"{HIPCC} {src} {COMPILE_OPTIONS} -I{inc} -I{os.path.join(SRC_ROOT, 'common')}"
    if extra:
        cmd += f" {extra}"
    for k, v in defines.items():
        cmd += f" -D{k}={v}"
    if link:
        cmd += f" {link}"
    cmd += f" -o {out}"
    return cmd


def compile_library(src, out, defines, link="", extra=""):
    """Returns (ok, stderr_text)."""
    os.makedirs(os.path.dirname(out), exist_ok=True)
    tmp = out + ".tmp"
    proc = subprocess.run(compile_command(src, tmp, defines, link, extra), shell=True, capture_output=True, text=True)
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        return False, proc.stderr
    os.replace(tmp, out)
    return True, proc.stderr


def parse_resource_usage(stderr_text):
    """{kernel function name: {"vgprs": n, "agprs": n, "scratch": bytes per lane, "occupancy": waves per SIMD}} from
    the -Rpass-analysis=kernel-resource-usage remarks of one hipcc run."""
    out, cur = {}, None
    for line in stderr_text.splitlines():
        m = re.search(r"remark:\s+Function Name: (\S+)", line)
        if m:
            cur = out.setdefault(m.group(1), {})
            continue
        if cur is None:
            continue
        for label, field in (("VGPRs:", "vgprs"), ("AGPRs:", "agprs"), ("ScratchSize [bytes/lane]:", "scratch"),
                             ("Occupancy [waves/SIMD]:", "occupancy")):
            m = re.search(r"remark:\s+" + re.escape(label) + r"\s+(\d+)", line)
            if m:
                cur[field] = int(m.group(1))
    return out


def total_scratch(usage):
    """Scratch bytes per lane summed over the kernels of one library (parse_resource_usage's dict)."""
    return sum(res.get("scratch", 0) for res in usage.values())


def spills_less(usage, than):
    """True when no kernel of `usage` has more scratch than the same kernel in `than` and the sum is smaller."""
    if set(usage) != set(than):
        return False
    if any(usage[k].get("scratch", 0) > than[k].get("scratch", 0) for k in usage):
        return False
    return total_scratch(usage) < total_scratch(than)


def resource_usage_path(directory):
    return os.path.join(directory, "resource_usage.json")


def compile_many(jobs, max_workers=None, progress=None):
    """jobs: iterable of (src, out, defines[, link flags]).  Compiles in parallel; returns list of failed outs.
    The per-kernel register / scratch figures hipcc reports are merged into resource_usage.json next to the
    libraries, keyed by library file name."""
    jobs = list(jobs)
    if max_workers is None:
        max_workers = int(os.environ.get("MAX_JOBS", min(16, os.cpu_count() or 1)))
    failed = []
    usage = {}

    def run(job):
        ok, err = compile_library(*job)
        if ok and total_scratch(parse_resource_usage(err)) > 0:
            alt = job[1] + ".nosched"
            ok_alt, err_alt = compile_library(job[0], alt, job[2], *job[3:4], extra=NO_SCHEDULER_OPTION)
            if ok_alt and spills_less(parse_resource_usage(err_alt), parse_resource_usage(err)):
                os.replace(alt, job[1])
                err = err_alt
            elif os.path.exists(alt):
                os.remove(alt)
        return job, ok, err

    with ThreadPoolExecutor(max_workers=max_workers) as ex:
        for job, ok, err in ex.map(run, jobs):
            if not ok:
                failed.append((job[1], err))
            else:
                usage.setdefault(os.path.dirname(job[1]), {})[os.path.basename(job[1])] = parse_resource_usage(err)
            if progress is not None:
                progress.update(1)
    for directory, per_lib in usage.items():
        path = resource_usage_path(directory)
        merged = {}
        if os.path.exists(path):
            try:
                with open(path) as f:
                    merged = json.load(f)
            except ValueError:
                merged = {}
        merged.update(per_lib)
        with open(path, "w") as f:
            json.dump(merged, f)
    return failed


_resource_cache = {}


def kernel_resources(library_path):
    """The kernels of one built library with their registers and scratch bytes, {} when the build left no record."""
    directory = os.path.dirname(library_path)
    if directory not in _resource_cache:
        path = resource_usage_path(directory)
        try:
            with open(path) as f:
                _resource_cache[directory] = json.load(f)
        except (OSError, ValueError):
            _resource_cache[directory] = {}
    return _resource_cache[directory].get(os.path.basename(library_path), {})


_lib_cache = {}


def load(path):
    """Process-wide cache of loaded kernel libraries (raises FileNotFoundError if not built)."""
    lib = _lib_cache.get(path)
    if lib is None:
        lib = HelixLib(path)
        _lib_cache[path] = lib
    return lib


# extra profile points kept beside the reference's dict: attribute of ProfDict -> file name suffix
EXTRA_PROFILE_POINTS = {"short": "shortK", "two_rounds": "2rounds", "short_two_rounds": "shortK_2rounds"}


class ProfDict(dict):
    """{config tuple: seconds per round of tiles at the profile K}, the reference's dict, plus optional
    extra points for the same keys, each {} when its file is absent:
      .short             one round at a short K: separates a round's fixed part (launch, pipeline fill,
                         epilogue) from its per-K part;
      .two_rounds        two rounds at the profile K (whole launch, not per round);
      .short_two_rounds  two rounds at the short K: what a further round costs once workgroups of
                         consecutive rounds share a compute unit."""

    def __init__(self, *a, **kw):
        super().__init__(*a, **kw)
        for attr in EXTRA_PROFILE_POINTS:
            setattr(self, attr, {})


def extra_prof_dict_path(backend, suffix):
    return f"{root_path}/build/prof_dict/{backend}_cost_model_{suffix}.dict"


def _read_dict_file(path):
    with open(path, "r") as f:
        lines = f.readlines()
        # same `eval(lines[0])` as the reference (benchmark_Ampere_FP16_gemm.py:10-12); `inf` is bound because
        # skipped configurations are stored as float('inf'), whose repr is not a Python literal
        return eval(lines[0], {"inf": float("inf"), "nan": float("nan")})


def read_prof_dict(backend):
    prof_dict = ProfDict(_read_dict_file(prof_dict_path(backend)))
    for attr, suffix in EXTRA_PROFILE_POINTS.items():
        if os.path.exists(extra_prof_dict_path(backend, suffix)):
            setattr(prof_dict, attr, _read_dict_file(extra_prof_dict_path(backend, suffix)))
    return prof_dict


def write_prof_dict(backend, prof_dict):
    os.makedirs(os.path.dirname(prof_dict_path(backend)), exist_ok=True)
    forget_winners(backend)   # winners were chosen among the old profile's rankings
    with open(prof_dict_path(backend), "w") as f:
        f.write(str(dict(prof_dict)))
    for attr, suffix in EXTRA_PROFILE_POINTS.items():
        path = extra_prof_dict_path(backend, suffix)
        extra = getattr(prof_dict, attr, None)
        if extra:
            with open(path, "w") as f:
                f.write(str(dict(extra)))
        elif os.path.exists(path):
            os.remove(path)   # never pair a new profile with stale extra points


# ---- per-problem winners ------------------------------------------------------------------------------------
# The cost model ranks configurations from two profile points each; the first few of its ranking lie within a few
# per cent of each other in prediction and 5 - 25 % apart on the device.  The runners therefore time the first few
# candidates the first time they meet a problem (a few dozen launches) and keep the winner in a dict file beside the
# profile, {problem tuple: configuration key} plus one entry that names the profile by its contents; later calls under
# the same profile, in this process or another, go straight to it; under any other profile the record starts afresh.  A
# new profile file (write_prof_dict) discards the file.  HELIX_SELECTION=model switches this off: the cost model alone
# picks, as in the reference (scripts/Ampere_FP16/Ampere_FP16_gemm.py:433-446).
def winners_path(backend):
    return f"{root_path}/build/prof_dict/{backend}_winners.dict"


def selection_mode():
    mode = os.environ.get("HELIX_SELECTION", "tuned")
    if mode not in ("tuned", "model"):
        raise ValueError(f"HELIX_SELECTION={mode!r}: expected 'tuned' or 'model'")
    return mode


_winners = {}
PROFILE_TAG = ("profile",)     # the entry of a winners file that names the profile its winners were ranked and timed under


def profile_fingerprint(prof_dict):
    """Names a profile by its contents: winners recorded under one profile are not handed out under another (a profile
    of other libraries or another machine state, a hand-made dict in a test)."""
    import hashlib
    return hashlib.md5(repr(sorted(prof_dict.items())).encode()).hexdigest()


def read_winners(backend, prof_dict):
    """The winners recorded for this backend under this profile ({} when there is no file yet or the file belongs to
    another profile); the file is read once per process."""
    if backend not in _winners:
        path = winners_path(backend)
        _winners[backend] = _read_dict_file(path) if os.path.exists(path) else {}
    tag = profile_fingerprint(prof_dict)
    if _winners[backend].get(PROFILE_TAG) != tag:
        _winners[backend] = {PROFILE_TAG: tag}
    return _winners[backend]


def store_winner(backend, problem, key, prof_dict):
    winners = read_winners(backend, prof_dict)
    winners[tuple(problem)] = tuple(key)
    path = winners_path(backend)
    os.makedirs(os.path.dirname(path), exist_ok=True)
    tmp = f"{path}.{os.getpid()}.tmp"
    with open(tmp, "w") as f:
        f.write(str(winners))
    os.replace(tmp, path)


def forget_winners(backend):
    _winners.pop(backend, None)
    if os.path.exists(winners_path(backend)):
        os.remove(winners_path(backend))


SETTLE_FINALISTS = 4        # candidates timed a second time ...
SETTLE_WITHIN = 1.10        # ... those within this factor of the fastest of the first pass


def fastest_of(keys, time_config, what):
    """The fastest of `keys` on the device.  time_config(key, warmup, iters) -> mean seconds per launch, raising for a
    configuration that cannot run the problem (skipped, as the profile skips it).  First pass: 2 + 5 launches each.  The
    leaders of that pass lie within its noise of each other (a 5-launch mean right behind another kernel moves by
    5 - 10 % with the engine clock), so up to SETTLE_FINALISTS of them within SETTLE_WITHIN of the fastest are timed
    again, two rounds of 5 + 20 launches in turn, and the smallest mean decides."""
    timed, last_error = [], None
    for k in keys:
        try:
            timed.append((time_config(k, 2, 5), k))
        except Exception as e:
            last_error = e
    if not timed:
        raise RuntimeError(f"none of the {len(keys)} ranked configurations could run {what}") from last_error
    timed.sort(key=lambda tk: tk[0])
    finalists = [k for t, k in timed[:SETTLE_FINALISTS] if t <= timed[0][0] * SETTLE_WITHIN]
    if len(finalists) == 1:
        return finalists[0]
    best = {k: float("inf") for k in finalists}
    for _ in range(2):
        for k in finalists:
            best[k] = min(best[k], time_config(k, 5, 20))
    return min(finalists, key=lambda k: best[k])


def tuned_config(backend, problem, prof_dict, model_pick, verify):
    """The configuration a runner launches for `problem`: the recorded winner if the profile still holds it, else
    `verify()` (the fastest of the cost model's first candidates, timed now) which is then recorded; with
    HELIX_SELECTION=model always `model_pick()`."""
    if selection_mode() == "model":
        return model_pick()
    key = read_winners(backend, prof_dict).get(tuple(problem))
    if key is not None and key in prof_dict:
        return key
    key = verify()
    store_winner(backend, problem, key, prof_dict)
    return key


def reference_line(M, N, K, min_s, avg_s, max_s):
    """The stdout line of the reference executables (src_template/Ampere_FP16/gemm.cu:687-689); its
    whitespace-split token [-8] is the mean seconds, which is what the reference profilers parse."""
    tflops = 2.0 * M * N * K / 1e12 / avg_s
    return (f"M N K = {M:6d} {N:6d} {K:6d}, Time = {min_s:12.8f} {avg_s:12.8f} {max_s:12.8f} s, "
            f"AVG Performance = {tflops:10.4f} Tflops")


class Stopwatch:
    def __enter__(self):
        self.t0 = time.perf_counter()
        return self

    def __exit__(self, *a):
        self.seconds = time.perf_counter() - self.t0
