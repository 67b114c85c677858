"""Merge rocprofv3 measurements into a captured profile.

``capture_profile`` fixes the row order and count of a profile (what the
interception layer will see) and times kernels with HIP events.  This module
adds what only the profiler knows -- per-kernel HBM traffic and matrix-core
utilisation -- and from them the bound class, replacing the name-based guess.
Counterpart of the reference's ``profiling/postprocessing/process_ncu.py`` and
``roofline_analysis.py`` (Nsight Compute metrics -> class, :37-71).

Collection (each counter set in a run of its own; from /tmp with TMPDIR=/tmp):

    rocprofv3 --kernel-trace --output-format csv -d D/trace -o t -- python3 -m orion_amd.profiling.standalone ...
    rocprofv3 --pmc FETCH_SIZE --output-format csv -d D/fetch -o t -- python3 -m orion_amd.profiling.standalone ...
    rocprofv3 --pmc WRITE_SIZE --output-format csv -d D/write -o t -- python3 -m orion_amd.profiling.standalone ...
    rocprofv3 --pmc MfmaUtil   --output-format csv -d D/mfma  -o t -- python3 -m orion_amd.profiling.standalone ...

(``python -m orion_amd.profiling.rocprof --collect ...`` runs these four.)  With an
optional D/flops run holding SQ_INSTS_VALU_{ADD,MUL,FMA}_{F32,F16} and
SQ_INSTS_VALU_MFMA_MOPS_{BF16,F32}, the class comes from arithmetic intensity
(``cu_need.classify_roofline``); without it from utilisation (>= 60 % of the
matrix cores or of HBM bandwidth), the reference's rule for kernels without
floating-point counts.

then ``python -m orion_amd.profiling.rocprof --profile P_fwd --rocprof-dir D --out P_fwd``.
Rows are joined by ORDER: the trailing ``rows x k`` kernel dispatches of every
run are the last k iterations of the client; runtime-internal kernels
(``__amd_rocclr_*``: fills and copies the interception layer sees as memory
records, not kernels) are dropped first, and the join is refused if the kernel
names of the profile and of the trace disagree.
"""

import argparse
import csv
import glob
import os
import re
import statistics

from . import cu_need

FLOP_COUNTERS = ("ADD_F32", "MUL_F32", "FMA_F32", "ADD_F16", "MUL_F16", "FMA_F16",
                 "MFMA_MOPS_BF16", "MFMA_MOPS_F32")
PASSES = {
    "trace": ["--kernel-trace"],
    "fetch": ["--pmc", "FETCH_SIZE"],
    "write": ["--pmc", "WRITE_SIZE"],
    "mfma": ["--pmc", "MfmaUtil"],
}
# Not among the passes `collect` runs: a pass with these eight SQ counters over
# a training client (about 8500 dispatches) made no progress for three minutes
# on the MI355X box and was killed.  `merge` still uses a flops/ directory when
# a user has collected one (fewer counters per pass, or fewer iterations).
FLOPS_PASS = ["--pmc"] + ["SQ_INSTS_VALU_" + c for c in FLOP_COUNTERS]
HBM_PEAK_BYTES_PER_NS = 8000.0          # 8 TB/s
FETCH_UNIT_BYTES = 2048.0               # FETCH_SIZE unit, from a copy kernel of known size
WRITE_UNIT_BYTES = 1024.0               # WRITE_SIZE unit


def short_name(full):
    """The name the capture layer records: demangled, anonymous namespaces
    removed, cut at the first template or call bracket, commas replaced."""
    s = full.replace("(anonymous namespace)::", "")
    m = re.search(r"[<(]", s)
    if m and m.start() > 0:
        s = s[:m.start()]
    return s.replace(",", ";").strip()


def _find(directory, suffix):
    hits = glob.glob(os.path.join(directory, "**", "*" + suffix), recursive=True)
    if not hits:
        raise FileNotFoundError(f"no *{suffix} under {directory}")
    return hits[0]


def _user_kernels(rows):
    return [r for r in rows if not r["Kernel_Name"].startswith("__amd_rocclr_")]


def read_kernel_trace(directory):
    with open(_find(directory, "_kernel_trace.csv")) as f:
        rows = sorted(csv.DictReader(f), key=lambda r: int(r["Dispatch_Id"]))
    return _user_kernels(rows)


def read_counter(directory, counter):
    """Per-dispatch values of one counter, in dispatch order."""
    by_dispatch = {}
    with open(_find(directory, "_counter_collection.csv")) as f:
        for r in csv.DictReader(f):
            if r["Counter_Name"] == counter:
                by_dispatch[int(r["Dispatch_Id"])] = r
    rows = [by_dispatch[k] for k in sorted(by_dispatch)]
    return _user_kernels(rows)


def read_profile(path):
    with open(path) as f:
        lines = f.read().splitlines()
    return [l.split(",") for l in lines[1:]]


def trailing_iterations(rows, n_rows, names, max_iters=5):
    """Split the tail of a dispatch list into iterations of n_rows kernels whose
    short names equal ``names``; returns the list of iterations (newest last)."""
    out = []
    end = len(rows)
    while end - n_rows >= 0 and len(out) < max_iters:
        chunk = rows[end - n_rows:end]
        if [short_name(r["Kernel_Name"]) for r in chunk] != names:
            break
        out.append(chunk)
        end -= n_rows
    return list(reversed(out))


def merge(profile_path, rocprof_dir, out_path, threshold=0.6):
    prof = read_profile(profile_path)
    names = [r[0] for r in prof]
    n = len(prof)
    trace = trailing_iterations(read_kernel_trace(os.path.join(rocprof_dir, "trace")), n, names)
    if not trace:
        raise RuntimeError("the kernel trace does not end with the profile's kernel sequence")
    dur = [statistics.median(float(it[i]["End_Timestamp"]) - float(it[i]["Start_Timestamp"])
                             for it in trace) for i in range(n)]

    def counter(sub, name):
        d = os.path.join(rocprof_dir, sub)
        if not os.path.isdir(d):
            return None
        its = trailing_iterations(read_counter(d, name), n, names)
        if not its:
            raise RuntimeError(f"{name}: counter run does not end with the profile's kernels")
        return [statistics.median(float(it[i]["Counter_Value"]) for it in its) for i in range(n)]

    fetch = counter("fetch", "FETCH_SIZE")
    write = counter("write", "WRITE_SIZE")
    mfma = counter("mfma", "MfmaUtil")
    fl = {c: counter("flops", "SQ_INSTS_VALU_" + c) for c in FLOP_COUNTERS}
    rows, stats = [], {"compute": 0, "memory": 0, "unknown": 0}
    last = trace[-1]
    for i, r in enumerate(prof):
        hbm_frac = mfma_frac = None
        if fetch is not None and write is not None:
            bytes_moved = fetch[i] * FETCH_UNIT_BYTES + write[i] * WRITE_UNIT_BYTES
            hbm_frac = bytes_moved / max(dur[i], 1.0) / HBM_PEAK_BYTES_PER_NS
        if mfma is not None:
            mfma_frac = mfma[i] / 100.0
        if fetch is not None and write is not None and all(v is not None for v in fl.values()):
            # wave-level instruction counts: 64 lanes each, an FMA is two flops;
            # one MFMA "MOPS" unit is 512 operations
            v32 = 64.0 * (fl["ADD_F32"][i] + fl["MUL_F32"][i] + 2 * fl["FMA_F32"][i])
            v16 = 64.0 * (fl["ADD_F16"][i] + fl["MUL_F16"][i] + 2 * fl["FMA_F16"][i])
            cls = cu_need.classify_roofline(
                bytes_moved, v32, v16, 512.0 * fl["MFMA_MOPS_F32"][i],
                512.0 * fl["MFMA_MOPS_BF16"][i], hbm_frac, mfma_frac, threshold)
        else:
            cls = cu_need.classify(r[0], hbm_frac, mfma_frac, threshold)
        k = last[i]
        threads = int(k["Workgroup_Size_X"]) * int(k["Workgroup_Size_Y"]) * int(k["Workgroup_Size_Z"])
        grid = int(k["Grid_Size_X"]) * int(k["Grid_Size_Y"]) * int(k["Grid_Size_Z"])
        regs = int(k["VGPR_Count"]) + int(k["Accum_VGPR_Count"])
        need = cu_need.cu_needed(max(1, grid // max(1, threads)), threads, regs,
                                 int(k["LDS_Block_Size"]))
        rows.append((r[0], cls, r[2], need, max(1, int(round(dur[i])))))
        stats[{1: "compute", 0: "memory", -1: "unknown"}[cls]] += 1
    with open(out_path, "w") as f:
        f.write("Name,Profile,Memory_footprint,SM_usage,Duration\n")
        for row in rows:
            f.write(",".join(str(x) for x in row) + "\n")
    stats["rows"] = n
    stats["iterations_joined"] = len(trace)
    stats["duration_ms"] = sum(dur) / 1e6
    return stats


def collect(config, client, rocprof_dir, iters=12, timeout=300):
    """Run the four rocprofv3 passes over the standalone client.  The caller
    must not have touched the GPU (the profiler starts a fresh process)."""
    import subprocess
    pkg_root = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    env = dict(os.environ, TMPDIR="/tmp")
    env["PYTHONPATH"] = pkg_root + (":" + env["PYTHONPATH"] if env.get("PYTHONPATH") else "")
    env["LD_PRELOAD"] = ":".join(p for p in env.get("LD_PRELOAD", "").split(":")
                                 if p and "libinttemp.so" not in p)
    for name, flags in PASSES.items():
        out = os.path.join(os.path.abspath(rocprof_dir), name)
        os.makedirs(out, exist_ok=True)
        cmd = ["rocprofv3"] + flags + ["--output-format", "csv", "-d", out, "-o", "t", "--",
                                       "python3", "-m", "orion_amd.profiling.standalone",
                                       "--config", os.path.abspath(config), "--client",
                                       str(client), "--iters", str(iters)]
        with open(out + ".log", "w") as log:
            subprocess.run(cmd, check=True, cwd="/tmp", env=env, stdout=log,
                           stderr=subprocess.STDOUT, timeout=timeout)


def main(argv=None):
    p = argparse.ArgumentParser()
    p.add_argument("--collect", action="store_true",
                   help="run the rocprofv3 passes first (needs --config and --client)")
    p.add_argument("--config")
    p.add_argument("--client", type=int, default=0)
    p.add_argument("--profile", required=True, help="profile written by capture_profile")
    p.add_argument("--rocprof-dir", required=True, help="directory holding trace/ fetch/ write/ mfma/")
    p.add_argument("--out", required=True)
    p.add_argument("--threshold", type=float, default=0.6)
    a = p.parse_args(argv)
    if a.collect:
        collect(a.config, a.client, a.rocprof_dir)
    print(merge(a.profile, a.rocprof_dir, a.out, a.threshold))


if __name__ == "__main__":
    main()
