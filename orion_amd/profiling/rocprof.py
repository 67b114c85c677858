"""Merge rocprofv3 measurements into a captured profile.

``capture_profile`` fixes the row order and count of a profile (what the
interception layer will see) and times kernels with HIP events.  This module
adds what only the profiler knows -- per-kernel traffic past the L2s, matrix-core
and vector-ALU busy time -- and from them the bound class.  Counterpart of the
reference's ``profiling/postprocessing/process_ncu.py`` and
``roofline_analysis.py`` (Nsight Compute metrics -> class, :37-71).

Collection: one rocprofv3 run per counter (from /tmp with TMPDIR=/tmp), each
over the same stand-alone client:

    rocprofv3 --kernel-trace --output-format csv -d D/trace -o t -- python3 -m orion_amd.profiling.standalone ...
    rocprofv3 --pmc FETCH_SIZE --output-format csv -d D/fetch -o t -- python3 -m orion_amd.profiling.standalone ...
    rocprofv3 --pmc WRITE_SIZE ... -d D/write ...
    rocprofv3 --pmc MfmaUtil   ... -d D/mfma  ...
    rocprofv3 --pmc VALUBusy   ... -d D/valu  ...

(``python -m orion_amd.profiling.rocprof --collect ...`` runs these five.)

Class.  The reference places a kernel left or right of the roofline's knee by
its arithmetic intensity (flops / DRAM bytes against 9.72 flop/byte,
roofline_analysis.py:51-62), i.e. it asks which of the two roofs the kernel is
closer to.  The same question is answered here from busy fractions, which one
counter each gives: the fraction of the kernel's time the matrix cores were
busy (MfmaUtil) against the fraction of the 8 TB/s the kernel's traffic past
the L2s amounts to.  Compute-bound (1) when the matrix-core fraction is the
larger one, memory-bound (0) otherwise, unknown (-1) when neither reaches 5 %
(a kernel that loads neither resource cannot contend for one).  The vector
ALUs' busy fraction (VALUBusy) counts address arithmetic and issue time as much
as arithmetic -- copy, concatenation, index and pooling kernels reach 0.3-0.6 of
it -- so it stands in for the matrix cores only for kernels whose name puts them
in a convolution or GEMM family (MIOpen's Winograd and naive convolutions do
their FMAs there, matrix cores idle).  The fractions are taken per kernel NAME, summed over all dispatches
of that name in the joined iterations, weighted by duration: a 5-microsecond
dispatch on its own says little, the family it belongs to does.  Rows whose name
no counter run covered fall back to the name table of ``cu_need.classify`` and
are counted as such in the returned statistics.

Counting floating-point instructions instead (SQ_INSTS_VALU_{ADD,MUL,FMA}_* and
SQ_INSTS_VALU_MFMA_MOPS_*: eight SQ counters in one pass) is not offered: such a
pass over a training client made no progress for three minutes on an MI355X and
had to be killed; ``collect`` refuses it.

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
import json
import os
import re
import statistics

from . import cu_need

PASSES = {
    "trace": ["--kernel-trace"],
    "fetch": ["--pmc", "FETCH_SIZE"],
    "write": ["--pmc", "WRITE_SIZE"],
    "mfma": ["--pmc", "MfmaUtil"],
    "valu": ["--pmc", "VALUBusy"],
}
REFUSED_PASSES = {
    "flops": "a pass with the eight SQ_INSTS_VALU_* flop counters over a training client made "
             "no progress for three minutes on an MI355X and was killed; classes come from "
             "the single-counter passes instead",
}
HBM_PEAK_BYTES_PER_NS = 8000.0          # 8 TB/s
FETCH_UNIT_BYTES = 2048.0               # FETCH_SIZE unit, from a copy kernel of known size
WRITE_UNIT_BYTES = 1024.0               # WRITE_SIZE unit
UTILISATION_FLOOR = 0.05


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


def compute_family(name):
    """True for names of convolution / GEMM / attention families: kernels whose
    arithmetic may run on the vector ALUs with the matrix cores idle (MIOpen's
    Winograd and naive convolutions do)."""
    low = name.lower()
    return any(h in low for h in cu_need.COMPUTE_HINTS)


def classify_utilisation(memory_fraction, mfma_fraction, valu_fraction=0.0, name=None,
                         floor=UTILISATION_FLOOR):
    """1 compute-bound, 0 memory-bound, -1 unknown: which roof the kernel is
    closer to (see the module docstring).

    The matrix cores are the compute roof.  Vector-ALU busy time counts address
    arithmetic and issue time as much as arithmetic -- copy, index and pooling
    kernels show 0.3-0.6 of it while doing next to no floating-point work (the
    reference asks for flop/byte right of the knee, or >= 60 % utilisation:
    roofline_analysis.py:51-66) -- so by itself it does not make a kernel
    compute-bound.  It counts only for a kernel whose name puts it in a
    convolution or GEMM family (``compute_family``).  Everything else is
    memory-bound when its traffic reaches the floor, else unknown."""
    if mfma_fraction >= floor and mfma_fraction > memory_fraction:
        return 1
    if (valu_fraction >= floor and valu_fraction > memory_fraction
            and name is not None and compute_family(name)):
        return 1
    return 0 if memory_fraction >= floor else -1


def merge(profile_path, rocprof_dir, out_path, use_name_hints=True, classes_out=None):
    """Writes ``out_path``: the profile's rows with duration and CU need from the
    kernel trace and the class from the counter runs.  ``use_name_hints=False``
    leaves rows that no counter covers unknown instead of consulting the name
    table.  ``classes_out`` (default ``out_path + ".classes.json"``) receives the
    per-name fractions the classes came from."""
    if os.path.isdir(os.path.join(rocprof_dir, "flops")):
        raise ValueError("a flops/ directory is not used: " + REFUSED_PASSES["flops"])
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
    valu = counter("valu", "VALUBusy")
    have_memory = fetch is not None and write is not None
    have_compute = mfma is not None or valu is not None
    # per kernel name: bytes, time, busy time of the matrix cores and vector ALUs
    family = {}
    for i, name in enumerate(names):
        f = family.setdefault(name, {"ns": 0.0, "bytes": 0.0, "mfma_ns": 0.0, "valu_ns": 0.0,
                                     "dispatches": 0})
        f["ns"] += dur[i]
        f["dispatches"] += 1
        if have_memory:
            f["bytes"] += fetch[i] * FETCH_UNIT_BYTES + write[i] * WRITE_UNIT_BYTES
        if mfma is not None:
            f["mfma_ns"] += mfma[i] / 100.0 * dur[i]
        if valu is not None:
            f["valu_ns"] += valu[i] / 100.0 * dur[i]
    classes = {}
    for name, f in family.items():
        entry = {"dispatches": f["dispatches"], "ns": f["ns"]}
        if have_memory and have_compute:
            ns = max(f["ns"], 1.0)
            entry["memory_fraction"] = f["bytes"] / ns / HBM_PEAK_BYTES_PER_NS
            entry["mfma_fraction"] = f["mfma_ns"] / ns
            entry["valu_fraction"] = f["valu_ns"] / ns
            entry["class"] = classify_utilisation(
                entry["memory_fraction"], entry["mfma_fraction"], entry["valu_fraction"], name)
            entry["source"] = "counters"
        elif use_name_hints:
            entry["class"] = cu_need.classify(name)
            entry["source"] = "name"
        else:
            entry["class"] = -1
            entry["source"] = "none"
        classes[name] = entry
    rows = []
    stats = {"compute": 0, "memory": 0, "unknown": 0, "from_counters": 0, "from_names": 0}
    unknown_ns = 0.0
    last = trace[-1]
    for i, r in enumerate(prof):
        entry = classes[r[0]]
        cls = entry["class"]
        k = last[i]
        threads = int(k["Workgroup_Size_X"]) * int(k["Workgroup_Size_Y"]) * int(k["Workgroup_Size_Z"])
        grid = int(k["Grid_Size_X"]) * int(k["Grid_Size_Y"]) * int(k["Grid_Size_Z"])
        regs = int(k["VGPR_Count"]) + int(k["Accum_VGPR_Count"])
        need = cu_need.cu_needed(max(1, grid // max(1, threads)), threads, regs,
                                 int(k["LDS_Block_Size"]))
        rows.append((r[0], cls, r[2], need, max(1, int(round(dur[i])))))
        stats[{1: "compute", 0: "memory", -1: "unknown"}[cls]] += 1
        stats["from_counters"] += entry["source"] == "counters"
        stats["from_names"] += entry["source"] == "name"
        if cls == -1:
            unknown_ns += dur[i]
    with open(out_path, "w") as f:
        f.write("Name,Profile,Memory_footprint,SM_usage,Duration\n")
        for row in rows:
            f.write(",".join(str(x) for x in row) + "\n")
    with open(classes_out or out_path + ".classes.json", "w") as f:
        json.dump(classes, f, indent=1, sort_keys=True)
    stats["rows"] = n
    stats["iterations_joined"] = len(trace)
    stats["duration_ms"] = sum(dur) / 1e6
    stats["unknown_time_fraction"] = unknown_ns / max(sum(dur), 1.0)
    return stats


def build_table(class_files, out_path):
    """Joins the per-name fractions of several merged profiles (``*.classes.json``)
    into one table, name -> class, weighting every workload by the time it spent
    in the kernel: the table ``cu_need.classify`` consults before its name hints."""
    acc = {}
    for path in class_files:
        with open(path) as f:
            for name, e in json.load(f).items():
                if e.get("source") != "counters":
                    continue
                a = acc.setdefault(name, {"ns": 0.0, "memory": 0.0, "mfma": 0.0, "valu": 0.0,
                                          "dispatches": 0})
                a["ns"] += e["ns"]
                a["dispatches"] += e["dispatches"]
                a["memory"] += e["memory_fraction"] * e["ns"]
                a["mfma"] += e["mfma_fraction"] * e["ns"]
                a["valu"] += e["valu_fraction"] * e["ns"]
    table = {}
    for name, a in sorted(acc.items()):
        ns = max(a["ns"], 1.0)
        mem, mfma, valu = a["memory"] / ns, a["mfma"] / ns, a["valu"] / ns
        table[name] = {"class": classify_utilisation(mem, mfma, valu, name),
                       "memory_fraction": round(mem, 4), "mfma_fraction": round(mfma, 4),
                       "valu_fraction": round(valu, 4), "dispatches": a["dispatches"]}
    with open(out_path, "w") as f:
        json.dump(table, f, indent=0, sort_keys=True)
        f.write("\n")
    return table


def table_for_jobs(job_files, workdir, out_path, iters=12, log=print):
    """The whole pipeline for every distinct client of the given job files:
    capture its profile under the interception layer, run the rocprofv3 passes
    over it stand-alone, merge, and join all of them into the class table
    ``out_path``.  Per client ``workdir/<profile name>/`` keeps the merged
    profile, ``merged.classes.json`` and ``stats.json``; the profiler's raw
    output is deleted.  The caller must not have touched the GPU."""
    import shutil
    from . import capture_profile
    clients = {}
    for path in job_files:
        with open(path) as f:
            for entry in json.load(f):
                entry = dict(entry, num_iters=30)
                clients.setdefault(capture_profile.profile_name(entry), entry)
    os.makedirs(workdir, exist_ok=True)
    class_files, summary = [], {}
    for name, entry in clients.items():
        wd = os.path.join(os.path.abspath(workdir), name)
        os.makedirs(wd, exist_ok=True)
        cfg = os.path.join(wd, "job.json")
        with open(cfg, "w") as f:
            json.dump([entry], f)
        rdir = os.path.join(wd, "rocprof")
        try:
            filled = capture_profile.fill_job(cfg, wd, os.path.join(wd, "filled.json"),
                                              quiet=True, reuse=True)
            profile = filled[0].get("additional_kernel_file", filled[0]["kernel_file"])
            collect(cfg, 0, rdir, iters=iters)
            stats = merge(profile, rdir, os.path.join(wd, "merged"))
        except Exception as e:      # one client that cannot be joined does not end the rest
            log(f"{name}: skipped ({type(e).__name__}: {e})")
            summary[name] = {"skipped": str(e)}
            continue
        finally:
            shutil.rmtree(rdir, ignore_errors=True)
        with open(os.path.join(wd, "stats.json"), "w") as f:
            json.dump(stats, f)
        log(f"{name}: {stats}")
        summary[name] = stats
        class_files.append(os.path.join(wd, "merged.classes.json"))
    table = build_table(class_files, out_path)
    return table, summary


def collect(config, client, rocprof_dir, iters=12, timeout=300, passes=None):
    """Run the rocprofv3 passes over the standalone client, one run per counter.
    The caller must not have touched the GPU (the profiler starts a fresh
    process)."""
    import subprocess
    passes = list(passes or PASSES)
    for name in passes:
        if name in REFUSED_PASSES:
            raise ValueError(f"pass {name!r} is not run: {REFUSED_PASSES[name]}")
        if name not in PASSES:
            raise ValueError(f"unknown pass {name!r}")
    pkg_root = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    env = dict(os.environ, TMPDIR="/tmp")
    env["PYTHONPATH"] = pkg_root + (":" + env["PYTHONPATH"] if env.get("PYTHONPATH") else "")
    env["LD_PRELOAD"] = ":".join(p for p in env.get("LD_PRELOAD", "").split(":")
                                 if p and "libinttemp.so" not in p)
    for name in passes:
        flags = PASSES[name]
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
    p.add_argument("--iters", type=int, default=12)
    p.add_argument("--profile", help="profile written by capture_profile")
    p.add_argument("--rocprof-dir", help="directory holding trace/ fetch/ write/ mfma/ valu/")
    p.add_argument("--out")
    p.add_argument("--build-table", nargs="+", metavar="CLASSES_JSON",
                   help="join *.classes.json files of merged profiles into the name -> class "
                        "table written to --out")
    p.add_argument("--jobs", nargs="+", metavar="JOB_JSON",
                   help="capture, profile and merge every client of these job files (in "
                        "--workdir) and write the class table to --out")
    p.add_argument("--workdir", default="kernel_classes_work")
    a = p.parse_args(argv)
    if a.jobs:
        table, _ = table_for_jobs(a.jobs, a.workdir, a.out, iters=a.iters)
        counts = {c: sum(1 for v in table.values() if v["class"] == c) for c in (1, 0, -1)}
        print(f"{len(table)} kernel names -> {a.out}: {counts[1]} compute-bound, "
              f"{counts[0]} memory-bound, {counts[-1]} unknown")
        return
    if a.build_table:
        table = build_table(a.build_table, a.out)
        print(f"{len(table)} kernel names -> {a.out}")
        return
    if a.collect:
        collect(a.config, a.client, a.rocprof_dir, iters=a.iters)
    print(merge(a.profile, a.rocprof_dir, a.out))


if __name__ == "__main__":
    main()
