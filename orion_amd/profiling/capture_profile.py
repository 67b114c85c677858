"""Run one client alone under the interception layer and write its profile.

    LD_PRELOAD=$(python -m orion_amd.launch_jobs --print-preload) \\
    python -m orion_amd.profiling.capture_profile --config job.json --client 0 \\
        --out profiles/resnet50_32

The client runs the same loop it runs under the scheduler, so the number and
order of kernel-like records per iteration in the profile are, by construction,
what the scheduler will count (the reference matches Nsight output to
interposer records by hand, PROFILE.md:40-54).  Every kernel is timed with HIP
events attached to its launch; rocprofv3 counter columns can be merged in
afterwards (``orion_amd.profiling.rocprof``).

Outputs ``<out>_fwd`` for inference clients, ``<out>_fb0`` (first iteration) and
``<out>_fb1`` (steady state) for training clients, plus ``<out>.json`` naming
the row counts to put in the job file.
"""

import argparse
import csv
import ctypes
import json
import os
import statistics
import threading

from .. import scheduler_frontend as fe
from . import cu_need

HEADER = "Name,Profile,Memory_footprint,SM_usage,Duration"
GRAPH_LAUNCH = "hipGraphLaunch"      # name the capture gives a hipGraphLaunch record


def read_trace(path):
    iters = {}
    with open(path) as f:
        for row in csv.DictReader(f):
            iters.setdefault(int(row["iteration"]), []).append(row)
    return [iters[k] for k in sorted(iters)]


def profile_rows(reference_iter, all_iters):
    """One profile row per kernel record of ``reference_iter``; the duration is
    the median over every iteration with the same record sequence."""
    names = [r["name"] for r in reference_iter]
    same = [it for it in all_iters if [r["name"] for r in it] == names]
    out = []
    for i, r in enumerate(reference_iter):
        if r["name"] == GRAPH_LAUNCH:
            # a whole captured graph is one record: every CU, class unknown
            dur = statistics.median(float(it[i]["duration_ns"]) for it in same)
            out.append((r["name"], -1, 0, cu_need.TOTAL_CUS, max(1, int(round(dur)))))
            continue
        threads = int(r["block_x"]) * int(r["block_y"]) * int(r["block_z"])
        blocks = int(r["grid_x"]) * int(r["grid_y"]) * int(r["grid_z"])
        lds = int(r["dyn_lds"]) + int(r["static_lds"])
        need = cu_need.cu_needed(blocks, threads, int(r["regs"]), lds)
        dur = statistics.median(float(it[i]["duration_ns"]) for it in same)
        out.append((r["name"], cu_need.classify(r["name"]), 0, need, max(1, int(round(dur)))))
    return out


def write_profile(path, rows):
    with open(path, "w") as f:
        f.write(HEADER + "\n")
        for name, prof, mem, sm, dur in rows:
            f.write(f"{name},{prof},{mem},{sm},{dur}\n")


def capture(entry, out_prefix, iters=14, function_dict=None):
    """``entry`` is one element of a job file.  Returns the summary dict."""
    from ..launch_jobs import _function_dict, check_preloaded
    check_preloaded()
    function_dict = function_dict or _function_dict()
    sched = fe.load_scheduler_library()
    sched.orion_profile_begin.argtypes = [ctypes.c_int, ctypes.c_char_p]
    sched.orion_profile_run.argtypes = [ctypes.c_int]
    barriers = [threading.Barrier(2)]
    kwargs = dict(entry["args"])
    kwargs.update({"num_iters": iters, "local_rank": 0, "barriers": barriers,
                   "client_barrier": threading.Barrier(1), "tid": 0})
    # a profile run must not pace itself: closed loop
    kwargs["rps"] = 0
    os.environ.setdefault("ORION_RESULT_DIR", os.path.dirname(out_prefix) or ".")
    def target():
        try:
            function_dict[entry["arch"]](**kwargs)
        except BaseException:
            import traceback
            traceback.print_exc()
            print("orion: the profiled client failed; aborting", flush=True)
            os._exit(1)

    thread = threading.Thread(target=target)
    thread.start()
    trace_path = out_prefix + ".trace.csv"
    rc = sched.orion_profile_begin(thread.native_id, trace_path.encode())
    if rc != 0:
        raise RuntimeError(f"orion_profile_begin failed ({rc})")
    barriers[0].wait()
    for until in (1, 10, iters):
        sched.orion_profile_run(until)
        barriers[0].wait()
    sched.orion_profile_end()
    thread.join()

    its = read_trace(trace_path)
    train = bool(entry["args"]["train"])
    steady = its[-1]
    summary = {"arch": entry["arch"], "train": train, "iterations": len(its),
               "records_per_iteration": [len(it) for it in its]}
    steady_rows = profile_rows(steady, its[2:])
    first_rows = profile_rows(its[0], its[:1])
    summary["steady_duration_ms"] = sum(r[4] for r in steady_rows) / 1e6
    stable = all(len(it) == len(steady) for it in its[1:])
    summary["stable_after_first"] = stable
    if not stable:
        raise RuntimeError(f"record count varies between iterations: "
                           f"{summary['records_per_iteration']}")
    if train or len(its[0]) != len(steady):
        write_profile(out_prefix + "_fb0", first_rows)
        write_profile(out_prefix + "_fb1", steady_rows)
        summary.update(kernel_file=out_prefix + "_fb0", num_kernels=len(first_rows),
                       additional_kernel_file=out_prefix + "_fb1",
                       additional_num_kernels=len(steady_rows))
    else:
        write_profile(out_prefix + "_fwd", steady_rows)
        summary.update(kernel_file=out_prefix + "_fwd", num_kernels=len(steady_rows))
    with open(out_prefix + ".json", "w") as f:
        json.dump(summary, f, indent=1)
    return summary


def profile_name(entry):
    a = entry["args"]
    phase = "train" if a["train"] else "inf"
    # a HIP-graph client submits one record where the eager one submits hundreds:
    # the two must not share a profile
    graph = "_hipgraph" if a.get("hip_graph") else ""
    return (f"{a.get('model_name', entry['arch'])}_{a['batchsize']}_{a.get('dtype', 'fp32')}_"
            f"{phase}{graph}")


def fill_job(config_path, out_dir, filled_path, iters=14, quiet=False, use_rocprof=False):
    """Profile every client of a job file, each alone in a process of its own,
    and write a copy of the job file with kernel_file / num_kernels (and the
    additional_* pair) filled in."""
    import subprocess
    import sys
    from .. import _lib
    with open(config_path) as f:
        job = json.load(f)
    os.makedirs(out_dir, exist_ok=True)
    # the profiling children need the interception library preloaded; the caller
    # does not
    env = dict(os.environ)
    preload = [p for p in env.get("LD_PRELOAD", "").split(":") if p]
    if _lib.CAPTURE_LIB not in preload:
        env["LD_PRELOAD"] = ":".join(preload + [_lib.CAPTURE_LIB])
    done = {}
    for idx, entry in enumerate(job):
        prefix = os.path.abspath(os.path.join(out_dir, profile_name(entry)))
        if prefix not in done:
            cmd = [sys.executable, "-m", "orion_amd.profiling.capture_profile",
                   "--config", config_path, "--client", str(idx), "--out", prefix,
                   "--iters", str(iters)]
            if quiet:     # keep the caller's stdout clean; the log stays beside the profile
                with open(prefix + ".log", "w") as log:
                    subprocess.run(cmd, check=True, stdout=log, stderr=subprocess.STDOUT, env=env)
            else:
                subprocess.run(cmd, check=True, env=env)
            with open(prefix + ".json") as f:
                done[prefix] = json.load(f)
            if use_rocprof:
                # bound class, durations and register counts from rocprofv3
                from . import rocprof
                summary = done[prefix]
                steady = summary.get("additional_kernel_file", summary["kernel_file"])
                rdir = prefix + ".rocprof"
                rocprof.collect(config_path, idx, rdir)
                stats = rocprof.merge(steady, rdir, steady)
                if "additional_kernel_file" in summary:
                    import shutil
                    shutil.copyfile(steady, summary["kernel_file"])
                summary["rocprof"] = stats
                with open(prefix + ".json", "w") as f:
                    json.dump(summary, f, indent=1)
        summary = done[prefix]
        for key in ("kernel_file", "num_kernels", "additional_kernel_file",
                    "additional_num_kernels"):
            entry.pop(key, None)
            if key in summary:
                entry[key] = summary[key]
    with open(filled_path, "w") as f:
        json.dump(job, f, indent=1)
    return job


def main(argv=None):
    p = argparse.ArgumentParser()
    p.add_argument("--config", required=True, help="job file (JSON list)")
    p.add_argument("--client", type=int, default=0, help="index of the entry to profile")
    p.add_argument("--out", help="output prefix (one client)")
    p.add_argument("--iters", type=int, default=14)
    p.add_argument("--fill", help="profile every client and write the completed "
                                  "job file here (profiles go to --out-dir)")
    p.add_argument("--out-dir", default="profiles_gfx950")
    p.add_argument("--rocprof", action="store_true",
                   help="with --fill: also run rocprofv3 and take class, duration and "
                        "register counts from it")
    a = p.parse_args(argv)
    if a.fill:
        fill_job(a.config, a.out_dir, a.fill, a.iters, use_rocprof=a.rocprof)
        return
    import torch
    torch.cuda.set_device(0)
    with open(a.config) as f:
        entry = json.load(f)[a.client]
    print(json.dumps(capture(entry, a.out, a.iters)))


if __name__ == "__main__":
    main()
