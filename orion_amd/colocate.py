"""Isolated-versus-co-located experiment on one GPU.

Runs a job file three ways, each in a fresh process with the interception
library preloaded: the high-priority client alone, every best-effort client
alone, and all of them together under the chosen policy.  Reports the
high-priority latency percentiles and every client's throughput, absolute and
as a fraction of the isolated run -- the quantities the reference's artifact
scripts gather from ``client_*.json`` (artifact_evaluation/fig7/run_orion.py:20-28,
gather_latency.py, gather_throughput.py).
"""

import argparse
import copy
import json
import os
import subprocess
import sys
import tempfile

import numpy as np

from . import _lib


def preload_env(extra=None):
    env = dict(os.environ)
    prev = env.get("LD_PRELOAD", "")
    if _lib.CAPTURE_LIB not in prev.split(":"):
        env["LD_PRELOAD"] = (prev + ":" if prev else "") + _lib.CAPTURE_LIB
    env.update(extra or {})
    return env


def run_job(job, algo, workdir, max_be_duration, reef_depth=12, env=None,
            timeout=900, log_name="launch.log", hp_limit=None, start_update=None):
    """One launcher process; returns the list of client result dicts.
    ``hp_limit`` (ms) and ``start_update`` (kernel index) are the launcher's
    --orion_hp_limit / --orion_start_update, used when the high-priority client
    trains."""
    os.makedirs(workdir, exist_ok=True)
    cfg = os.path.join(workdir, "job.json")
    with open(cfg, "w") as f:
        json.dump(job, f, indent=1)
    e = preload_env({"ORION_RESULT_DIR": workdir, "ORION_QUIET": "1"})
    if algo == "streams":      # the baseline without scheduler: no interception either
        e["LD_PRELOAD"] = ":".join(p for p in e.get("LD_PRELOAD", "").split(":")
                                   if p and p != _lib.CAPTURE_LIB)
    e.update(env or {})
    cmd = [sys.executable, "-u", "-m", "orion_amd.launch_jobs", "--algo", algo,
           "--config_file", cfg, "--orion_max_be_duration", str(max_be_duration),
           "--reef_depth", str(reef_depth)]
    if hp_limit is not None:
        cmd += ["--orion_hp_limit", str(hp_limit)]
    if start_update is not None:
        cmd += ["--orion_start_update", str(start_update)]
    with open(os.path.join(workdir, log_name), "w") as log:
        proc = subprocess.run(cmd, stdout=log, stderr=subprocess.STDOUT, env=e,
                              timeout=timeout,
                              cwd=os.path.dirname(_lib.PKG_DIR))
    if proc.returncode != 0:
        with open(os.path.join(workdir, log_name)) as log:
            tail = log.read()[-3000:]
        raise RuntimeError(f"launcher failed ({proc.returncode}) in {workdir}:\n{tail}")
    out = []
    for i in range(len(job)):
        with open(os.path.join(workdir, f"client_{i}.json")) as f:
            out.append(json.load(f))
    return out


def pooled(runs):
    """One result for a client measured in several runs: latency percentiles
    over all runs' requests together, throughput averaged."""
    out = {"throughput": sum(r["throughput"] for r in runs) / len(runs)}
    lat = [t for r in runs for t in r.get("latencies_ms", [])]
    if lat and all("latencies_ms" in r for r in runs):
        for p in (50, 95, 99):
            out[f"p{p}_latency"] = float(np.percentile(lat, p))
        out["requests"] = len(lat)
    elif "p99_latency" in runs[0]:
        assert len(runs) == 1
        out.update({k: runs[0][k] for k in ("p50_latency", "p95_latency", "p99_latency")})
    if len(runs) > 1:
        out["runs"] = [{k: r[k] for k in ("p50_latency", "p95_latency", "p99_latency",
                                          "throughput") if k in r} for r in runs]
    return out


def experiment(job, algo="orion", max_be_duration=100_000, workdir=None,
               be_isolated_iters=60, env=None, skip_isolated=False, repeats=1,
               be_isolated_known=None, plain_streams_too=False):
    """Runs the high-priority client alone, every best-effort client alone, and
    the whole job; reports the high-priority client's latency ratios and what
    each best-effort client keeps of its own throughput.

    With ``repeats`` > 1 the isolated and the co-located run of the high-priority
    client alternate that many times and their requests are pooled: the speed of
    one run drifts by 10-20 % on the same machine (clock and power state), which
    is as large as the effect being measured.

    ``be_isolated_known``: one entry per best-effort client, a result of an
    earlier isolated run of the same client under the same settings, or None to
    measure it here.

    ``plain_streams_too``: every repeat also runs the high-priority client alone
    on a plain stream, with no scheduler and no interception library in the
    process (``hp_plain_isolated`` in the result), and once more with its
    thread-local accesses kept on the loader's fast path as the library keeps a
    scheduled client's (``hp_plain_tls_fresh_isolated``): what the path itself
    costs the client, measured in the same alternation as everything else."""
    workdir = workdir or tempfile.mkdtemp(prefix="orion_colocate_")
    hp = job[-1]
    result = {"algo": algo, "max_be_duration_ns": max_be_duration, "workdir": workdir}
    env = dict(env or {})
    record_dir = env.pop("ORION_RECORD_DIR", None)
    if not skip_isolated:
        result["be_isolated"] = []
        for k, be in enumerate(job[:-1]):
            if be_isolated_known and be_isolated_known[k] is not None:
                result["be_isolated"].append(be_isolated_known[k])
                continue
            entry = copy.deepcopy(be)
            entry["num_iters"] = be_isolated_iters
            result["be_isolated"].append(
                run_job([entry], algo, os.path.join(workdir, f"iso_be{k}"),
                        max_be_duration, env=env)[0])
    iso_runs, co_runs, plain_runs, plain_fresh_runs = [], [], [], []
    for rep in range(repeats):
        tag = f"_{rep}" if repeats > 1 else ""
        if plain_streams_too:
            plain = copy.deepcopy(hp)
            plain["kernel_file"], plain["num_kernels"] = "", 0
            plain_runs.append(run_job([plain], "streams", os.path.join(workdir, "plain_hp" + tag),
                                      max_be_duration)[0])
            # the same, its thread-local accesses kept off the dynamic loader's
            # slow path the way the interception library keeps a scheduled
            # client's (csrc/capture/tls_fresh.h)
            plain_fresh_runs.append(
                run_job([copy.deepcopy(plain)], "streams",
                        os.path.join(workdir, "plain_fresh_hp" + tag), max_be_duration,
                        env={"ORION_PLAIN_TLS_REFRESH": "1"})[0])
        if not skip_isolated:
            iso_runs.append(run_job([copy.deepcopy(hp)], algo,
                                    os.path.join(workdir, "iso_hp" + tag),
                                    max_be_duration, env=env)[0])
        if len(job) > 1:
            co_env = dict(env)
            if record_dir and rep == repeats - 1:      # the last run keeps the logs
                co_env["ORION_RECORD_DIR"] = record_dir
            co_runs.append(run_job(copy.deepcopy(job), algo,
                                   os.path.join(workdir, "colocated" + tag),
                                   max_be_duration, env=co_env))
    if plain_runs:
        result["hp_plain_isolated"] = pooled(plain_runs)
        result["hp_plain_tls_fresh_isolated"] = pooled(plain_fresh_runs)
    if iso_runs:
        result["hp_isolated"] = pooled(iso_runs)
    if co_runs:
        result["hp_colocated"] = pooled([co[-1] for co in co_runs])
        result["be_colocated"] = [pooled([co[k] for co in co_runs])
                                  for k in range(len(job) - 1)]
        if iso_runs:
            iso, co_hp = result["hp_isolated"], result["hp_colocated"]
            if "p99_latency" in co_hp and "p99_latency" in iso:
                for p in ("p50", "p95", "p99"):
                    result[f"hp_{p}_ratio"] = co_hp[f"{p}_latency"] / iso[f"{p}_latency"]
            else:
                result["hp_throughput_retained"] = co_hp["throughput"] / iso["throughput"]
            result["be_retained"] = [
                c["throughput"] / i["throughput"] if i["throughput"] > 0 else 0.0
                for c, i in zip(result["be_colocated"], result["be_isolated"])]
    return result


def main(argv=None):
    p = argparse.ArgumentParser()
    p.add_argument("--config_file", required=True)
    p.add_argument("--algo", default="orion")
    p.add_argument("--orion_max_be_duration", type=int, default=100_000)
    p.add_argument("--workdir")
    a = p.parse_args(argv)
    with open(a.config_file) as f:
        job = json.load(f)
    print(json.dumps(experiment(job, a.algo, a.orion_max_be_duration, a.workdir), indent=1))


if __name__ == "__main__":
    main()
