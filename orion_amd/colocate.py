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


def experiment(job, algo="orion", max_be_duration=100_000, workdir=None,
               be_isolated_iters=60, env=None, skip_isolated=False):
    workdir = workdir or tempfile.mkdtemp(prefix="orion_colocate_")
    hp = job[-1]
    result = {"algo": algo, "max_be_duration_ns": max_be_duration, "workdir": workdir}
    if not skip_isolated:
        iso_hp = run_job([copy.deepcopy(hp)], algo, os.path.join(workdir, "iso_hp"),
                         max_be_duration, env=env)[0]
        result["hp_isolated"] = iso_hp
        result["be_isolated"] = []
        for k, be in enumerate(job[:-1]):
            entry = copy.deepcopy(be)
            entry["num_iters"] = be_isolated_iters
            result["be_isolated"].append(
                run_job([entry], algo, os.path.join(workdir, f"iso_be{k}"),
                        max_be_duration, env=env)[0])
    if len(job) > 1:
        co = run_job(copy.deepcopy(job), algo, os.path.join(workdir, "colocated"),
                     max_be_duration, env=env)
        result["hp_colocated"] = co[-1]
        result["be_colocated"] = co[:-1]
        if not skip_isolated:
            if "p99_latency" in co[-1] and "p99_latency" in result["hp_isolated"]:
                for p in ("p50", "p95", "p99"):
                    result[f"hp_{p}_ratio"] = (co[-1][f"{p}_latency"]
                                               / result["hp_isolated"][f"{p}_latency"])
            else:
                result["hp_throughput_retained"] = (
                    co[-1]["throughput"] / result["hp_isolated"]["throughput"])
            result["be_retained"] = [
                c["throughput"] / i["throughput"] if i["throughput"] > 0 else 0.0
                for c, i in zip(co[:-1], result["be_isolated"])]
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
