"""Sweep driver: job files x policies x duration budgets x runs, one CSV row per
run -- the counterpart of the reference's figure drivers, which loop over its
job files and copy ``client_*.json`` away after every run
(artifact_evaluation/fig7/run_orion.py:5-33, fig10/run_orion.py).

    python -m orion_amd.sweep --configs orion_amd/configs/rnet_train_rnet_inf.json \\
        --algos orion reef --budgets 160000 --runs 3 --out results.csv

Every job file is profiled once on this GPU (``capture_profile.fill_job``), the
high-priority and best-effort clients are measured alone once, and every run is
one launcher process started the way a user starts it.
"""

import argparse
import copy
import csv
import json
import os
import statistics
import tempfile

FIELDS = ["config", "algo", "budget_ns", "run", "hp_p50_ms", "hp_p95_ms", "hp_p99_ms",
          "hp_throughput", "hp_iso_p50_ms", "hp_iso_p99_ms", "hp_p99_ratio",
          "be_throughput", "be_iso_throughput", "be_retained"]


def row_of(config, algo, budget, run, iso_hp, iso_be, colocated):
    """One CSV row from the client result dicts (``client_{tid}.json`` contents:
    reference train_imagenet.py:228-239).  ``colocated`` lists the clients in job
    order, the high-priority client last; ``iso_be`` the best-effort clients."""
    hp = colocated[-1]
    row = {"config": config, "algo": algo, "budget_ns": budget, "run": run,
           "hp_throughput": hp.get("throughput"),
           "be_throughput": ";".join(f"{c['throughput']:.3f}" for c in colocated[:-1]),
           "be_iso_throughput": ";".join(f"{c['throughput']:.3f}" for c in iso_be),
           "be_retained": ";".join(
               f"{c['throughput'] / i['throughput']:.3f}" if i["throughput"] > 0 else "nan"
               for c, i in zip(colocated[:-1], iso_be))}
    for p in ("p50", "p95", "p99"):
        row[f"hp_{p}_ms"] = hp.get(f"{p}_latency")
    row["hp_iso_p50_ms"] = iso_hp.get("p50_latency")
    row["hp_iso_p99_ms"] = iso_hp.get("p99_latency")
    if hp.get("p99_latency") and iso_hp.get("p99_latency"):
        row["hp_p99_ratio"] = hp["p99_latency"] / iso_hp["p99_latency"]
    return row


def summarise(rows):
    """Median over runs of every (config, algo, budget) cell."""
    cells = {}
    for r in rows:
        cells.setdefault((r["config"], r["algo"], r["budget_ns"]), []).append(r)
    out = []
    for (config, algo, budget), rs in sorted(cells.items()):
        med = {"config": config, "algo": algo, "budget_ns": budget, "runs": len(rs)}
        for key in ("hp_p50_ms", "hp_p99_ms", "hp_p99_ratio"):
            vals = [r[key] for r in rs if r.get(key) is not None]
            med[key] = statistics.median(vals) if vals else None
        first = [float(r["be_retained"].split(";")[0]) for r in rs if r["be_retained"]]
        med["be_retained_first"] = statistics.median(first) if first else None
        out.append(med)
    return out


def sweep(configs, algos, budgets, runs, out_csv, workdir=None, reef_depth=12, run_job=None,
          fill_job=None, be_isolated_iters=60):
    from . import colocate
    from .profiling import capture_profile
    run_job = run_job or colocate.run_job
    fill_job = fill_job or capture_profile.fill_job
    workdir = workdir or tempfile.mkdtemp(prefix="orion_sweep_")
    rows = []
    with open(out_csv, "w", newline="") as f:
        writer = csv.DictWriter(f, fieldnames=FIELDS)
        writer.writeheader()
        for cfg in configs:
            name = os.path.splitext(os.path.basename(cfg))[0]
            base = os.path.join(workdir, name)
            os.makedirs(base, exist_ok=True)
            job = fill_job(cfg, os.path.join(base, "profiles"),
                           os.path.join(base, "filled.json"), quiet=True)
            iso_hp = run_job([copy.deepcopy(job[-1])], "orion", os.path.join(base, "iso_hp"),
                             budgets[0])[0]
            iso_be = []
            for k, be in enumerate(job[:-1]):
                entry = copy.deepcopy(be)
                entry["num_iters"] = be_isolated_iters
                iso_be.append(run_job([entry], "orion", os.path.join(base, f"iso_be{k}"),
                                      budgets[0])[0])
            for algo in algos:
                for budget in (budgets if algo == "orion" else budgets[:1]):
                    for run in range(runs):
                        d = os.path.join(base, f"{algo}_{budget}_{run}")
                        co = run_job(copy.deepcopy(job), algo, d, budget, reef_depth=reef_depth)
                        row = row_of(name, algo, budget, run, iso_hp, iso_be, co)
                        writer.writerow(row)
                        f.flush()
                        rows.append(row)
    return rows


def main(argv=None):
    p = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    p.add_argument("--configs", nargs="+", required=True)
    p.add_argument("--algos", nargs="+", default=["orion"],
                   choices=["orion", "reef", "sequential"])
    p.add_argument("--budgets", nargs="+", type=int, default=[160000],
                   help="--orion_max_be_duration values (ns); other policies run once")
    p.add_argument("--runs", type=int, default=3)
    p.add_argument("--reef_depth", type=int, default=12)
    p.add_argument("--out", default="sweep.csv")
    p.add_argument("--workdir")
    a = p.parse_args(argv)
    rows = sweep(a.configs, a.algos, a.budgets, a.runs, a.out, a.workdir, a.reef_depth)
    print(json.dumps(summarise(rows), indent=1))


if __name__ == "__main__":
    main()
