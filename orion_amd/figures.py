"""The reference's two headline experiments as job sets for this GPU.

* figure 7 (inference beside training): a high-priority ResNet-50 or
  MobileNetV2 inference client, batch 4, open loop, beside one best-effort
  trainer out of ResNet-50 bs32, MobileNetV2 bs64, ResNet-101 bs32, BERT-base
  bs8 and Transformer-XL bs8 -- the ten pairs and the per-pair duration budget
  of artifact_evaluation/fig7/run_orion.py:5-16 and fig7/config_files/*.json.
* figure 10 (inference beside inference): the same two high-priority clients
  beside a best-effort *inference* client at a uniform request rate, batch 4
  (BERT: batch 2) -- fig10/config_files/*.json.

The pairs, batch sizes, training flags and budgets are the reference's.  Request
rates are this build's: the reference's (15 / 40 req/s high priority) load a
V100; on an MI355X the high-priority clients run at 80 (ResNet-50) and 100
(MobileNetV2) req/s, Poisson, bf16.  The reference's figure 10 drives the
high-priority client from a recorded trace (``inter_arrival_times.json``, 20.8
req/s on average); pass it with ``--hp-trace`` to do the same.

    LD_PRELOAD=... is not needed here: every run is a child process that the
    driver starts with the interception library preloaded.

    python -m orion_amd.figures --figure 7 --out fig7 [--pairs rnet_rnet bert_mnet]
        [--algo orion|reef|sequential|streams] [--hp-hip-graph]
        [--env ORION_RESERVE_HP_CUS=1 ...] [--budget-scale 2.5]
        [--hp-trace inter_arrival_times.json]
"""

import argparse
import csv
import json
import os

# best-effort client -> (arch, model_name, training batch, inference batch, inference req/s)
BEST_EFFORT = {
    "rnet": ("resnet50", "resnet50", 32, 4, 80),
    "mnet": ("mobilenet_v2", "mobilenet_v2", 64, 4, 100),
    "rnet101": ("resnet101", "resnet101", 32, 4, 40),
    "bert": ("bert", None, 8, 2, 8),
    "trans": ("transformer", None, 8, 4, 20),
}
# high-priority client -> (arch, req/s, duration budget in ns: run_orion.py:5-16)
HIGH_PRIORITY = {"rnet": ("resnet50", 80, 160_000), "mnet": ("mobilenet_v2", 100, 100_000)}


def _entry(arch, model_name, batch, rps, uniform, train, num_iters, dtype, trace=None):
    args = {"batchsize": batch, "rps": rps, "uniform": uniform, "dummy_data": True,
            "train": train, "dtype": dtype}
    if model_name:
        args["model_name"] = model_name
    if trace:
        args["input_file"] = trace
    return {"arch": arch, "kernel_file": "", "num_kernels": 0, "num_iters": num_iters,
            "args": args}


def jobs(figure, hp_requests=1200, hp_trace=None, hp_hip_graph=False):
    """name -> (job, duration budget): the last entry of a job is the
    high-priority client, as the launcher expects.  ``hp_hip_graph``: the
    high-priority client replays a captured HIP graph (one record per request)."""
    if figure not in (7, 10):
        raise ValueError("figure 7 (inference + training) or 10 (inference + inference)")
    out = {}
    for be_key, (arch, model, train_bs, inf_bs, inf_rps) in BEST_EFFORT.items():
        for hp_key, (hp_arch, hp_rps, budget) in HIGH_PRIORITY.items():
            if figure == 7:
                be = _entry(arch, model, train_bs, 0, False, True, 1_000_000, "fp32")
            else:
                be = _entry(arch, model, inf_bs, inf_rps, True, False, 1_000_000, "bf16")
            hp = _entry(hp_arch, hp_arch, 4, 0 if hp_trace else hp_rps, False, False,
                        hp_requests + 10, "bf16", trace=hp_trace)
            if hp_hip_graph:
                hp["args"]["hip_graph"] = True
            out[f"{be_key}_{hp_key}"] = ([be, hp], budget)
    return out


FIELDS = ["pair", "budget_ns", "hp_iso_p50_ms", "hp_iso_p99_ms", "hp_p50_ms", "hp_p99_ms",
          "hp_p50_ratio", "hp_p99_ratio", "be_iso", "be_colocated", "be_retained",
          "be_iso_p50_ms", "be_p50_ms", "hp_records", "be_records"]


def row_of(name, budget, res, filled):
    hi, hc = res["hp_isolated"], res["hp_colocated"]
    bi, bc = res["be_isolated"][0], res["be_colocated"][0]
    return {"pair": name, "budget_ns": budget,
            "hp_iso_p50_ms": hi["p50_latency"], "hp_iso_p99_ms": hi["p99_latency"],
            "hp_p50_ms": hc["p50_latency"], "hp_p99_ms": hc["p99_latency"],
            "hp_p50_ratio": res["hp_p50_ratio"], "hp_p99_ratio": res["hp_p99_ratio"],
            "be_iso": bi["throughput"], "be_colocated": bc["throughput"],
            "be_retained": res["be_retained"][0],
            "be_iso_p50_ms": bi.get("p50_latency"), "be_p50_ms": bc.get("p50_latency"),
            "hp_records": filled[-1]["num_kernels"],
            "be_records": filled[0].get("additional_num_kernels") or filled[0]["num_kernels"]}


def markdown(rows, figure):
    unit = "it/s" if figure == 7 else "req/s"
    lines = ["| pair (BE_HP) | budget | HP p50 iso → co (ms) | HP p99 iso → co (ms) | "
             f"p99 ratio | BE {unit} iso → co | BE kept |", "|---|---|---|---|---|---|---|"]
    for r in rows:
        lines.append(
            f"| {r['pair']} | {r['budget_ns'] // 1000} µs | {r['hp_iso_p50_ms']:.2f} → "
            f"{r['hp_p50_ms']:.2f} | {r['hp_iso_p99_ms']:.2f} → {r['hp_p99_ms']:.2f} | "
            f"{r['hp_p99_ratio']:.2f} | {r['be_iso']:.1f} → {r['be_colocated']:.1f} | "
            f"{100 * r['be_retained']:.0f} % |")
    return "\n".join(lines)


def run(figure, out_dir, pairs=None, hp_requests=1200, repeats=2, hp_trace=None,
        experiment=None, fill_job=None, log=print, algo="orion", hp_hip_graph=False,
        env=None, budget_scale=1.0):
    """``algo``: ``orion``, ``reef`` (depth 12), ``sequential``, or ``streams`` -- the
    same clients on plain streams with no scheduler, the reference's "Streams"
    baseline; it needs no profiles.  ``budget_scale`` multiplies every pair's
    duration budget (the reference's own per-pair figures were chosen on a
    V100)."""
    from . import colocate
    from .profiling import capture_profile
    experiment = experiment or colocate.experiment
    fill_job = fill_job or capture_profile.fill_job
    os.makedirs(out_dir, exist_ok=True)
    todo = jobs(figure, -(-hp_requests // repeats), hp_trace, hp_hip_graph)
    unknown = set(pairs or []) - set(todo)
    if unknown:
        raise KeyError(f"unknown pairs {sorted(unknown)}; known: {sorted(todo)}")
    rows = []
    suffix = ("" if algo == "orion" else "_" + algo) + ("_hip_graph" if hp_hip_graph else "")
    with open(os.path.join(out_dir, f"fig{figure}{suffix}.csv"), "w", newline="") as f:
        writer = csv.DictWriter(f, fieldnames=FIELDS)
        writer.writeheader()
        for name, (job, budget) in todo.items():
            if pairs and name not in pairs:
                continue
            budget = int(round(budget * budget_scale))
            base = os.path.join(out_dir, name)
            os.makedirs(base, exist_ok=True)
            cfg = os.path.join(base, "job.json")
            with open(cfg, "w") as jf:
                json.dump(job, jf, indent=1)
            if algo == "streams":
                filled = job
            else:
                filled = fill_job(cfg, os.path.join(base, "profiles"),
                                  os.path.join(base, "filled.json"), quiet=True)
            extra = {"env": dict(env)} if env else {}
            res = experiment(filled, algo, budget, base, repeats=repeats,
                             be_isolated_iters=60, **extra)
            row = row_of(name, budget, res, filled)
            writer.writerow(row)
            f.flush()
            rows.append(row)
            log(f"{name}: HP p99 x{row['hp_p99_ratio']:.2f}, BE keeps "
                f"{100 * row['be_retained']:.0f} %")
    with open(os.path.join(out_dir, f"fig{figure}{suffix}.md"), "w") as f:
        f.write(markdown(rows, figure) + "\n")
    return rows


def main(argv=None):
    p = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    p.add_argument("--figure", type=int, choices=[7, 10], required=True)
    p.add_argument("--out", required=True)
    p.add_argument("--pairs", nargs="*", help="subset, e.g. rnet_rnet bert_mnet (BE_HP)")
    p.add_argument("--hp-requests", type=int, default=1200)
    p.add_argument("--repeats", type=int, default=2)
    p.add_argument("--algo", default="orion",
                   choices=["orion", "reef", "sequential", "streams"],
                   help="policy, or streams: plain streams without a scheduler (baseline)")
    p.add_argument("--hp-hip-graph", action="store_true",
                   help="the high-priority client replays a captured HIP graph per request")
    p.add_argument("--env", nargs="*", default=[], metavar="KEY=VALUE",
                   help="environment of every run, e.g. ORION_MAX_SMS=8")
    p.add_argument("--budget-scale", type=float, default=1.0,
                   help="multiply every pair's duration budget (1.0 = the reference's own)")
    p.add_argument("--hp-trace", help="JSON list of inter-arrival times (s) for the "
                                      "high-priority client instead of Poisson arrivals")
    a = p.parse_args(argv)
    rows = run(a.figure, a.out, a.pairs, a.hp_requests, a.repeats, a.hp_trace, algo=a.algo,
               hp_hip_graph=a.hp_hip_graph, env=dict(kv.split("=", 1) for kv in a.env),
               budget_scale=a.budget_scale)
    print(markdown(rows, a.figure))


if __name__ == "__main__":
    main()
