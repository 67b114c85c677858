"""The sweep driver's bookkeeping (the reference's figure drivers,
artifact_evaluation/fig7/run_orion.py:5-33): which runs are started, and the
CSV row built from the clients' result files -- checked with stand-in runners,
closed forms only."""

import csv
import json

from orion_amd import sweep


def test_rows_and_summary(tmp_path):
    calls = []

    def fill_job(cfg, profiles, filled, quiet=False):
        return [{"arch": "be", "num_iters": 10 ** 6}, {"arch": "be2", "num_iters": 10 ** 6},
                {"arch": "hp", "num_iters": 100}]

    def run_job(job, algo, workdir, budget, reef_depth=12):
        calls.append((len(job), algo, budget, workdir.rsplit("/", 1)[-1]))
        if len(job) == 1:
            if job[0]["arch"] == "hp":
                return [{"p50_latency": 4.0, "p95_latency": 8.0, "p99_latency": 10.0,
                         "throughput": 80.0}]
            assert job[0]["num_iters"] == 60          # best-effort alone: bounded run
            return [{"throughput": 50.0 if job[0]["arch"] == "be" else 20.0}]
        run = int(workdir.rsplit("_", 1)[-1])
        return [{"throughput": 25.0 + run}, {"throughput": 5.0},
                {"p50_latency": 4.4, "p95_latency": 9.0, "p99_latency": 11.0 + run,
                 "throughput": 79.0}]

    out = tmp_path / "s.csv"
    rows = sweep.sweep(["a/pair.json"], ["orion", "reef"], [100000, 400000], 3, str(out),
                       workdir=str(tmp_path / "w"), run_job=run_job, fill_job=fill_job)
    # isolated: HP once, each BE once; orion: 2 budgets x 3 runs; reef: 1 x 3
    assert [c[:3] for c in calls[:3]] == [(1, "orion", 100000)] * 3
    assert len(calls) == 3 + 6 + 3
    assert [c[1:3] for c in calls[3:]] == [("orion", 100000)] * 3 + [("orion", 400000)] * 3 \
        + [("reef", 100000)] * 3
    assert len(rows) == 9
    got = list(csv.DictReader(open(out)))
    assert len(got) == 9 and list(got[0].keys()) == sweep.FIELDS
    r = got[1]
    assert (r["config"], r["algo"], r["budget_ns"], r["run"]) == ("pair", "orion", "100000", "1")
    assert float(r["hp_p99_ratio"]) == 12.0 / 10.0
    assert r["be_retained"] == "0.520;0.250" and r["be_iso_throughput"] == "50.000;20.000"
    summary = sweep.summarise(rows)
    assert len(summary) == 3
    cell = [s for s in summary if s["algo"] == "orion" and s["budget_ns"] == 400000][0]
    assert cell["runs"] == 3 and cell["hp_p99_ms"] == 12.0 and cell["be_retained_first"] == 0.52
    json.dumps(summary)
