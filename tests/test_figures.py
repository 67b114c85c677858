"""The figure-7 / figure-10 job sets against the reference's own job files, and
the driver's bookkeeping with stand-in runs."""

import csv
import json
import os
import re

import pytest

from orion_amd import figures, launch_jobs


@pytest.mark.parametrize("figure", [7, 10])
def test_pairs_match_the_references_job_files(reference_root, figure):
    ref_dir = os.path.join(reference_root, "artifact_evaluation", f"fig{figure}", "config_files")
    ours = figures.jobs(figure)
    names = sorted(f[:-5] for f in os.listdir(ref_dir) if f.endswith(".json"))
    assert sorted(ours) == names and len(names) == 10
    for name, (job, _) in ours.items():
        with open(os.path.join(ref_dir, name + ".json")) as f:
            ref = json.load(f)
        assert len(job) == len(ref) == 2
        for mine, theirs in zip(job, ref):
            assert mine["arch"] == theirs["arch"]
            assert mine["args"]["train"] == theirs["args"]["train"]
            assert mine["args"]["batchsize"] == theirs["args"]["batchsize"]
            assert mine["args"].get("model_name") == theirs["args"].get("model_name")
        # best-effort inference runs at a uniform rate there too
        if figure == 10:
            assert job[0]["args"]["uniform"] and ref[0]["args"]["uniform"]
        launch_jobs.job_lists(job)          # the launcher accepts it


def test_budgets_are_the_references(reference_root):
    text = open(os.path.join(reference_root, "artifact_evaluation", "fig7", "run_orion.py")).read()
    ref = {m.group(1): int(m.group(2))
           for m in re.finditer(r'"(\w+)",\s*(\d+)\)', text)}
    assert len(ref) == 10
    assert {name: budget for name, (_, budget) in figures.jobs(7).items()} == ref


def test_trace_replaces_poisson_arrivals():
    job, _ = figures.jobs(10, hp_requests=100, hp_trace="/tmp/trace.json")["trans_rnet"]
    assert job[-1]["args"]["input_file"] == "/tmp/trace.json" and job[-1]["args"]["rps"] == 0
    assert job[-1]["num_iters"] == 110
    with pytest.raises(ValueError):
        figures.jobs(8)


def test_driver_writes_one_row_per_pair(tmp_path):
    seen = []

    def fill_job(cfg, profile_dir, out, quiet=True):
        job = json.load(open(cfg))
        for k, c in enumerate(job):
            c["num_kernels"] = 100 + k
        job[0]["additional_num_kernels"] = 700
        return job

    def experiment(job, algo, budget, workdir, repeats, be_isolated_iters):
        seen.append((job[0]["arch"], job[-1]["arch"], budget, repeats, job[-1]["num_iters"]))
        return {"hp_isolated": {"p50_latency": 2.0, "p99_latency": 4.0},
                "hp_colocated": {"p50_latency": 2.2, "p99_latency": 4.4},
                "hp_p50_ratio": 1.1, "hp_p99_ratio": 1.1,
                "be_isolated": [{"throughput": 50.0}], "be_colocated": [{"throughput": 30.0}],
                "be_retained": [0.6]}

    rows = figures.run(7, str(tmp_path), pairs=["bert_mnet", "rnet_rnet"], hp_requests=400,
                       repeats=2, experiment=experiment, fill_job=fill_job, log=lambda *_: None)
    assert seen == [("resnet50", "resnet50", 160_000, 2, 210),
                    ("bert", "mobilenet_v2", 100_000, 2, 210)]
    with open(tmp_path / "fig7.csv") as f:
        got = list(csv.DictReader(f))
    assert [r["pair"] for r in got] == ["rnet_rnet", "bert_mnet"]
    assert got[0]["be_records"] == "700" and got[0]["hp_records"] == "101"
    assert float(got[1]["be_retained"]) == 0.6
    table = open(tmp_path / "fig7.md").read()
    assert "| rnet_rnet | 160 µs | 2.00 → 2.20 | 4.00 → 4.40 | 1.10 | 50.0 → 30.0 | 60 % |" in table
    assert rows[0]["pair"] == "rnet_rnet"
    with pytest.raises(KeyError):
        figures.run(7, str(tmp_path), pairs=["nope"], experiment=experiment, fill_job=fill_job)
    # every pair's budget scaled (the reference's own figures were chosen on a V100)
    del seen[:]
    figures.run(7, str(tmp_path / "scaled"), pairs=["bert_mnet", "rnet_rnet"], hp_requests=400,
                repeats=2, experiment=experiment, fill_job=fill_job, log=lambda *_: None,
                budget_scale=2.5)
    assert [s[2] for s in seen] == [400_000, 250_000]
    assert "| rnet_rnet | 400 µs |" in open(tmp_path / "scaled" / "fig7.md").read()


def test_hip_graph_and_other_policies_are_options_of_the_same_pairs(tmp_path):
    plain = figures.jobs(7)
    graph = figures.jobs(7, hp_hip_graph=True)
    for name in plain:
        assert graph[name][0][-1]["args"]["hip_graph"] is True
        assert "hip_graph" not in plain[name][0][-1]["args"]
        assert graph[name][0][0] == plain[name][0][0] and graph[name][1] == plain[name][1]
    calls = []

    def experiment(job, algo, budget, workdir, repeats, be_isolated_iters):
        calls.append((algo, job[0]["num_kernels"]))
        return {"hp_isolated": {"p50_latency": 1.0, "p99_latency": 2.0},
                "hp_colocated": {"p50_latency": 1.0, "p99_latency": 2.0},
                "hp_p50_ratio": 1.0, "hp_p99_ratio": 1.0,
                "be_isolated": [{"throughput": 1.0}], "be_colocated": [{"throughput": 1.0}],
                "be_retained": [1.0]}

    def no_profiles(*a, **k):
        raise AssertionError("the streams baseline needs no profiles")

    figures.run(7, str(tmp_path), pairs=["rnet_rnet"], algo="streams", experiment=experiment,
                fill_job=no_profiles, log=lambda *_: None)
    assert calls == [("streams", 0)]
    assert os.path.exists(tmp_path / "fig7_streams.csv") and os.path.exists(tmp_path / "fig7_streams.md")
