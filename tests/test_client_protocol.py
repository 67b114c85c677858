"""The Python side of the path: arrival schedules, latency accounting, the
request loop's barrier protocol, job-file handling, front-end marshalling.
Pinned by closed forms and by the reference's own job files and arrival trace
read in place (reference: benchmarking/benchmark_suite/train_imagenet.py:71-241,
benchmarking/launch_jobs.py:44-148, src/scheduler_frontend.py:17-94)."""

import glob
import json
import os
import threading

import numpy as np
import pytest

from orion_amd import launch_jobs
from orion_amd.benchmark_suite import client_common as cc


def test_arrival_gaps_closed_forms():
    assert cc.arrival_gaps(50, True, 4) == [0.02] * 4
    assert cc.arrival_gaps(0, False, 3) == [0.0] * 3
    # the reference seeds numpy's global generator with 42 and then draws
    # np.random.exponential(scale=1/rps, size=num_iters) (:22-30, :93)
    np.random.seed(42)
    want = np.random.exponential(scale=1 / 80, size=100)
    assert np.array_equal(np.asarray(cc.arrival_gaps(80, False, 100)), want)
    assert abs(np.mean(cc.arrival_gaps(80, False, 200_000)) - 1 / 80) < 1e-4


def test_arrival_trace_file(reference_root, tmp_path):
    path = os.path.join(reference_root, "artifact_evaluation", "fig10", "inter_arrival_times.json")
    gaps = cc.arrival_gaps(15, False, 10, input_file=path)
    assert len(gaps) == 6240
    assert sum(gaps) == pytest.approx(299.733, abs=1e-3)
    assert np.mean(gaps) == pytest.approx(0.0480, abs=1e-4)


def test_latency_summary_closed_forms():
    timings = [9.0] * 10 + [i / 1000 for i in range(1, 101)]     # 1..100 ms after warm-up
    res = cc.latency_summary(timings, batch_idx=110, total_time=2.0, train=False)
    assert res["p50_latency"] == pytest.approx(50.5)
    assert res["p95_latency"] == pytest.approx(95.05)
    assert res["p99_latency"] == pytest.approx(99.01)
    assert res["throughput"] == pytest.approx((110 - 10) / 2.0)      # :232
    assert cc.latency_summary(timings, 110, 2.0, train=True) == {"throughput": 50.0}
    # BERT inference drops 50 requests (bert_trainer_mock.py:213-214)
    res = cc.latency_summary([9.0] * 50 + [0.002] * 20, 70, 1.0, False, drop=50)
    assert res["p99_latency"] == pytest.approx(2.0)


class FakeBackend:
    def __init__(self, stop_after=None):
        self.blocked = []
        self.stop_after = stop_after

    def block(self, it):
        self.blocked.append(it)

    def stop(self):
        return self.stop_after is not None and len(self.blocked) >= self.stop_after


class CountingBarrier:
    def __init__(self):
        self.waits_at = []
        self.owner = None

    def wait(self):
        self.waits_at.append(len(self.owner.blocked))


def _run(train, num_iters, rps=0, stop_after=None, tmp_path=None):
    backend = FakeBackend(stop_after)
    barrier = CountingBarrier()
    barrier.owner = backend
    os.environ["ORION_RESULT_DIR"] = str(tmp_path)
    steps = []
    res = cc.run_client(7, train, num_iters, cc.arrival_gaps(rps, True, num_iters), [barrier],
                        steps.append, backend)
    return res, steps, backend, barrier


def test_request_loop_protocol_training(tmp_path):
    res, steps, backend, barrier = _run(True, 25, tmp_path=tmp_path)
    assert steps == list(range(25)) and backend.blocked == list(range(25))
    # rendezvous after iterations 1 and 10 (:160-165) and once at the end (:217)
    assert barrier.waits_at == [1, 10, 25]
    assert res["iterations"] == 25 and "p50_latency" not in res
    saved = json.load(open(tmp_path / "client_7.json"))
    assert saved["throughput"] == res["throughput"]


def test_request_loop_protocol_inference_and_stop(tmp_path):
    res, steps, backend, barrier = _run(False, 40, rps=2000, tmp_path=tmp_path)
    assert steps == list(range(40)) and barrier.waits_at == [1, 10, 40]
    assert set(res) >= {"p50_latency", "p95_latency", "p99_latency", "throughput"}
    # open loop: request i is due 1/rps after request i-1, so 30 requests after
    # warm-up cannot finish faster than 29 gaps
    assert (40 - 10) / res["throughput"] >= 29 / 2000 * 0.95
    # a stop request ends the loop after the current iteration (:202-204)
    res, steps, backend, barrier = _run(True, 1000, stop_after=13, tmp_path=tmp_path)
    assert len(steps) == 13 and barrier.waits_at == [1, 10, 13]


def test_job_lists_accept_the_references_job_files(reference_root):
    files = [os.path.join(reference_root, "artifact_evaluation", "example", "config.json"),
             os.path.join(reference_root, "benchmarking", "multi_client_example.json")]
    files += sorted(glob.glob(os.path.join(reference_root, "artifact_evaluation", "fig7",
                                           "config_files", "*.json")))
    assert len(files) > 10
    known = {"resnet50", "resnet101", "mobilenet_v2", "bert", "transformer"}
    for path in files:
        with open(path) as f:
            job = json.load(f)
        lists = launch_jobs.job_lists(job)
        n = len(job)
        assert all(len(v) == n for v in lists.values())
        assert set(lists["model_names"]) <= known
        # training clients come with a first-iteration profile and a steady one
        for i, entry in enumerate(job):
            if entry["args"]["train"]:
                assert lists["additional_model_files"][i] is not None
                assert lists["additional_num_kernels"][i] > 0


def test_job_lists_reject_incomplete_entries():
    with pytest.raises(KeyError):
        launch_jobs.job_lists([{"arch": "resnet50", "num_kernels": 1, "num_iters": 1, "args": {}}])


def test_cli_matches_the_reference():
    a = launch_jobs.build_parser().parse_args(
        ["--algo", "reef", "--config_file", "x.json", "--reef_depth", "12",
         "--orion_max_be_duration", "160000", "--orion_start_update", "5",
         "--orion_hp_limit", "30"])
    assert (a.algo, a.config_file, a.reef_depth, a.orion_max_be_duration,
            a.orion_start_update, a.orion_hp_limit) == ("reef", "x.json", 12, 160000, 5, 30)
    d = launch_jobs.build_parser().parse_args(["--algo", "orion", "--config_file", "x"])
    assert (d.reef_depth, d.orion_max_be_duration, d.orion_start_update, d.orion_hp_limit) == (1, 1, 1, 1)


def test_launcher_refuses_to_run_without_the_preloaded_library():
    with pytest.raises(RuntimeError, match="not preloaded"):
        launch_jobs.check_preloaded()


def test_frontend_rejects_mismatched_lists():
    from orion_amd import scheduler_frontend as fe

    class Lib:
        def sched_init(self):
            return 0
    py = fe.PyScheduler(Lib(), 2)
    with pytest.raises(ValueError):
        py.run_scheduler([threading.Barrier(1)], [1], ["a", "b"], ["f", "g"], [None, None],
                         [1, 1], [None, None], [1, 1], True, True, False, False, 1, 1, 1,
                         [False, False])
    with pytest.raises(NotImplementedError):
        py.run_scheduler([threading.Barrier(1)], [1, 2], ["a", "b"], ["f", "g"], [None, None],
                         [1, 1], [None, None], [1, 1], True, False, False, False, 1, 1, 1,
                         [False, False])


def test_repeated_runs_are_pooled_request_by_request():
    """colocate.pooled: percentiles over all runs' requests together (not a mean
    of per-run percentiles), throughput averaged, the runs kept one by one."""
    from orion_amd import colocate
    a = {"throughput": 80.0, "p50_latency": 1.0, "p95_latency": 1.0, "p99_latency": 1.0,
         "latencies_ms": [1.0] * 99 + [50.0]}
    b = {"throughput": 60.0, "p50_latency": 3.0, "p95_latency": 3.0, "p99_latency": 3.0,
         "latencies_ms": [3.0] * 100}
    res = colocate.pooled([a, b])
    want = np.percentile([1.0] * 99 + [50.0] + [3.0] * 100, [50, 95, 99])
    assert [res["p50_latency"], res["p95_latency"], res["p99_latency"]] == list(want)
    assert res["throughput"] == 70.0 and res["requests"] == 200 and len(res["runs"]) == 2
    # a training client has no latencies: throughput only
    assert colocate.pooled([{"throughput": 30.0}, {"throughput": 34.0}])["throughput"] == 32.0
    # one run without the raw list (an older result file) keeps its own percentiles
    old = {k: v for k, v in a.items() if k != "latencies_ms"}
    assert colocate.pooled([old])["p99_latency"] == 1.0


def test_streams_baseline_runs_the_same_loops_without_a_scheduler(tmp_path, monkeypatch):
    """``--algo streams``: the clients rendezvous with each other after iterations
    1 and 10, the high-priority client's end raises the stop flag, the best-effort
    client stops at its next iteration; result files as under the scheduler."""
    monkeypatch.setenv("ORION_RESULT_DIR", str(tmp_path))
    cc.UNSCHEDULED_STOP.clear()
    steps = {0: 0, 1: 0}

    def loop(batchsize, train, num_iters, rps, uniform, dummy_data, local_rank, barriers,
             client_barrier, tid):
        class NoGpu(cc.Backend):
            def __init__(self):
                pass

            def block(self, it):
                pass

            def stop(self):
                return cc.UNSCHEDULED_STOP.is_set()

        def step(i):
            steps[tid] += 1

        barriers[0].wait()      # every client loop starts with this rendezvous
        return cc.run_client(tid, train, num_iters, [0.0] * num_iters, barriers, step, NoGpu())

    job = [{"arch": "x", "kernel_file": "", "num_kernels": 0, "num_iters": 10_000_000,
            "args": {"batchsize": 1, "rps": 0, "uniform": False, "dummy_data": True,
                     "train": True}},
           {"arch": "x", "kernel_file": "", "num_kernels": 0, "num_iters": 60,
            "args": {"batchsize": 1, "rps": 0, "uniform": False, "dummy_data": True,
                     "train": False}}]
    args = launch_jobs.build_parser().parse_args(["--algo", "streams", "--config_file", "x"])
    res = launch_jobs.launch_jobs(job, args, function_dict={"x": loop})
    cc.UNSCHEDULED_STOP.clear()
    assert res[1]["iterations"] == 60 and steps[1] == 60
    assert 10 <= res[0]["iterations"] < 10_000_000
    assert json.load(open(tmp_path / "client_1.json"))["iterations"] == 60
    assert "p99_latency" in res[1] and "throughput" in res[0]


def test_deterministic_solvers_are_a_property_of_the_whole_job():
    """``deterministic`` switches the convolution solvers of the process: a job
    whose model clients disagree on it would run every client on kernels its
    profile was not captured with (a different kernel count ends the job), so
    the launcher refuses it; clients without a model do not take part."""
    from orion_amd import launch_jobs as lj

    def entry(arch, det=None, train=False):
        args = {"batchsize": 4, "rps": 0, "uniform": False, "dummy_data": True, "train": train}
        if det is not None:
            args["deterministic"] = det
        return {"arch": arch, "kernel_file": "", "num_kernels": 0, "num_iters": 1, "args": args}

    lj.job_lists([entry("resnet50", True, True), entry("resnet50", True)])
    lj.job_lists([entry("bert", None, True), entry("mobilenet_v2", False)])
    lj.job_lists([entry("triad_f32", None, True), entry("resnet50", True)])
    with pytest.raises(ValueError, match="for all model clients of a job or for none"):
        lj.job_lists([entry("resnet50", None, True), entry("resnet50", True)])
    from orion_amd.profiling.capture_profile import profile_name
    assert profile_name(entry("resnet50", True)) != profile_name(entry("resnet50", False))


def test_queueing_ahead_is_refused_for_framework_trainers(monkeypatch):
    """ORION_BE_RUN_AHEAD=1 is supported for the kernel-pair clients; with a
    framework model as a best-effort client it has faulted the GPU, so the
    launcher refuses the job before anything reaches the device."""
    from orion_amd import launch_jobs as lj

    def entry(arch, train):
        return {"arch": arch, "kernel_file": "", "num_kernels": 0, "num_iters": 1,
                "args": {"batchsize": 4, "rps": 0, "uniform": False, "dummy_data": True,
                         "train": train}}

    trainer_pair = [entry("resnet50", True), entry("resnet50", False)]
    kernel_pair = [entry("triad_f32", True), entry("gemm_bf16", False)]
    monkeypatch.setenv("ORION_BE_RUN_AHEAD", "0")
    lj.job_lists(trainer_pair)
    monkeypatch.setenv("ORION_BE_RUN_AHEAD", "1")
    lj.job_lists(kernel_pair)
    lj.job_lists([entry("triad_f32", True), entry("resnet50", False)])   # the model is the HP client
    lj.job_lists([entry("resnet50", False)])                              # a client alone
    with pytest.raises(RuntimeError, match="gemm_bf16, triad_f32"):
        lj.job_lists(trainer_pair)
    # no environment variable opens the door again
    monkeypatch.setenv("ORION_BE_RUN_AHEAD_UNSAFE", "1")
    with pytest.raises(RuntimeError, match="gemm_bf16, triad_f32"):
        lj.job_lists(trainer_pair)


def test_the_experiment_alternates_plain_isolated_and_colocated_runs(tmp_path, monkeypatch):
    """colocate.experiment with plain_streams_too: every repeat runs the
    high-priority client on a plain stream as it is, on a plain stream with the
    thread-local cure, alone through the library, and co-located -- in that
    order, so that the four are compared inside one alternation."""
    from orion_amd import colocate
    calls = []

    def fake_run_job(job, algo, workdir, max_be_duration, env=None, **kw):
        calls.append((os.path.basename(workdir), algo, len(job), dict(env or {})))
        out = []
        for k, entry in enumerate(job):
            res = {"throughput": 10.0 + k}
            if not entry["args"]["train"]:
                lat = [1.0 + 0.01 * len(calls)] * 20
                res.update({"p50_latency": lat[0], "p95_latency": lat[0], "p99_latency": lat[0],
                            "latencies_ms": lat})
            out.append(res)
        return out

    monkeypatch.setattr(colocate, "run_job", fake_run_job)
    job = [{"arch": "x", "kernel_file": "be.csv", "num_kernels": 3, "num_iters": 100,
            "args": {"train": True}},
           {"arch": "x", "kernel_file": "hp.csv", "num_kernels": 5, "num_iters": 30,
            "args": {"train": False}}]
    res = colocate.experiment(job, workdir=str(tmp_path), repeats=2, plain_streams_too=True,
                              env={"ORION_RECORD_DIR": str(tmp_path / "rec")})
    names = [c[0] for c in calls]
    assert names == ["iso_be0",
                     "plain_hp_0", "plain_fresh_hp_0", "iso_hp_0", "colocated_0",
                     "plain_hp_1", "plain_fresh_hp_1", "iso_hp_1", "colocated_1"]
    by_name = {c[0]: c for c in calls}
    assert by_name["plain_hp_0"][1] == "streams" and by_name["plain_hp_0"][3] == {}
    assert by_name["plain_fresh_hp_1"][1] == "streams"
    assert by_name["plain_fresh_hp_1"][3] == {"ORION_PLAIN_TLS_REFRESH": "1"}
    assert by_name["iso_hp_0"][1] == "orion" and by_name["colocated_0"][2] == 2
    # only the last co-located run keeps the recorded logs
    assert "ORION_RECORD_DIR" not in by_name["colocated_0"][3]
    assert by_name["colocated_1"][3]["ORION_RECORD_DIR"] == str(tmp_path / "rec")
    for key in ("hp_plain_isolated", "hp_plain_tls_fresh_isolated", "hp_isolated", "hp_colocated"):
        assert res[key]["requests"] == 40, key
    assert res["hp_p99_ratio"] == pytest.approx(
        res["hp_colocated"]["p99_latency"] / res["hp_isolated"]["p99_latency"])
    assert res["be_retained"] == [1.0]
