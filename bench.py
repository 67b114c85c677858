#!/usr/bin/env python3
"""Headline benchmark: the co-location metric of the job description on one
MI355X, with the hand-written kernels' roofline and CPU baselines beside it.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one BLOCK of high-priority requests through the whole hot path
(interception -> queue -> policy -> dispatch): 100 requests, or more when K is
small, so that every leg of the headline measures at least 1000 requests
whatever K is (a p99 over fewer is not a p99).  K blocks are measured with the
high-priority client alone and K blocks co-located, in --repeats alternating
runs (fresh process each, same seeded Poisson arrivals), and the percentiles are
taken over all requests of each kind.  Every run starts with the client
protocol's own 10 untimed warm-up requests (fixed by the protocol; W does not
change it).  W is the number of untimed launches before the triad timings; the
GEMM always gets 100, which is what the power-limited package needs to settle.
Prints ONE JSON line.

Work done, in order (child processes first, so that this process has not touched
the GPU when it starts them); legs after the headline are skipped, and said to
be, when the time budget (--time-budget) would not hold them:
  1. profile both clients alone under the interception layer (gfx950 profiles);
  2. best-effort client alone; then, alternating --repeats times: the
     high-priority client alone on a plain stream with the interception library
     not preloaded (once as PyTorch runs it, once with its thread-local accesses
     kept on the dynamic loader's fast path as the library keeps a scheduled
     client's: the like-for-like baseline), alone behind the interception layer
     and the scheduler, and co-located;
  3. replay the recorded observation log through the CPU oracle and the native
     policy core: decision sequences must be identical;
  4. the same pair on plain streams with no scheduler and no interception
     (`no_scheduler_baseline`: what the scheduler is for);
  5. short legs of the other two job configurations (MobileNetV2 beside
     BERT-base training; BERT-large beside three trainers), the kernel pair
     through the scheduler, and three variants of the headline pair (the client
     replaying a HIP graph; the throttle option T1; T1 with a 400 us budget);
  6. kernel pair in this process: GEMM and triad alone and side by side per
     CU-mask size, timed with HIP events on the streams they run on;
  7. CPU baselines on this host's cores: the same requests on the PyTorch CPU
     path, host triad and host fp32 GEMM.
"""

import argparse
import copy
import json
import os
import sys
import tempfile
import threading
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# Bytes past the L2s per launch: constants taken from the committed rocprofv3
# FETCH_SIZE / WRITE_SIZE runs of the same kernels and shapes, not measured by
# this program (a counter run needs the profiler around the process).
TRAFFIC_SOURCE = ("profiles/bench_kernels_gemm8192_triad1GiB_counters.txt (rocprofv3 --pmc "
                  "FETCH_SIZE and WRITE_SIZE runs of this kernel and shape, scaled by a copy "
                  "kernel of known size; a constant in bench.py, not re-measured by this run)")
GEMM_TRAFFIC_BYTES = int((786877.9 * 2.0 + 131106.5 * 1.0) * 1024)
TRIAD_TRAFFIC_BYTES = int((1048588.2 * 2.0 + 1048576.1 * 1.0) * 1024)

METRIC = "HP p99 latency vs isolated + BE iters/sec retained, co-located on 1 MI355X"
WORKLOAD = ("HP: ResNet-50 inference, batch 4, bf16, Poisson arrivals at 80 req/s, inputs "
            "4x3x224x224 N(0,1); BE: ResNet-50 training, batch 32, SGD momentum 0.9, "
            "synthetic images N(0,1), labels uniform over 1000 classes, random-init weights")

REQUESTS_PER_STEP = 100      # one step = one block of high-priority requests
MIN_REQUESTS = 1020          # per leg of the headline, whatever --steps says


def _entry(arch, model_name, batch, rps, train, iters, dtype, **more):
    args = {"batchsize": batch, "rps": rps, "uniform": False, "dummy_data": True,
            "train": train, "dtype": dtype}
    if model_name:
        args["model_name"] = model_name
    args.update(more)
    return {"arch": arch, "kernel_file": "", "num_kernels": 0, "num_iters": iters, "args": args}


BE_RESNET50 = _entry("resnet50", "resnet50", 32, 0, True, 1_000_000, "fp32", momentum=0.9)
BE_MOBILENET = _entry("mobilenet_v2", "mobilenet_v2", 64, 0, True, 1_000_000, "fp32", momentum=0.9)
BE_BERT_BASE = _entry("bert", None, 8, 0, True, 1_000_000, "fp32")


def c3_job(hp_iters, hip_graph=False):
    """configs[2]: the headline pair."""
    hp = _entry("resnet50", "resnet50", 4, 80, False, hp_iters, "bf16")
    if hip_graph:
        hp["args"]["hip_graph"] = True
    return [copy.deepcopy(BE_RESNET50), hp]


def c4_job(hp_iters):
    """configs[3]: MobileNetV2 inference at Poisson 100 req/s beside BERT-base training."""
    return [copy.deepcopy(BE_BERT_BASE),
            _entry("mobilenet_v2", "mobilenet_v2", 4, 100, False, hp_iters, "bf16")]


def c5_job(hp_iters):
    """configs[4]: BERT-large inference, closed loop, beside three trainers."""
    return [copy.deepcopy(BE_RESNET50), copy.deepcopy(BE_MOBILENET), copy.deepcopy(BE_BERT_BASE),
            _entry("bert", None, 8, 0, False, hp_iters, "bf16")]


class Progress:
    """A line on stderr whenever a leg starts and every 30 s while it runs: the
    JSON line on stdout comes only at the very end, and a run that says nothing
    for minutes is indistinguishable from a hung one."""

    def __init__(self):
        self.start = time.time()
        self.leg = "starting"
        threading.Thread(target=self._beat, daemon=True).start()

    def note(self, leg):
        self.leg = leg
        print(f"[bench {time.time() - self.start:5.0f} s] {leg}", file=sys.stderr, flush=True)

    def _beat(self):
        while True:
            time.sleep(30)
            print(f"[bench {time.time() - self.start:5.0f} s] ... {self.leg}", file=sys.stderr,
                  flush=True)


class Legs:
    """Shared state of the co-location legs: one profile directory (a client that
    appears in several jobs is profiled once) and one cache of best-effort
    clients' isolated rates."""

    def __init__(self, workdir, masks, deadline, progress=None):
        self.progress = progress
        self.workdir = workdir
        self.masks = masks
        self.deadline = deadline
        self.profiles = os.path.join(workdir, "profiles")
        self.be_isolated = {}

    def time_left(self):
        return self.deadline - time.time()

    def run(self, name, job, budget_ns, repeats=1, algo="orion", extra_env=None,
            use_rocprof=False, record=False, plain_streams_too=False):
        from orion_amd import colocate
        from orion_amd.profiling import capture_profile
        if self.progress:
            self.progress.note(f"{name}: {len(job)} client(s), algo {algo}, {repeats} repeat(s)")
        wd = os.path.join(self.workdir, name)
        os.makedirs(wd, exist_ok=True)
        env = dict(extra_env or {})
        if algo != "streams":
            cfg = os.path.join(wd, "job.json")
            with open(cfg, "w") as f:
                json.dump(job, f)
            job = capture_profile.fill_job(cfg, self.profiles, os.path.join(wd, "job_filled.json"),
                                           quiet=True, use_rocprof=use_rocprof, reuse=True)
            if self.masks:
                env["ORION_BE_CU_MASKS"] = self.masks
            if record:
                env["ORION_RECORD_DIR"] = os.path.join(wd, "colocated")
                os.makedirs(env["ORION_RECORD_DIR"], exist_ok=True)
        # a best-effort client's isolated rate is measured once per (client, mode)
        known = []
        for be in job[:-1]:
            known.append(self.be_isolated.get((capture_profile.profile_name(be), algo,
                                               tuple(sorted(env.items())))))
        res = colocate.experiment(job, algo, budget_ns, wd, env=env, repeats=repeats,
                                  be_isolated_known=known, plain_streams_too=plain_streams_too)
        for be, iso in zip(job[:-1], res["be_isolated"]):
            self.be_isolated[(capture_profile.profile_name(be), algo,
                              tuple(sorted(env.items())))] = iso
        res["num_kernels"] = {"hp": job[-1].get("num_kernels"),
                              "be": [b.get("additional_num_kernels", b.get("num_kernels"))
                                     for b in job[:-1]]}
        return res


def hp_summary(co):
    keys = ("p50", "p95", "p99")
    out = {"isolated_ms": {k: co["hp_isolated"][f"{k}_latency"] for k in keys},
           "colocated_ms": {k: co["hp_colocated"][f"{k}_latency"] for k in keys},
           "p50_ratio": co["hp_p50_ratio"], "p99_ratio": co["hp_p99_ratio"],
           "requests_per_s": co["hp_colocated"]["throughput"],
           "requests": {"isolated": co["hp_isolated"].get("requests"),
                        "colocated": co["hp_colocated"].get("requests")}}
    if co["hp_isolated"].get("runs"):
        # the alternating runs one by one (percentiles above: all requests)
        out["isolated_runs_p99_ms"] = [r["p99_latency"] for r in co["hp_isolated"]["runs"]]
        out["colocated_runs_p99_ms"] = [r["p99_latency"] for r in co["hp_colocated"]["runs"]]
    return out


def be_summary(co):
    return [{"isolated_iters_per_s": i["throughput"], "colocated_iters_per_s": c["throughput"],
             "retained": r}
            for i, c, r in zip(co["be_isolated"], co["be_colocated"], co["be_retained"])]


def policy_replay(record_dir):
    """Bit-exact check and replay rate over the co-located run's own log."""
    from oracle import obslog          # the checker (CPU baseline of the policy)
    from orion_amd import replay
    obs = open(os.path.join(record_dir, "observations.log")).read()
    dec = open(os.path.join(record_dir, "decisions.log")).read()
    n_dec = dec.count("\nD ") + dec.startswith("D ")
    t0 = time.perf_counter()
    native = replay.native_replay(obs)
    t_native = time.perf_counter() - t0
    # the oracle is pure Python: replay a bounded prefix (whole segments)
    lines = obs.splitlines(keepends=True)
    cut, polls = len(lines), 0
    for i, l in enumerate(lines):
        polls += l.startswith("P ")
        if l.startswith("E") and polls > 60_000:
            cut = i + 1
            break
    t0 = time.perf_counter()
    oracle_dec = obslog.replay("".join(lines[:cut]))
    t_oracle = time.perf_counter() - t0
    return {
        "decisions": n_dec,
        "native_equals_recorded": native == dec,
        "oracle_equals_recorded_prefix": dec.startswith(oracle_dec),
        "oracle_prefix_decisions": oracle_dec.count("\nD "),
        "native_decisions_per_s": n_dec / t_native if t_native > 0 else None,
        "oracle_decisions_per_s": oracle_dec.count("\nD ") / t_oracle if t_oracle > 0 else None,
    }


def own_children():
    """Process ids whose parent is this process (threads are not processes)."""
    me, found = os.getpid(), []
    for name in os.listdir("/proc"):
        if not name.isdigit():
            continue
        try:
            with open(f"/proc/{name}/stat") as f:
                stat = f.read()
            # pid (comm) state ppid ...: comm may hold spaces and parentheses
            ppid = int(stat[stat.rindex(")") + 2:].split()[1])
        except (OSError, ValueError, IndexError):
            continue
        if ppid == me:
            found.append(int(name))
    return found


def end_own_children(grace_s=2.0):
    """Ends child processes that are still alive, each by its own process id:
    first asked to terminate, then killed.  Returns how many there were."""
    import signal
    children = own_children()
    found = len(children)
    for pid in children:
        try:
            os.kill(pid, signal.SIGTERM)
        except OSError:
            pass
    deadline = time.time() + grace_s
    while children and time.time() < deadline:
        for pid in list(children):
            try:
                done, _ = os.waitpid(pid, os.WNOHANG)
            except ChildProcessError:
                done = pid
            if done:
                children.remove(pid)
        time.sleep(0.05)
    for pid in children:
        try:
            os.kill(pid, signal.SIGKILL)
            os.waitpid(pid, 0)
        except OSError:
            pass
    return found


def host_cores():
    """Threads the CPU baselines use: the CPUs this process may run on, capped by
    OMP_NUM_THREADS when the environment sets one (a shared host hands out a
    share of its cores that way)."""
    n = len(os.sched_getaffinity(0))
    try:
        n = min(n, int(os.environ.get("OMP_NUM_THREADS", n)))
    except ValueError:
        pass
    return max(1, n)


def _time_requests(fn, budget_s, max_n=500, warm=2):
    import numpy as np
    for _ in range(warm):
        fn()
    times = []
    t_end = time.perf_counter() + budget_s
    while (time.perf_counter() < t_end or len(times) < 3) and len(times) < max_n:
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return {"p50_ms": float(np.percentile(times, 50) * 1000),
            "p99_ms": float(np.percentile(times, 99) * 1000),
            "requests": len(times), "cpu_seconds": float(sum(times))}


def cpu_baseline(budget_s=10.0, others_budget_s=4.0, with_others=True):
    """The reference's clients on the PyTorch CPU path, on this host's cores:
    the headline request (ResNet-50, batch 4, fp32, N(0,1) input from a seed) as
    `value`; beside it the high-priority requests of the other job
    configurations and the host versions of the kernel pair."""
    import torch
    from orion_amd.benchmark_suite.vision_models import mobilenet_v2, resnet50
    cores = host_cores()
    torch.set_num_threads(cores)
    torch.manual_seed(42)
    x = torch.randn(4, 3, 224, 224, generator=torch.Generator().manual_seed(42))
    model = resnet50().eval()
    with torch.no_grad():
        r50 = _time_requests(lambda: model(x), budget_s)
    out = {"value": r50["p50_ms"], "unit": "ms per request (p50)", "p99_ms": r50["p99_ms"],
           "cores": cores, "kind": "port",
           "sample": f"{r50['requests']} ResNet-50 batch-4 fp32 requests on the PyTorch CPU "
                     f"path ({r50['cpu_seconds']:.1f} s of CPU work)"}
    if not with_others:
        return out
    others = {}
    with torch.no_grad():
        model = mobilenet_v2().eval()
        others["mobilenet_v2_bs4_fp32_request"] = _time_requests(lambda: model(x), others_budget_s)
        from transformers import BertForQuestionAnswering
        from orion_amd.benchmark_suite.bert_trainer import SEQ_LEN, VOCAB, bert_config
        ids = torch.randint(0, VOCAB, (8, SEQ_LEN), generator=torch.Generator().manual_seed(42))
        for name, train in (("bert_base_seq384_bs8_fp32_forward", True),
                            ("bert_large_seq384_bs8_fp32_request", False)):
            torch.manual_seed(42)
            model = BertForQuestionAnswering(bert_config(train)).eval()
            others[name] = _time_requests(lambda: model(input_ids=ids), others_budget_s, warm=1)
        del model
        # host versions of the kernel pair: a = b + s*c over 3 x 1 GiB of fp32,
        # and an fp32 GEMM of the GPU kernel's shape
        n = 1 << 28
        b = torch.rand(n) * 2 - 1
        c = torch.rand(n) * 2 - 1
        a = torch.empty(n)
        t = _time_requests(lambda: torch.add(b, c, alpha=1.7, out=a), 2.0, warm=1)
        others["host_triad_f32_3x1GiB"] = {"gb_per_s": 12 * n / (t["p50_ms"] * 1e6), **t}
        del a, b, c
        m = 8192
        p = torch.rand(m, m) * 2 - 1
        q = torch.rand(m, m) * 2 - 1
        t = _time_requests(lambda: torch.matmul(p, q.t()), 3.0, max_n=5, warm=1)
        others["host_gemm_f32_8192"] = {"gflop_per_s": 2 * m ** 3 / (t["p50_ms"] * 1e6), **t}
    out["others"] = others
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20,
                    help="blocks of high-priority requests per leg (100 requests a block; "
                         f"more when that would give fewer than {MIN_REQUESTS} per leg)")
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--max-be-duration", type=int, default=160_000,
                    help="budget (ns) of outstanding best-effort work; the default is the "
                         "value the reference uses for this pair "
                         "(artifact_evaluation/fig7/run_orion.py:6-15)")
    ap.add_argument("--be-cu-masks", default="",
                    help="override ORION_BE_CU_MASKS for the co-located run")
    ap.add_argument("--rocprof-profiles", action="store_true",
                    help="take the profiles' class, duration and register columns from "
                         "rocprofv3 runs (adds about two minutes)")
    ap.add_argument("--kernels-only", action="store_true",
                    help="only the in-process kernel measurements (for profiler runs: "
                         "starts no child process)")
    ap.add_argument("--headline-only", action="store_true",
                    help="skip every leg after the headline, its replay, the kernels and "
                         "the headline's CPU baseline")
    ap.add_argument("--short-requests", type=int, default=400,
                    help="measured high-priority requests of the short legs (HIP-graph and "
                         "throttle variants; MobileNetV2 beside BERT training runs twice, "
                         "BERT-large beside three trainers five times as many)")
    ap.add_argument("--pair-requests", type=int, default=300,
                    help="measured GEMM requests of the scheduled kernel pair")
    ap.add_argument("--repeats", type=int, default=4,
                    help="the isolated and the co-located run of the high-priority client "
                         "alternate this many times and the percentiles are taken over "
                         "all of them")
    ap.add_argument("--time-budget", type=float, default=520.0,
                    help="seconds this run may take; optional legs that would not fit "
                         "are skipped and listed in `skipped`")
    ap.add_argument("--workdir", default="")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the scheduler shares a single device and "
              "nothing in this build uses a second one (run with --gpus 1)", file=sys.stderr)
        return 2
    t_start = time.time()
    workdir = args.workdir or tempfile.mkdtemp(prefix="orion_bench_")
    os.makedirs(workdir, exist_ok=True)
    steps = max(1, args.steps)
    per_step = max(REQUESTS_PER_STEP, -(-MIN_REQUESTS // steps))
    repeats = max(1, args.repeats)
    per_run = -(-steps * per_step // repeats)

    out = {"metric": METRIC, "unit": "x isolated p99 (high-priority, co-located / isolated)",
           "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
           "dtype": "bf16", "data": "synthetic",
           "config": {"workload": WORKLOAD, "baseline_config": "configs[2]",
                      "algo": "orion", "max_be_duration_ns": args.max_be_duration,
                      "requests_per_step": per_step, "repeats": repeats,
                      "requests_per_run": per_run}}
    skipped = []
    progress = Progress()
    legs = Legs(workdir, args.be_cu_masks, t_start + args.time_budget, progress)

    # what the legs that always run, after the child processes, need: the kernels
    # in this process and the CPU baselines
    reserve = 75.0

    def fits(name, seconds):
        left = legs.time_left() - reserve
        if args.headline_only or left < seconds:
            skipped.append(name if args.headline_only else
                           f"{name} (needs ~{seconds:.0f} s, {left:.0f} s left)")
            return False
        return True

    if not args.kernels_only:
        t0 = time.time()
        # every repeat: the client alone on a plain stream (the library not
        # preloaded; as it is and with the thread-local cure), alone behind the
        # interception layer and the scheduler, and co-located -- so that what the
        # path costs and what co-location costs are differences inside one
        # alternation, not between boxes or minutes
        co = legs.run("c3", c3_job(per_run + 10), args.max_be_duration, repeats=repeats,
                      use_rocprof=args.rocprof_profiles, record=True, plain_streams_too=True)
        out["value"] = co["hp_p99_ratio"]
        # one step = `per_step` requests of the co-located run
        out["ms_per_step"] = 1000.0 * per_step / co["hp_colocated"]["throughput"]
        out["hp"] = hp_summary(co)
        out["be"] = be_summary(co)[0]
        out["config"]["records_per_iteration"] = co["num_kernels"]
        plain = co["hp_plain_isolated"]
        out["hp"]["plain_streams_isolated_ms"] = {
            k: plain[f"{k}_latency"] for k in ("p50", "p95", "p99")}
        out["hp"]["requests"]["plain_streams_isolated"] = plain.get("requests")
        out["hp"]["plain_streams_isolated_runs_p50_ms"] = [r["p50_latency"] for r in plain["runs"]] \
            if plain.get("runs") else [plain["p50_latency"]]
        out["hp"]["isolated_runs_p50_ms"] = [r["p50_latency"] for r in co["hp_isolated"]["runs"]] \
            if co["hp_isolated"].get("runs") else [co["hp_isolated"]["p50_latency"]]
        # the plain-stream client again, its thread-local accesses kept off the
        # dynamic loader's slow path the way the library keeps a scheduled
        # client's (ORION_PLAIN_TLS_REFRESH=1): the like-for-like baseline
        fresh = co["hp_plain_tls_fresh_isolated"]
        out["hp"]["plain_streams_tls_fresh_isolated_ms"] = {
            k: fresh[f"{k}_latency"] for k in ("p50", "p95", "p99")}
        out["hp"]["requests"]["plain_streams_tls_fresh_isolated"] = fresh.get("requests")
        out["hp"]["plain_streams_tls_fresh_isolated_runs_p50_ms"] = \
            [r["p50_latency"] for r in fresh["runs"]] if fresh.get("runs") else [fresh["p50_latency"]]
        # what the path costs the client when there is nothing to schedule:
        # against the like-for-like plain client, and against the plain client as
        # PyTorch runs it
        out["hp"]["path_cost_p50_ms"] = co["hp_isolated"]["p50_latency"] - fresh["p50_latency"]
        out["hp"]["path_cost_vs_plain_as_is_p50_ms"] = \
            co["hp_isolated"]["p50_latency"] - plain["p50_latency"]
        for p in ("p50", "p99"):
            out["hp"][f"{p}_ratio_vs_plain_streams_isolated"] = (
                co["hp_colocated"][f"{p}_latency"] / plain[f"{p}_latency"])
            out["hp"][f"{p}_ratio_vs_plain_streams_tls_fresh_isolated"] = (
                co["hp_colocated"][f"{p}_latency"] / fresh[f"{p}_latency"])
        out["colocation_wall_s"] = time.time() - t0
        progress.note("replaying the recorded decisions")
        out["policy_replay"] = policy_replay(os.path.join(workdir, "c3", "colocated"))
        # The same pair with no scheduler and no interception (--algo streams):
        # what the scheduler is for
        if fits("no_scheduler_baseline", 60):
            sres = legs.run("streams", c3_job(MIN_REQUESTS + 10), args.max_be_duration,
                            algo="streams")
            out["no_scheduler_baseline"] = {**hp_summary(sres), "be": be_summary(sres)[0]}

        short = args.short_requests
        # configs[3] and configs[4], short: a p99 over `short` requests is a few
        # samples deep; the parity tests of these configurations are in tests/
        # (twice and five times `short`: their request rates are higher, so the
        # legs stay a few seconds long while the p99 gets 8 and 20 samples deep)
        if fits("c4_mobilenet_beside_bert_base_training", 100):
            c4 = legs.run("c4", c4_job(2 * short + 10), 100_000)
            out["c4_mobilenet_beside_bert_base_training"] = {
                "workload": "configs[3], budget 100 us", "hp": hp_summary(c4), "be": be_summary(c4),
                "records_per_iteration": c4["num_kernels"]}
        if fits("c5_bert_large_beside_three_trainers", 170):
            c5 = legs.run("c5", c5_job(5 * short + 50), 100_000)
            out["c5_bert_large_beside_three_trainers"] = {
                "workload": "configs[4], budget 100 us, closed loop", "hp": hp_summary(c5),
                "be": be_summary(c5), "records_per_iteration": c5["num_kernels"]}
        # configs[1] through the same hot path: GEMM requests (high priority)
        # beside the triad loop (best effort), default CU masks; back-to-back
        # requests (the high-priority client never idle) and Poisson arrivals
        from orion_amd import kernel_pair as kp_child
        out["kernel_pair_scheduled"] = {}
        # (the third leg keeps best-effort kernels that alone outlast the budget
        # off the whole-GPU stream: ORION_CONFINE_LONG_BE=1)
        # (the fourth lets the triad client queue its launches ahead of their
        # dispatch, ORION_BE_RUN_AHEAD=1: the configuration that option is
        # verified with on the GPU)
        for label, rps, confine, ahead in (
                ("closed_loop", 0, False, False), ("poisson_400rps", 400, False, False),
                ("poisson_400rps_long_be_confined", 400, True, False),
                ("closed_loop_be_run_ahead", 0, False, True)):
            if not fits("kernel_pair_scheduled." + label, 30):
                continue
            progress.note("kernel pair through the scheduler: " + label)
            pair = kp_child.run_child(small=False, check=True, rps=rps, confine_long=confine,
                                      run_ahead=ahead,
                                      hp_iters=args.pair_requests + 10,
                                      max_be_duration=args.max_be_duration,
                                      workdir=os.path.join(workdir, "pair_" + label))
            out["kernel_pair_scheduled"][label] = {
                "hp_gemm_ms": {"isolated_p50": pair["hp_isolated"]["p50_latency"],
                               "isolated_p99": pair["hp_isolated"]["p99_latency"],
                               "colocated_p50": pair["hp_colocated"]["p50_latency"],
                               "colocated_p99": pair["hp_colocated"]["p99_latency"]},
                "hp_p99_ratio": (pair["hp_colocated"]["p99_latency"]
                                 / pair["hp_isolated"]["p99_latency"]),
                "be_triad_iters_per_s": {"isolated": pair["be_isolated"]["throughput"],
                                         "colocated": pair["be_colocated"]["throughput"]},
                "be_retained": pair["be_retained"],
                "outputs_match_isolated": pair["outputs_match"]}
        # The headline pair with the high-priority client replaying a captured HIP
        # graph: one copy record and one hipGraphLaunch record per request instead
        # of 371 kernel records.  (Not the headline: the reference schedules the
        # request kernel by kernel.)
        if fits("hp_hip_graph_variant", 60):
            cg = legs.run("hip_graph", c3_job(short + 10, hip_graph=True), args.max_be_duration,
                          extra_env={"ORION_RESERVE_HP_CUS": "1"})
            out["hp_hip_graph_variant"] = {
                # the graph record needs every CU by profile; with this option the
                # policy leaves best-effort kernels no room beside it
                "options": {"ORION_RESERVE_HP_CUS": 1}, "hp": hp_summary(cg),
                "be": be_summary(cg)[0], "records_per_iteration": cg["num_kernels"]}
        # The headline pair with the duration throttle letting go at its half-way
        # mark (ORION_SLIDING_THROTTLE=1, recorded as T1): not the headline, whose
        # decisions follow the reference's rule
        if fits("sliding_throttle_variant", 60):
            ct = legs.run("sliding_throttle", c3_job(short + 10), args.max_be_duration,
                          extra_env={"ORION_SLIDING_THROTTLE": "1"})
            out["sliding_throttle_variant"] = {
                "options": {"ORION_SLIDING_THROTTLE": 1}, "hp": hp_summary(ct),
                "be": be_summary(ct)[0]}
        # The same with a duration budget of 400 us instead of the reference's own
        # 160 us for this pair: the request is bound by its submission on the host
        # and leaves the GPU slack, so on this GPU the larger budget costs the
        # high-priority client next to nothing and the trainer gains
        if fits("tuned_budget_variant", 60):
            cb = legs.run("tuned_budget", c3_job(short + 10), 400_000,
                          extra_env={"ORION_SLIDING_THROTTLE": "1"})
            out["tuned_budget_variant"] = {
                "options": {"ORION_SLIDING_THROTTLE": 1, "orion_max_be_duration_ns": 400_000},
                "hp": hp_summary(cb), "be": be_summary(cb)[0]}
    progress.note("kernels in this process: GEMM and triad alone and side by side")
    import torch
    from orion_amd import kernel_pair as kp
    reps = max(20, min(200, steps * 10))
    alone = kp.measure_alone(reps=reps, warmup=max(1, args.warmup))
    pairs = [kp.measure_pair(m, reps=reps) for m in (32, 64, 128, 0)]
    torch.cuda.synchronize()
    gemm = alone["gemm"]
    flops = 2 * kp.GEMM_N ** 3
    out["roofline"] = {"kernel": "gemm_bf16_nt_kernel<bf16 out> 8192x8192x8192", "bound": "mfma",
                       "achieved": gemm["tflops"], "peak": kp.MFMA_BF16_PEAK_TFLOPS,
                       "unit": "TFLOP/s", "frac": gemm["tflops"] / kp.MFMA_BF16_PEAK_TFLOPS,
                       "flops_per_launch": flops, "ms_per_launch": gemm["ms"],
                       # settled rate (100 untimed launches first); the first 20
                       # launches after an idle period, while the clocks of the
                       # power-limited package still settle, are slower
                       "burst_achieved": gemm["burst_tflops"],
                       # bytes past the L2s per launch, from the committed rocprofv3
                       # FETCH_SIZE / WRITE_SIZE runs (scaled by a copy kernel)
                       "traffic": GEMM_TRAFFIC_BYTES, "traffic_source": TRAFFIC_SOURCE}
    tri = alone["triad"]["256"]
    out["roofline_triad"] = {"kernel": "triad_f32_kernel 3 x 1 GiB", "bound": "hbm",
                             "achieved": tri["gbs"], "peak": kp.HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": tri["gbs"] / kp.HBM_PEAK_GBS,
                             "bytes_per_launch": 12 * kp.TRIAD_ELEMS,
                             "ms_per_launch": tri["ms"], "traffic": TRIAD_TRAFFIC_BYTES,
                             "traffic_source": TRAFFIC_SOURCE}
    out["kernel_pair"] = {
        "workload": "configs[1]: HP bf16 GEMM 8192^3 beside BE fp32 triad over 1 GiB arrays",
        "triad_alone_gbs_by_cu_mask": {k: v["gbs"] for k, v in alone["triad"].items()},
        "colocated_by_be_cu_mask": [
            {"be_cus": p["mask"], "gemm_tflops": p["gemm_tflops"],
             "gemm_slowdown": p["gemm_ms"] / gemm["ms"],
             "mfma_frac_of_peak": p["gemm_tflops"] / kp.MFMA_BF16_PEAK_TFLOPS,
             "triad_gbs": p["triad_gbs"],
             "triad_slowdown": p["triad_ms"] / alone["triad"][str(p["mask"])]["ms"],
             "hbm_frac_of_peak": p["triad_gbs"] / kp.HBM_PEAK_GBS} for p in pairs]}
    if out.get("kernel_pair_scheduled"):
        # What bounds the scheduled pair whatever the policy does: the GEMM holds
        # the package at its power limit, so a triad confined to the smallest mask
        # (32 of 256 CUs) already costs it this much, measured directly on two
        # streams in this process -- beside the ratios of the scheduled legs above
        by_mask = {str(p["mask"] or 256): p["gemm_ms"] / gemm["ms"] for p in pairs}
        out["kernel_pair_scheduled"]["physical_bound"] = {
            "gemm_slowdown_beside_triad_by_be_cu_mask": by_mask,
            "note": "closed-loop GEMM requests beside the triad cannot do better than the "
                    "32-CU figure: compare it with closed_loop.hp_p99_ratio"}
    if args.kernels_only:
        out["value"] = gemm["tflops"]
        out["metric"] = "kernel pair only (profiler run)"
        out["unit"] = "TFLOP/s"
        out["higher_is_better"] = True
        out["ms_per_step"] = gemm["ms"]
        print(json.dumps(out))
        return 0
    progress.note("CPU baselines")
    others = legs.time_left() > 30 and not args.headline_only
    out["cpu_baseline"] = cpu_baseline(with_others=others)
    if not others:
        skipped.append("cpu_baseline.others")
    out["skipped"] = skipped
    # every leg waits for the children it started; whatever is still there now
    # (there should be nothing) is ended here, by process id, and counted
    out["children_ended_at_exit"] = end_own_children()
    out["wall_s"] = time.time() - t_start
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
