"""Interception + scheduler end to end on a host without a GPU.

A child process loads libinttemp.so and scheduler_eval.so against a recording
stand-in for the HIP runtime (tests/fakehip) and runs the reference's job
protocol: client threads submit copies and order-sensitive kernels, the
scheduler thread runs the three-phase schedule.  Checked here:

* every client's final buffer equals the same kernel sequence run in isolation
  (bit-exact: the kernels are deterministic host functions);
* every launch was issued by the scheduler thread, none by a client thread --
  except that a high-priority inference client, whose records the policy
  dispatches unconditionally, issues its own calls on the one unmasked stream
  the scheduler gave it (ORION_HP_DIRECT=0 switches that off);
* best-effort kernels ran on CU-masked streams, the high-priority client on an
  unmasked one;
* the stop protocol ended the best-effort clients once the high-priority client
  had finished (reference: scheduler_eval.cpp:459-468, intercept_temp.cpp:132-141);
* the decision log the live scheduler recorded is reproduced, byte for byte, by
  the CPU oracle and by the native core replaying the recorded observations.
"""

import json
import os
import subprocess
import sys

import pytest

from oracle import obslog
from tests import jobs

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FAKEHIP = os.path.join(ROOT, "tests", "fakehip", "libfakehip.so")


def run_child(workdir, algo, n_be, hp_iters, direct=True, graph=False, pin=True,
              untyped=False, run_ahead=True, async_exec=False, extra_env=None):
    if not os.path.exists(FAKEHIP):
        pytest.fail("tests/fakehip/libfakehip.so is not built (make -C orion_amd/csrc)")
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "tests", "fake_runner.py"), workdir,
         algo, str(n_be), str(hp_iters)] + (["graph"] if graph else []),
        capture_output=True, text=True, timeout=300,
        env=dict(os.environ, ORION_HP_DIRECT="1" if direct else "0",
                 ORION_PIN_THREADS="1" if pin else "0",
                 FAKE_RUNNER_UNTYPED="1" if untyped else "",
                 ORION_BE_RUN_AHEAD="1" if run_ahead else "0",
                 # the stand-in runtime runs queued work later, stream by stream in
                 # an order of its own choosing, instead of at the call
                 FAKEHIP_ASYNC="1" if async_exec else "0", **(extra_env or {})))
    assert proc.returncode == 0, proc.stdout + proc.stderr
    line = [l for l in proc.stdout.splitlines() if l.startswith("{")][-1]
    return json.loads(line)


@pytest.mark.parametrize("async_exec", [False, True])
@pytest.mark.parametrize("direct", [True, False])
@pytest.mark.parametrize("algo,n_be", [("orion", 0), ("orion", 1), ("orion", 3),
                                       ("reef", 2), ("sequential", 1)])
def test_job_protocol_on_fake_runtime(tmp_path, algo, n_be, direct, async_exec):
    hp_iters = 40
    res = run_child(str(tmp_path), algo, n_be, hp_iters, direct, async_exec=async_exec)
    assert not any(res["alive"])
    assert res["iters_done"][-1] == hp_iters
    assert all(res["outputs_equal"]), res
    sched, hp_tid = res["sched_tid"][0], res["client_tids"][-1]
    if direct and algo != "sequential":
        assert set(res["launch_tids"]) <= {sched, hp_tid}
        # all but the records queued before the scheduler's first call
        assert res["launches_by_tid"][str(hp_tid)] >= (hp_iters - 1) * 5
        hp_streams = res["launch_streams_by_tid"][str(hp_tid)]
        assert len(hp_streams) == 1 and res["launch_stream_masks"][str(hp_streams[0])] == 0
        if n_be:
            assert str(sched) in res["launches_by_tid"]
    else:
        assert res["launch_tids"] == res["sched_tid"]
        assert not set(res["launch_tids"]) & set(res["client_tids"])
    if algo == "orion" and n_be > 0:
        masked = [b for b in res["launch_stream_masks"].values() if b > 0]
        assert masked and all(b in (32, 64, 128) for b in masked)
    # hipMallocAsync / hipFreeAsync of every client: run by the client's own
    # thread, on a stream the scheduler assigned (not the null stream they named)
    assert sorted(t for s, t in res["async_allocs"]) == sorted(res["client_tids"])
    assert sorted(t for s, t in res["async_frees"]) == sorted(res["client_tids"])
    for c in range(n_be):      # stopped early, not run to their 10000 iterations
        assert 0 < res["iters_done"][c] < 10_000
    # hipStreamWriteValue32 / hipLaunchHostFunc of every client named the null
    # stream (id 0); each ran on the calling thread, on the stream the client's
    # work had been moved to
    assert len(res["stream_ops"]) == 2 * sum(res["iters_done"])
    assert all(s != 0 and t in res["client_tids"] for s, t in res["stream_ops"])
    # With ORION_BE_RUN_AHEAD=1 (set by run_child; the library's default is the
    # reference's synchronous hand-off of every record) best-effort clients do
    # not wait for the dispatch of launches that can carry
    # their arguments with them (hipLaunchKernel through a graph kernel node that
    # owns the copy, argument-buffer module launches through a copy in the queue
    # slot); launches with a kernelParams array, copies from host memory and
    # everything the high-priority client submits are handed over synchronously.
    # The runner overwrites its argument objects right after each call, so the
    # outputs above are only right if every queued record owned its arguments.
    assert res["deferred"][-1] == 0
    for c in range(n_be):
        assert 0 < res["deferred"][c] < res["submitted"][c]
    if n_be:
        assert res["holder_sets"] > 0

    obs = open(os.path.join(str(tmp_path), "observations.log")).read()
    dec = open(os.path.join(str(tmp_path), "decisions.log")).read()
    assert dec.count("\nD ") > 100
    assert obslog.replay(obs) == dec            # CPU oracle, bit-exact
    assert jobs.native_replay(obs) == dec       # native core, replayed
    if algo == "orion" and n_be:
        # the scheduler's own account of what became of waiting best-effort
        # records, poll by poll: as many admitted as the log shows dispatched
        adm = json.load(open(os.path.join(str(tmp_path), "admission.json")))
        for c, a in enumerate(adm["polls_with_a_record_waiting"][:n_be]):
            dispatched = sum(1 for l in dec.splitlines() if l.startswith(f"D {c} {c} "))
            assert a["client"] == c and a["admitted"] == dispatched
            assert a["refused_cu_budget"] + a["refused_same_class"] + a["throttled"] > 0


def test_every_record_is_handed_over_synchronously_by_default(tmp_path):
    """Without ORION_BE_RUN_AHEAD=1 no client queues a record it does not wait
    for (reference: intercept_temp.cpp:404-416, every caller spins until its
    record has been taken); same outputs, same replay."""
    res = run_child(str(tmp_path), "orion", 2, 30, run_ahead=False)
    assert not any(res["alive"]) and all(res["outputs_equal"]), res
    assert res["deferred"] == [0, 0, 0] and res["holder_sets"] == 0
    obs = open(os.path.join(str(tmp_path), "observations.log")).read()
    dec = open(os.path.join(str(tmp_path), "decisions.log")).read()
    assert obslog.replay(obs) == dec and jobs.native_replay(obs) == dec


def test_only_clients_of_the_librarys_own_kernels_queue_ahead(tmp_path):
    """ORION_BE_RUN_AHEAD=1 in a GPU process: setup() clears a best-effort client
    for queueing ahead by its model name -- the two hand-written kernel clients
    only.  A framework model keeps the synchronous hand-off whatever the
    environment says (with a trainer queueing ahead a GPU has faulted, cause not
    found), and no variable overrides that.  The stand-in runtime asks to be
    treated like a device here; by itself it clears every client, which is what
    the other host tests rely on."""
    strict = {"ORION_STAND_IN_AS_DEVICE": "1", "ORION_BE_RUN_AHEAD_UNSAFE": "1",
              "FAKE_RUNNER_MODEL_NAMES": "resnet50,triad_f32,gemm_bf16"}
    res = run_child(str(tmp_path), "orion", 2, 30, extra_env=strict)
    assert not any(res["alive"]) and all(res["outputs_equal"]), res
    assert res["deferred"][0] == 0 and res["deferred"][2] == 0
    assert 0 < res["deferred"][1] < res["submitted"][1]
    obs = open(os.path.join(str(tmp_path), "observations.log")).read()
    dec = open(os.path.join(str(tmp_path), "decisions.log")).read()
    assert obslog.replay(obs) == dec and jobs.native_replay(obs) == dec
    # the knob that takes the graph kernel nodes out is for the stand-in only
    strict["ORION_BE_RUN_AHEAD_HOLDERS"] = "0"
    res = run_child(str(tmp_path), "orion", 2, 30, extra_env=strict)
    assert res["holder_sets"] > 0, "ORION_BE_RUN_AHEAD_HOLDERS was honoured in a device process"


@pytest.mark.parametrize("algo,n_be", [("orion", 1), ("orion", 2), ("reef", 1)])
def test_the_reference_calling_convention_without_prototypes(tmp_path, algo, n_be):
    """The reference's front end and client loops call both libraries through
    ``cdll.LoadLibrary`` with no ``argtypes``/``restype`` (scheduler_frontend.py:56
    assigns them to the library object, which has no effect): ``sched_init``'s
    pointer comes back as a C int -- truncated -- and is re-passed as that,
    Python bools travel as ints, ``stop()`` is read as an int.  Same job, same
    three phases with ``setup_change`` between the first two; outputs equal the
    isolated sequence and the recorded log replays bit-exactly."""
    hp_iters = 40
    res = run_child(str(tmp_path), algo, n_be, hp_iters, untyped=True)
    assert not any(res["alive"])
    assert res["iters_done"][-1] == hp_iters and all(res["outputs_equal"]), res
    handle = res["handle"][0]
    assert isinstance(handle, int) and -2 ** 31 <= handle < 2 ** 31     # what a C int holds
    for c in range(n_be):
        assert 10 < res["iters_done"][c] < 10_000          # ran all three phases, then stopped
    obs = open(os.path.join(str(tmp_path), "observations.log")).read()
    dec = open(os.path.join(str(tmp_path), "decisions.log")).read()
    assert obs.count(".steady") == n_be                    # one setup_change per trainer
    assert dec.count("\nD ") > 100
    assert obslog.replay(obs) == dec and jobs.native_replay(obs) == dec


@pytest.mark.parametrize("direct", [True, False])
def test_a_captured_graph_is_one_record(tmp_path, direct):
    """The high-priority client submits every iteration as one executable graph
    (hipGraphLaunch): the scheduler counts one kernel-class record per iteration,
    the result is the same, the log replays bit-exactly."""
    hp_iters = 30
    res = run_child(str(tmp_path), "orion", 2, hp_iters, direct, graph=True)
    assert not any(res["alive"])
    assert res["iters_done"][-1] == hp_iters and all(res["outputs_equal"]), res
    hp_tid, sched = res["client_tids"][-1], res["sched_tid"][0]
    issuer = str(hp_tid if direct else sched)
    assert issuer in res["launches_by_tid"]
    if direct:      # one launch per iteration, all but the first by the client itself
        assert hp_iters - 1 <= res["launches_by_tid"][str(hp_tid)] <= hp_iters
    obs = open(os.path.join(str(tmp_path), "observations.log")).read()
    dec = open(os.path.join(str(tmp_path), "decisions.log")).read()
    hp = [l.split() for l in dec.splitlines() if l.startswith(f"D 2 ")]
    assert sum(1 for x in hp if x[3] == "k") == hp_iters      # one kernel record each
    assert obslog.replay(obs) == dec and jobs.native_replay(obs) == dec


@pytest.mark.parametrize("pin", [True, False])
def test_client_threads_are_pinned_while_the_job_runs(tmp_path, pin):
    """reference: utils_interc.cpp:36-49 -- each client thread gets a CPU of its
    own the first time it is identified.  Client i runs on the (i + 2)-th CPU
    the process may use (the first stays with the other threads); the mask is
    given back when the job ends; ORION_PIN_THREADS=0 pins nothing."""
    n_be = 2
    if len(os.sched_getaffinity(0)) < n_be + 3:
        pytest.skip("fewer CPUs than clients + scheduler + 1")
    res = run_child(str(tmp_path), "orion", n_be, 20, pin=pin)
    assert not any(res["alive"]) and all(res["outputs_equal"])
    allowed = res["allowed_cpus"]            # main thread, after the job: untouched
    assert allowed == sorted(os.sched_getaffinity(0))
    for i, (cpu, mask) in enumerate(res["placement"]):
        if pin:
            assert cpu == allowed[i + 1] and mask == [cpu]
        else:
            assert cpu == -1 and mask == allowed
    # the scheduler thread takes the slot after the last client
    assert res["scheduler_placement"] == ([allowed[n_be + 2]] if pin else allowed)
    assert res["scheduler_mask_after"] == allowed


def test_kernel_count_mismatch_ends_the_job_with_a_report(tmp_path):
    """The reference spins forever when a client submits fewer kernels per
    iteration than its profile names (scheduler_eval.cpp:282, :389).  Here the
    scheduler notices that nothing is dispatched or completed while a client
    waits, prints what it sees per client and aborts."""
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "tests", "fake_runner.py"), str(tmp_path),
         "orion", "1", "20"],
        capture_output=True, text=True, timeout=120,
        env=dict(os.environ, FAKE_RUNNER_MISCOUNT="1", ORION_STUCK_LIMIT_S="1"))
    assert proc.returncode != 0
    assert "kernel count probably differs" in proc.stderr
    # client 0 has handed over all 5 of the 6 kernels the scheduler was told about
    assert "client 0: 5 of 6 kernel records seen this iteration" in proc.stderr
    assert "block() calls 1, iterations released 0" in proc.stderr


def test_more_kernels_than_the_profile_names_is_reported_at_once(tmp_path):
    """The other direction of the mismatch: a client whose iteration holds more
    kernel records than its profile.  The reference matches every later kernel
    with the wrong profile row and runs on; here the scheduler sees the first
    kernel of the "next" iteration arrive before the client has called block()
    and ends the job."""
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "tests", "fake_runner.py"), str(tmp_path),
         "orion", "1", "20"],
        capture_output=True, text=True, timeout=120,
        env=dict(os.environ, FAKE_RUNNER_MISCOUNT="-1", ORION_STUCK_LIMIT_S="2"))
    assert proc.returncode != 0
    # seen by the scheduler (the extra kernel arrives while it polls, or is still
    # queued when a warm-up phase ends) or, when the scheduler has already left
    # for the rendezvous, by the client that waits for it in vain
    assert ("client 0 submits more kernel records per iteration than the 4 its profile names"
            in proc.stderr
            or "client 0 has had a record (type" in proc.stderr), proc.stderr[-2000:]


def test_a_count_mismatch_names_the_row_where_the_client_leaves_its_profile(tmp_path):
    """A profile captured with one kernel more than the run launches (a different
    convolution solver, an extra cast): the job still ends -- the count is what
    the policy runs on -- but the report now says where the two part: the first
    profile row whose name is not the name of the kernel launched there, and
    both names.  (The reference spins forever, scheduler_eval.cpp:282.)"""
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "tests", "fake_runner.py"), str(tmp_path),
         "orion", "1", "20"],
        capture_output=True, text=True, timeout=120,
        env=dict(os.environ, FAKE_RUNNER_MISCOUNT="1", ORION_STUCK_LIMIT_S="1",
                 FAKE_RUNNER_NAMED_PROFILE="1", FAKE_RUNNER_PROFILE_INSERT="2"))
    assert proc.returncode != 0
    assert "kernel count probably differs" in proc.stderr
    assert ("client 0: first difference at profile row 2: the profile names 'fake_extra', "
            "the client launched 'fake_kernel_saxpy'") in proc.stderr, proc.stderr[-2000:]


def test_a_kernel_beyond_the_profile_is_named(tmp_path):
    """The other direction: every row of the profile matches, and the client
    launches one kernel more.  The report names that kernel."""
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "tests", "fake_runner.py"), str(tmp_path),
         "orion", "1", "20"],
        capture_output=True, text=True, timeout=120,
        env=dict(os.environ, FAKE_RUNNER_MISCOUNT="-1", ORION_STUCK_LIMIT_S="2",
                 FAKE_RUNNER_NAMED_PROFILE="1"))
    assert proc.returncode != 0
    if "submits more kernel records per iteration" in proc.stderr:
        # the scheduler saw it: rows 0..3 agree, the fifth kernel (an even row: saxpy) is extra
        assert "carry the names of profile rows 0..3" in proc.stderr, proc.stderr[-2000:]
        assert "after the profile's last row (4 rows) it launched 'fake_kernel_saxpy'" in proc.stderr
    else:   # the scheduler had left for the rendezvous; the waiting client reports
        assert "client 0 has had a record (type" in proc.stderr, proc.stderr[-2000:]


@pytest.mark.parametrize("async_exec", [False, True])
def test_recorded_policy_options_on_the_fake_runtime(tmp_path, async_exec):
    """The policy options that are not in the reference (ORION_ADMIT_OVERSIZED,
    ORION_SLIDING_THROTTLE, with the two older ones) through the live scheduler:
    same outputs, the options named in the log header, and the recorded run
    replayed bit-exactly by the oracle and the native core -- the marks the
    sliding throttle asks about are events the live host has to keep."""
    options = {"ORION_ADMIT_OVERSIZED": "1", "ORION_SLIDING_THROTTLE": "1",
               "ORION_RESERVE_HP_CUS": "1", "ORION_CONFINE_LONG_BE": "1"}
    res = run_child(str(tmp_path), "orion", 2, 40, async_exec=async_exec, extra_env=options)
    assert not any(res["alive"]) and all(res["outputs_equal"]), res
    obs = open(os.path.join(str(tmp_path), "observations.log")).read()
    dec = open(os.path.join(str(tmp_path), "decisions.log")).read()
    assert obs.splitlines()[0].split(" ")[4:] == ["L1", "R1", "O1", "T1"]
    assert dec.count("\nD ") > 100
    assert obslog.replay(obs) == dec
    assert jobs.native_replay(obs) == dec
