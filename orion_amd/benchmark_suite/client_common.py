"""What every client loop shares: the control calls into libinttemp.so, the
arrival schedule, the request loop with its barrier protocol, and the result
file.  Behaviour follows the reference's loops
(benchmarking/benchmark_suite/train_imagenet.py:71-241,
bert_trainer_mock.py:49-234); the line numbers below are train_imagenet.py's.
"""

import json
import os
import random
import threading
import time

import numpy as np
import torch

from .. import scheduler_frontend as fe

WARMUP_ITERS = 10     # iterations before the measured run (:188-198, :220)

# Weight initialisation draws from the process-wide generator.  Clients seed it
# and build their model while holding this lock, so a client's weights do not
# depend on which other clients share the process (its output can then be
# compared with its isolated run).
MODEL_INIT_LOCK = threading.RLock()

# One client at a time runs its un-captured set-up (model build, library
# initialisation, warm-up steps, HIP-graph capture).  A stream capture in one
# thread makes calls of other threads that touch the legacy stream fail
# (hipBLASLt's initialisation does: "operation would make the legacy stream
# depend on a capturing blocking stream"), so the set-up phases must not overlap.
SETUP_LOCK = threading.RLock()


def seed_everything(seed):
    """:22-30."""
    random.seed(seed)
    os.environ["PYTHONHASHSEED"] = str(seed)
    np.random.seed(seed)
    torch.manual_seed(seed)
    if torch.cuda.is_available():
        torch.cuda.manual_seed(seed)


def arrival_gaps(rps, uniform, num_iters, input_file="", seed=42):
    """Inter-arrival gaps in seconds (:89-98): constant 1/rps, exponential with
    mean 1/rps from a generator seeded like the reference's global numpy seed,
    a JSON trace, or zeros (closed loop)."""
    if rps > 0 and input_file == "":
        if uniform:
            return [1.0 / rps] * num_iters
        return list(np.random.RandomState(seed).exponential(scale=1.0 / rps,
                                                            size=num_iters))
    if input_file != "":
        with open(input_file) as f:
            return list(json.load(f))
    return [0.0] * num_iters


def latency_summary(timings, batch_idx, total_time, train, drop=WARMUP_ITERS):
    """Result dictionary of a client (:220-237): drop the warm-up requests,
    percentiles in milliseconds, throughput over the measured run."""
    timings = sorted(timings[drop:])
    throughput = (batch_idx - WARMUP_ITERS) / total_time if total_time > 0 else 0.0
    if not train and len(timings) > 0:
        return {
            "p50_latency": float(np.percentile(timings, 50) * 1000),
            "p95_latency": float(np.percentile(timings, 95) * 1000),
            "p99_latency": float(np.percentile(timings, 99) * 1000),
            "throughput": throughput,
        }
    return {"throughput": throughput}


def loss_checkpoints():
    """ORION_LOSS_AT_ITERATION=N[,M...]: a training client keeps the loss tensors
    of these scheduled iterations (no copy, no wait: the tensors are simply not
    let go) and reports their values after the run.  The loss of iteration N
    depends on every parameter update before it, so two runs of the same client
    -- alone, and beside other clients -- can be compared at fixed points although
    they run for different numbers of iterations.  Empty: off."""
    text = os.environ.get("ORION_LOSS_AT_ITERATION", "")
    return {int(t) for t in text.split(",") if t.strip()}


def keep_loss(state, batch_idx, loss):
    if batch_idx in loss_checkpoints():
        state.setdefault("loss_at", {})[batch_idx] = loss     # read back after the run


def loss_checkpoint_report(state):
    """``loss_at_iteration``: iteration -> [value, bit pattern of the fp32 value]."""
    out = {}
    for it, loss in sorted(state.get("loss_at", {}).items()):
        value = loss.detach().float().cpu()
        out[str(it)] = [float(value), int(value.view(torch.int32))]
    return {"loss_at_iteration": out} if out else {}


def brief(data):
    """A result without its per-request list, for the one-line report."""
    return {k: v for k, v in data.items() if k != "latencies_ms"}


def write_result(tid, data):
    out_dir = os.environ.get("ORION_RESULT_DIR", ".")
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, f"client_{tid}.json"), "w") as f:
        json.dump(data, f)


# Raised by the launcher's ``--algo streams`` baseline (no scheduler: nobody else
# could tell the best-effort clients that the high-priority client is done).
UNSCHEDULED_STOP = threading.Event()


class Backend:
    """block()/stop() of libinttemp.so (:63-68, :88) plus stream registration."""

    def __init__(self):
        self.lib = fe.load_capture_library()
        # ORION_PLAIN_TLS_REFRESH=1: a client that runs unscheduled (plain stream)
        # gets, once per request, the same treatment scheduled clients get from
        # the interception library: its thread-local accesses are taken off the
        # dynamic loader's slow path (csrc/capture/tls_fresh.h).  For measuring
        # what the scheduling path itself costs, like for like.
        self.plain_tls_refresh = os.environ.get("ORION_PLAIN_TLS_REFRESH", "0") not in ("", "0")

    def block(self, it):
        """Wait until iteration ``it`` has completed on the GPU.  Under the
        scheduler that is libinttemp's block(); when the calling thread is not a
        scheduled client (stand-alone runs) the current stream is synchronised
        instead, so the loop measures the same thing either way."""
        if self.lib.orion_client_index() >= 0:
            self.lib.block(it)
        else:
            if self.plain_tls_refresh:
                self.lib.orion_tls_fresh_check()
            if torch.cuda.is_available():
                torch.cuda.current_stream().synchronize()

    def stop(self):
        return bool(self.lib.stop()) or UNSCHEDULED_STOP.is_set()

    def time_in_calls_ns(self):
        """Time this thread has spent inside the interposed launch and copy
        entry points (0 unless ORION_CALL_TIMING=1)."""
        return int(self.lib.orion_thread_time_in_calls_ns())

    def tls_fresh_stats(self):
        """Reloads of the thread-local helper library in this process so far, and
        calls of threads into a fresh copy (csrc/capture/tls_fresh.h)."""
        import ctypes
        lib = getattr(self, "lib", None)
        if lib is None:
            return None
        reloads, touches = ctypes.c_ulonglong(), ctypes.c_ulonglong()
        lib.orion_tls_fresh_stats(ctypes.byref(reloads), ctypes.byref(touches))
        return {"reloads": int(reloads.value), "touches": int(touches.value)}

    def register_stream(self, stream):
        self.lib.orion_register_stream(stream.cuda_stream)

    def passthrough(self, on):
        self.lib.orion_thread_passthrough(1 if on else 0)


class uncaptured:
    """Context in which the calling thread's GPU work bypasses the scheduler.

    On ROCm the first executions of a model run library auto-tuning (MIOpen
    tries several convolution solvers and times them) and lazy initialisation
    whose number of kernels is not reproducible, so no profile could name a row
    count for them.  A client therefore builds its model and runs its first
    steps here, synchronises, and only then starts the iterations the scheduler
    counts."""

    def __init__(self, backend):
        self.backend = backend

    def __enter__(self):
        SETUP_LOCK.acquire()
        self.backend.passthrough(True)

    def __exit__(self, *exc):
        try:
            self._leave()
        finally:
            SETUP_LOCK.release()

    def _leave(self):
        if torch.cuda.is_available():
            torch.cuda.synchronize()
        self.backend.passthrough(False)
        return False

UNCAPTURED_STEPS = 3  # auto-tuning, lazy init, first optimizer step, one more


def run_client(tid, train, num_iters, sleep_times, barriers, step, backend,
               drop=WARMUP_ITERS, extra=None):
    """The request loop.  ``step(batch_idx)`` submits one iteration's GPU work.

    Training clients run closed loop (:141-169).  Inference clients run open
    loop (:170-204): request i is due at ``next_startup``; its latency counts
    from that due time, so queueing delay is included; the due time advances by
    the arrival gap once the client is past warm-up.  Both rendezvous with the
    scheduler on ``barriers[0]`` after iterations 1 and 10 and once at the end.
    """
    timings = []
    # ORION_CLIENT_STAMPS=1: per request, how long the client spent submitting
    # (inside step) and how long waiting for completion (inside block)
    stamps = [] if os.environ.get("ORION_CLIENT_STAMPS", "0") not in ("", "0") else None
    batch_idx = 0
    start = time.time()
    next_startup = time.time()
    while batch_idx < num_iters:
        if train:
            start_iter = time.time()
            step(batch_idx)
            backend.block(batch_idx)
            timings.append(time.time() - start_iter)
            batch_idx += 1
            if batch_idx == 1:
                barriers[0].wait()
            if batch_idx == WARMUP_ITERS:
                barriers[0].wait()
                start = time.time()
            if backend.stop():
                break
        else:
            if time.time() < next_startup:
                continue
            t_begin = time.time()
            in_calls = backend.time_in_calls_ns() if stamps is not None else 0
            step(batch_idx)
            t_submitted = time.time()
            in_calls = backend.time_in_calls_ns() - in_calls if stamps is not None else 0
            backend.block(batch_idx)
            t_done = time.time()
            timings.append(t_done - next_startup)
            if stamps is not None:
                stamps.append((t_begin - next_startup, t_submitted - t_begin,
                               t_done - t_submitted, in_calls * 1e-9))
            if batch_idx >= WARMUP_ITERS and sleep_times[batch_idx] > 0:
                next_startup += sleep_times[batch_idx]
            else:
                # warm-up, or a closed loop (rps 0): the next request is due now.
                # (The reference adds a zero gap here, :188-189, which leaves the
                # due time in the past and inflates every later latency.)
                next_startup = time.time()
            batch_idx += 1
            if batch_idx in (1, WARMUP_ITERS):
                barriers[0].wait()
                if batch_idx == WARMUP_ITERS:
                    next_startup = time.time()
                    start = time.time()
            dur = next_startup - time.time()
            if dur > 0:
                time.sleep(dur)
            if backend.stop():
                break
    barriers[0].wait()
    total_time = time.time() - start
    data = latency_summary(timings, batch_idx, total_time, train, drop)
    if extra:
        data.update(extra())
    data["iterations"] = batch_idx
    fresh = backend.tls_fresh_stats() if hasattr(backend, "tls_fresh_stats") else None
    if fresh is not None:
        data["tls_fresh"] = fresh
    if not train:
        # every measured request, in arrival order (the reference's file holds
        # the percentiles only): lets runs be pooled
        data["latencies_ms"] = [round(float(t) * 1000, 4) for t in timings[drop:]]
        if stamps is not None:
            # submit_in_calls_ms: the part of submit_ms spent inside the interposed
            # launch and copy calls (ORION_CALL_TIMING=1 and the library preloaded)
            for k, name in enumerate(("start_delay_ms", "submit_ms", "wait_ms",
                                      "submit_in_calls_ms")):
                data[name] = [round(float(s[k]) * 1000, 4) for s in stamps[drop:]]
    write_result(tid, data)
    return data
