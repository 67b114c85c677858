"""Synthetic jobs for policy tests: random profiles and traces, run through the
oracle under the virtual-time model, and the native core's replay of the log."""

import ctypes
import os
import random

import numpy as np

from oracle import obslog, policy_oracle as po, virtual_gpu as vg
from orion_amd import _lib

HEADER = "Name,Profile,Memory_footprint,SM_usage,Duration\n"


def write_profile(path, ops):
    with open(path, "w") as f:
        f.write(HEADER)
        for o in ops:
            f.write(f"{o.name},{o.profile},{o.mem},{o.sm_used},{o.duration}\n")


def random_ops(rng, n, max_sm=400, max_ns=400_000, placeholder=False):
    ops = []
    for i in range(n):
        if placeholder:
            ops.append(po.OpInfo(f"op{i}", -1, 1, 1, np.float32(7)))
        else:
            ops.append(po.OpInfo(
                f"op{i}", rng.choice([-1, 0, 1]), 0, rng.randint(1, max_sm),
                np.float32(rng.randint(1_000, max_ns))))
    return ops


def random_trace(rng, num_kernels, extra_tail=True):
    """One iteration's records: exactly num_kernels kernel-like records with
    memory records sprinkled in (a copy first, like the H2D of the input)."""
    trace = [po.MEMCPY]
    for _ in range(num_kernels):
        if rng.random() < 0.15:
            trace.append(rng.choice([po.MEMSET, po.MEMCPY, po.MALLOC, po.FREE]))
        trace.append(po.KERNEL)
    if extra_tail and rng.random() < 0.5:
        trace.append(po.MEMCPY)     # the output copy after the last kernel
    return trace


class Job:
    pass


def make_job(tmp_path, seed, n_clients=2, algo=po.ALGO_ORION, hp_train=False,
             hp_iters=25, max_sms=256, masks=(32, 64, 128, 256), depth=None,
             be_first_iter_differs=True, sequential_fix=True):
    rng = random.Random(seed)
    job = Job()
    job.n = n_clients
    job.algo = algo
    job.max_sms = max_sms
    job.masks = list(masks)
    job.sequential_fix = sequential_fix
    job.paths, job.ops, job.nk, job.iters, job.train = [], [], [], [], []
    job.swap = {}
    traces = []
    for c in range(n_clients):
        is_hp = c == n_clients - 1
        train = hp_train if is_hp else (rng.random() < 0.8 or n_clients == 1)
        nk = rng.randint(3, 14)
        ops = random_ops(rng, nk)
        path = os.path.join(tmp_path, f"c{c}_main.csv")
        write_profile(path, ops)
        first_nk, first_path = nk, path
        if train and be_first_iter_differs and rng.random() < 0.7:
            first_nk = rng.randint(2, 10)
            first_path = os.path.join(tmp_path, f"c{c}_first.csv")
            write_profile(first_path, random_ops(rng, first_nk, placeholder=True))
            job.swap[c] = (path, nk)
        tr_main = random_trace(rng, nk)
        tr_first = random_trace(rng, first_nk)
        traces.append((tr_first, tr_main))
        job.paths.append(first_path)
        job.nk.append(first_nk)
        job.train.append(train)
        job.iters.append(hp_iters if is_hp else 10_000)
    job.depth = depth if depth is not None else rng.choice(
        [1, 50_000, 200_000, 1_000_000])
    job.hp_limit = rng.randint(1, 3)
    job.update_start = rng.randint(1, max(1, job.nk[-1] - 1))
    if algo == po.ALGO_REEF:
        job.depth = rng.randint(1, 12)
    job.traces = traces
    job.arrivals = [rng.randint(20_000, 2_000_000) for _ in range(16)]
    job.closed_loop_hp = rng.random() < 0.3 or hp_train
    job.confine_long = rng.random() < 0.5
    job.reserve_hp = rng.random() < 0.4
    job.admit_oversized = rng.random() < 0.4
    job.sliding_throttle = rng.random() < 0.4
    return job


def run_oracle(job, max_polls=3_000_000):
    profiles = [po.parse_profile(p) for p in job.paths]
    oracle = po.PolicyOracle(profiles, job.nk, job.iters, job.train,
                             max_sms=job.max_sms,
                             sequential_fix=job.sequential_fix,
                             reserve_hp=getattr(job, "reserve_hp", False),
                             admit_oversized=getattr(job, "admit_oversized", False),
                             sliding_throttle=getattr(job, "sliding_throttle", False))
    clients = []
    for c in range(job.n):
        first, main = job.traces[c]
        is_hp = c == job.n - 1
        arrivals = None
        if is_hp and not job.closed_loop_hp:
            arrivals = job.arrivals
        clients.append(vg.VClient(
            (lambda it, f=first, m=main: f if it == 0 else m),
            job.iters[c], gap_ns=1500 + 500 * c, arrivals=arrivals))
    env = vg.VirtualGpu(clients, lambda c, k: int(oracle.ops[c][k].duration))
    rec = obslog.RecordingEnv(env, job.n, job.masks,
                              lambda c, k: oracle.ops[c][k], algo=job.algo,
                              hp_active=lambda: oracle.seen[job.n - 1] > 0)
    rec.budget = job.depth
    rec.header(job.max_sms, [(job.nk[c], job.iters[c], job.train[c],
                              job.paths[c]) for c in range(job.n)],
               confine_long=getattr(job, "confine_long", False),
               reserve_hp=getattr(job, "reserve_hp", False),
               admit_oversized=getattr(job, "admit_oversized", False),
               sliding_throttle=getattr(job, "sliding_throttle", False))
    changes = {1: [(c, po.parse_profile(path), nk, path)
                   for c, (path, nk) in sorted(job.swap.items())]}
    vg.run_job(oracle, env, rec, [(True, 1), (True, 10), (False, 0)],
               setup_changes=changes, algo=job.algo, depth=job.depth,
               hp_limit=job.hp_limit, update_start=job.update_start,
               max_polls=max_polls)
    return oracle, env, rec


_policy = None


def policy_lib():
    global _policy
    if _policy is None:
        lib = _lib.load(_lib.POLICY_LIB)
        lib.orion_policy_replay.argtypes = [
            ctypes.c_char_p, ctypes.c_int, ctypes.POINTER(ctypes.c_void_p),
            ctypes.POINTER(ctypes.c_void_p)]
        lib.orion_policy_replay.restype = ctypes.c_int
        lib.orion_policy_replay_by_poll.argtypes = lib.orion_policy_replay.argtypes
        lib.orion_policy_replay_by_poll.restype = ctypes.c_int
        lib.orion_policy_free.argtypes = [ctypes.c_void_p]
        lib.orion_policy_free.restype = None
        lib.orion_profile_stats.argtypes = [
            ctypes.c_char_p, ctypes.POINTER(ctypes.c_int),
            ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_double),
            ctypes.POINTER(ctypes.c_void_p)]
        lib.orion_profile_row.argtypes = [
            ctypes.c_char_p, ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t,
            ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int),
            ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_float)]
        lib.orion_place_cu_slot.argtypes = [
            ctypes.POINTER(ctypes.c_int), ctypes.c_int, ctypes.c_int,
            ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        _policy = lib
    return _policy


def native_replay(obs_text, sequential_fix=True, by_poll=False):
    """Decision log of the native policy core for an observation log."""
    from orion_amd import replay
    try:
        return replay.native_replay(obs_text, by_poll=by_poll, sequential_fix=sequential_fix)
    except replay.ReplayError as e:
        raise RuntimeError(f"native replay failed: {e}") from e
