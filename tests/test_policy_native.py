"""The native policy core against the CPU oracle: bit-exact decision logs.

Each case builds a random job (profiles, traces, arrival gaps), runs the Python
oracle under the virtual-time model while recording what it observed, then has
the native core (liborion_policy.so) replay those observations.  The two
decision logs must be identical byte for byte.  The oracle's own replayer must
reproduce its log too (the log format loses nothing).
"""

import pytest

from oracle import obslog, policy_oracle as po
from tests import jobs


def _check(tmp_path, **kw):
    job = jobs.make_job(str(tmp_path), **kw)
    oracle, env, rec = jobs.run_oracle(job)
    want = rec.dec.text()
    assert want.count("\nD ") > 20
    got = jobs.native_replay(rec.obs_text(), job.sequential_fix)
    assert got == want
    again = obslog.replay(rec.obs_text(), sequential_fix=job.sequential_fix)
    assert again == want
    return oracle, env, rec


@pytest.mark.parametrize("seed", range(12))
@pytest.mark.parametrize("n_clients", [1, 2, 3, 4])
def test_orion_inference_hp(tmp_path, seed, n_clients):
    oracle, env, rec = _check(tmp_path, seed=seed, n_clients=n_clients)
    assert oracle.cur_iters[-1] == 25


@pytest.mark.parametrize("seed", range(4))
@pytest.mark.parametrize("n_clients", [2, 3])
def test_a_cu_budget_of_one_holds_best_effort_kernels_while_a_request_is_in_flight(
        tmp_path, seed, n_clients):
    """max_sms = 1 (ORION_MAX_SMS=1, the setting for inference beside inference):
    the CU clause ``size + sm_used <= max_sms`` (scheduler_eval.cpp:339-340) can
    admit no kernel that needs more than one CU, so while a high-priority request
    is in flight (``seen[hp] > 0``) no such best-effort kernel is dispatched;
    between requests they go at once (:333).  Oracle and native core agree bit
    for bit, and the rule is checked decision by decision on the oracle's log."""
    from tests.test_policy_properties import check_orion_invariants

    def held_kernels(max_sms):
        work = tmp_path / str(max_sms)
        work.mkdir()
        job = jobs.make_job(str(work), seed=400 + seed, n_clients=n_clients, max_sms=max_sms,
                            hp_iters=200)
        # the reference's rule alone (the random job may have drawn an option)
        job.admit_oversized = job.sliding_throttle = False
        job.reserve_hp = job.confine_long = False
        oracle, env, rec = jobs.run_oracle(job)
        marked = jobs.native_replay(rec.obs_text(), by_poll=True)
        assert "".join(l + "\n" for l in marked.splitlines() if l != "P") == rec.dec.text()
        # the reference's per-poll rules, re-stated on the logs, at this budget
        check_orion_invariants(rec.obs_text(), marked, job.depth)
        hp = n_clients - 1
        in_flight, done, during, between = False, [0] * n_clients, 0, 0
        for line in rec.dec.text().splitlines():
            f = line.split(" ")
            if f[0] == "D" and f[3] == "k":
                client = int(f[1])
                if client == hp:
                    in_flight = True
                elif (done[client] > 10 and done[hp] < oracle.max_iters[hp]      # past :335
                      and oracle.ops[client][int(f[4])].sm_used > 1):
                    during += in_flight
                    between += not in_flight
            elif f[0] == "F":
                done[int(f[1])] += 1
                if int(f[1]) == hp:
                    in_flight = False
            elif f[0] == "S":           # a new call of schedule(): iterations count from 0
                in_flight, done = False, [0] * n_clients
        return during, between

    during_1, between_1 = held_kernels(1)
    during_256, _ = held_kernels(256)
    assert during_1 == 0 and between_1 > 5
    assert during_256 > 0        # the same job under the device's budget admits some


@pytest.mark.parametrize("seed", range(8))
@pytest.mark.parametrize("n_clients", [2, 3])
def test_orion_training_hp(tmp_path, seed, n_clients):
    # exercises the update-phase admission and the threshold bisection
    _check(tmp_path, seed=100 + seed, n_clients=n_clients, hp_train=True,
           hp_iters=45)


@pytest.mark.parametrize("seed", range(8))
@pytest.mark.parametrize("n_clients", [1, 2, 4])
def test_reef(tmp_path, seed, n_clients):
    _check(tmp_path, seed=200 + seed, n_clients=n_clients, algo=po.ALGO_REEF)


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("n_clients", [1, 2, 3])
def test_sequential_repaired(tmp_path, seed, n_clients):
    _check(tmp_path, seed=300 + seed, n_clients=n_clients,
           algo=po.ALGO_SEQUENTIAL, sequential_fix=True)


def test_sequential_as_written_stalls_after_warmup(tmp_path):
    # The reference text cannot dispatch once a client is past iteration 10
    # (scheduler_eval.cpp:185-198, :211-223): the run never ends.
    job = jobs.make_job(str(tmp_path), seed=7, n_clients=2,
                        algo=po.ALGO_SEQUENTIAL, sequential_fix=False)
    with pytest.raises(RuntimeError, match="poll budget"):
        jobs.run_oracle(job, max_polls=20_000)


def test_replay_detects_divergence(tmp_path):
    job = jobs.make_job(str(tmp_path), seed=3, n_clients=2)
    _, _, rec = jobs.run_oracle(job)
    lines = rec.obs_text().splitlines()
    # flip one queue head: the policy must notice that the log no longer fits
    for i, l in enumerate(lines):
        if l.startswith("P ") and l.split(" ")[2][0] == "k":
            parts = l.split(" ")
            parts[2] = "." + parts[2][1:]
            lines[i] = " ".join(parts)
            break
    bad = "\n".join(lines) + "\n"
    with pytest.raises(RuntimeError, match="native replay failed"):
        jobs.native_replay(bad)
    with pytest.raises(obslog.ReplayDivergence):
        obslog.replay(bad)
