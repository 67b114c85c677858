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
