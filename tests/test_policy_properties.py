"""Invariants of the Orion policy, checked poll by poll on the NATIVE core.

hypothesis draws jobs (profiles, traces, arrival patterns, budgets, client
counts); the virtual-time model produces an observation log; the native core
replays it with poll marks (orion_policy_replay_by_poll).  The checks below are
read off the reference's loop (src/scheduler/scheduler_eval.cpp:277-400), not
off this build's oracle; the only state they keep is the reference's own
bookkeeping (seen[], iteration counts, the running best-effort duration sum):

* a client whose iteration is fully dispatched is not peeked (:281-282);
* a high-priority record at the head of its queue is dispatched in the same
  poll, before any best-effort record (:307-318);
* one dispatch per client and poll at most, of the record class that was peeked;
* best-effort clients are visited in rotation from the one after the last
  client dispatched (:320-323, :383);
* a best-effort record MUST go out when the high-priority client is idle, the
  record is a memory operation, the client is within its first ten iterations,
  or the high-priority client has finished (:330-335) -- unless the duration
  throttle is on;
* a best-effort kernel that goes out beside a running high-priority iteration
  fits the CU budget of this poll and is of the opposite (or unknown) class
  (:339);
* once the running sum of profiled durations exceeds the budget nothing
  best-effort goes out until a poll that queried events (:341-357, :363-367);
* (this build's recorded option R1) the room of the CU budget is what the
  high-priority op last dispatched leaves of it;
* (this build's recorded option O1) the one exception to the CU budget: a kernel
  whose own need exceeds the device, let in as the first best-effort kernel of
  a poll, on the smallest mask, beside an inference request whose running op
  has the other known class, and no longer than a quarter of the budget.

Profile durations are whole numbers below 2^24, so the reference's float/long
sum is exact here.

REEF (schedule_reef, :93-165) is simpler: which clients a poll dispatches is a
function of what the poll saw and three counters, so the whole rule is checked,
not only invariants of it.
"""

import csv
import os

import pytest
from hypothesis import HealthCheck, given, settings, strategies as st

from oracle import policy_oracle as po
from tests import jobs

RECORD = set("kcmfs")


def rows_of(path):
    with open(path) as f:
        return [(int(r["Profile"]), int(r["SM_usage"]), int(float(r["Duration"])))
                for r in csv.DictReader(f)]


def check_orion_invariants(obs_text, dec_text, depth):
    obs, dec = obs_text.splitlines(), dec_text.splitlines()
    at = 0                                   # cursor in dec

    def take(expect=None):
        nonlocal at
        line = dec[at]
        at += 1
        if expect is not None:
            assert line == expect, (line, expect)
        return line

    n = max_sms = None
    nk, max_iters, prof = {}, {}, {}
    seen, iters, event_ids = {}, {}, {}
    checked = {"must": 0, "budget": 0, "throttle": 0, "rotation": 0}
    for line in obs:
        p = line.split(" ")
        if p[0] == "J":
            n, max_sms = int(p[1]), int(p[2])
            hp = n - 1
            reserve_hp = "R1" in p[4:]      # this build's option: see below
            admit_oversized = "O1" in p[4:]
            # T1 changes WHEN the duration throttle lets go (at a half-way mark,
            # with part of the sum kept): the two throttle checks below describe
            # the reference's all-or-nothing release and are skipped for it; the
            # option has its own hand-worked trace (test_policy_sliding_throttle)
            sliding = "T1" in p[4:]
            hp_need = 0
            hp_trains = False
        elif p[0] == "K":
            c = int(p[1])
            nk[c], max_iters[c], prof[c] = int(p[2]), int(p[3]), rows_of(p[5])
            seen[c], iters[c], event_ids[c] = 0, 0, 0
            if c == n - 1:
                hp_trains = bool(int(p[4]))
        elif p[0] == "X":
            c = int(p[1])
            nk[c], prof[c] = int(p[2]), rows_of(p[3])
            take(f"X {c}")
        elif p[0] == "S":
            take("S")
            throttled, running, start = False, 0, -1      # locals of schedule() (:258-261)
            hp_profile = None                             # profiles[hp], last HP record's row
        elif p[0] == "E":
            take("E")
        elif p[0] == "P":
            take("P")
            heads, events = p[2], p[3]
            block = []
            while at < len(dec) and dec[at][0] in "DFT":
                block.append(take().split(" "))
            for c in range(n):
                if seen[c] == nk[c]:
                    assert heads[c] == "-", (line, c)
            ds = [b for b in block if b[0] == "D"]
            clients = [int(b[1]) for b in ds]
            assert len(set(clients)) == len(clients)
            for b in ds:
                assert heads[int(b[1])] == b[3], (line, b)
            if heads[hp] in RECORD:
                assert ds and int(ds[0][1]) == hp, (line, block)
            be_order = [c for c in clients if c != hp]
            if n > 1 and be_order:
                rotation = [(start + 1 + i) % (n - 1) for i in range(n - 1)]
                assert be_order == [c for c in rotation if c in be_order], (start, be_order)
                checked["rotation"] += 1
            size = 0
            poll_throttled = throttled or sliding     # on at any moment of this poll
            for b in ds:
                c, cls, op = int(b[1]), b[3], int(b[4])
                assert op == seen[c] and int(b[5]) == event_ids[c]
                row = prof[c][op] if op < len(prof[c]) else None
                if c == hp:
                    hp_profile = row[0] if row else None
                    hp_need = max(0, row[1]) if row else 0
                    if cls == "k":        # only kernel records advance either counter
                        seen[c] += 1      # (utils_sched.cpp:240-249 against :251-282)
                        event_ids[c] += 1
                    continue
                hp_done = iters[hp] >= max_iters[hp]
                if throttled:
                    # released only by a poll that asked the GPU about every
                    # best-effort client with an event outstanding (:343-352)
                    if any(event_ids[k] >= 1 for k in range(n - 1)) and not sliding:
                        assert "1" in events, (line, b)
                        checked["throttle"] += 1
                    throttled, running = False, 0
                free_pass = (n == 1 or seen[hp] == 0 or cls != "k" or iters[c] <= 10
                             or hp_done)
                if (not free_pass and row is not None and hp_profile is not None
                        and admit_oversized and size + row[1] > max_sms):
                    # the exception, and nothing but the exception
                    assert size == 0 and row[1] > max_sms and not hp_trains, (line, b, size)
                    assert row[0] != -1 and hp_profile != -1 and row[0] != hp_profile, (line, b)
                    assert row[2] <= depth // 4, (line, b, depth)
                    assert int(b[6]) == 0, (line, b)           # the smallest mask
                    checked["oversized"] = checked.get("oversized", 0) + 1
                elif not free_pass and row is not None and hp_profile is not None:
                    assert size + row[1] <= max_sms, (line, b, size)
                    if reserve_hp:      # the HP op's own CU need is taken out of the room
                        assert size + row[1] <= max(0, max_sms - hp_need), (line, b, hp_need)
                        checked["reserved"] = checked.get("reserved", 0) + 1
                    assert row[0] == -1 or hp_profile == -1 or row[0] != hp_profile, (line, b)
                    checked["budget"] += 1
                if row is not None:
                    size += row[1]
                    if cls == "k":
                        running += row[2]
                if cls == "k":
                    seen[c] += 1
                    event_ids[c] += 1
                if running > depth and not hp_done:
                    throttled = poll_throttled = True
                start = c
            # records that had to go out and did not
            for c in range(n - 1):
                if heads[c] in RECORD and c not in clients and not poll_throttled:
                    free_pass = (seen[hp] == 0 or heads[c] != "k" or iters[c] <= 10
                                 or iters[hp] >= max_iters[hp])
                    # (a poll during which the throttle was on at any moment does
                    # not count: on a live GPU the answers of the event queries
                    # change between two clients of the same rotation)
                    assert not free_pass, (line, c, block)
                    checked["must"] += 1
            for b in block:
                if b[0] == "F":
                    c = int(b[1])
                    assert seen[c] == nk[c] and int(b[2]) == iters[c]
                    seen[c], iters[c], event_ids[c] = 0, iters[c] + 1, 0
    assert at == len(dec)
    return checked


def check_reef_rule(obs_text, dec_text):
    """The REEF rule, poll by poll (reference: schedule_reef,
    scheduler_eval.cpp:93-165): which clients a poll dispatches is a function of
    the heads it saw, the iteration counts, the profile rows at seen[] and the
    penalty counter."""
    obs, dec = obs_text.splitlines(), dec_text.splitlines()
    at = 0
    n = None
    nk, max_iters, prof, seen, iters = {}, {}, {}, {}, {}
    penalty = 0                               # a member of the scheduler: never reset
    kinds = {"first": 0, "paired": 0, "unpaired": 0, "released": 0, "held": 0}
    for line in obs:
        p = line.split(" ")
        if p[0] == "J":
            n = int(p[1])
            hp = n - 1
        elif p[0] == "K":
            c = int(p[1])
            nk[c], max_iters[c], prof[c] = int(p[2]), int(p[3]), rows_of(p[5])
            seen[c], iters[c] = 0, 0
        elif p[0] == "X":
            c = int(p[1])
            nk[c], prof[c] = int(p[2]), rows_of(p[3])
            assert dec[at] == f"X {c}"
            at += 1
        elif p[0] == "S":
            assert dec[at] == "S" and p[3] == "reef"
            at += 1
            depth = int(p[4])
        elif p[0] == "E":
            assert dec[at] == "E"
            at += 1
        elif p[0] == "P":
            assert dec[at] == "P"
            at += 1
            heads = p[2]
            block = []
            while at < len(dec) and dec[at][0] in "DFT":
                block.append(dec[at].split(" "))
                at += 1
            got = [int(b[1]) for b in block if b[0] == "D"]
            present = [c for c in range(n) if heads[c] in RECORD]
            for c in range(n):
                if seen[c] == nk[c]:
                    assert heads[c] == "-"
            if n == 1:
                want = present
            else:
                first = [c for c in present
                         if heads[c] == "m" or iters[c] <= 10 or iters[hp] >= max_iters[hp]]
                if first:                                         # :108-116
                    want = first[:1]
                    kinds["first"] += 1
                elif hp in present:                               # :119-141
                    hp_row = prof[hp][seen[hp]]
                    fits = [c for c in present if c != hp
                            and prof[c][seen[c]][2] <= hp_row[2]
                            and prof[c][seen[c]][1] >= hp_row[1]]
                    want = [hp] + fits[:1]
                    kinds["paired" if fits else "unpaired"] += 1
                else:                                             # :143-163
                    penalty += len(present)
                    if penalty >= depth:
                        want, penalty = present, 0
                        kinds["released"] += bool(present)
                    else:
                        want = []
                        kinds["held"] += bool(present)
            assert got == want, (line, block, want)
            for b in block:
                c = int(b[1])
                if b[0] == "D" and b[3] == "k":
                    seen[c] += 1
                elif b[0] == "F":
                    assert seen[c] == nk[c]
                    seen[c], iters[c] = 0, iters[c] + 1
    assert at == len(dec)
    return kinds


@settings(max_examples=100, deadline=None,
          suppress_health_check=[HealthCheck.function_scoped_fixture, HealthCheck.too_slow])
@given(seed=st.integers(0, 10_000), n_clients=st.integers(1, 5), hp_iters=st.integers(11, 30))
def test_reef_rule_on_the_native_core(tmp_path_factory, seed, n_clients, hp_iters):
    tmp = str(tmp_path_factory.mktemp("job"))
    job = jobs.make_job(tmp, seed, n_clients=n_clients, algo=po.ALGO_REEF, hp_train=False,
                        hp_iters=hp_iters)
    _, _, rec = jobs.run_oracle(job)
    obs = rec.obs_text()
    marked = jobs.native_replay(obs, by_poll=True)
    assert "".join(l + "\n" for l in marked.splitlines() if l != "P") == rec.dec.text()
    check_reef_rule(obs, marked)


def test_reef_rule_fires_every_branch(tmp_path):
    seen = {}
    for seed in range(6):
        job = jobs.make_job(str(tmp_path), seed, n_clients=3, algo=po.ALGO_REEF, hp_iters=25)
        _, _, rec = jobs.run_oracle(job)
        for k, v in check_reef_rule(rec.obs_text(),
                                    jobs.native_replay(rec.obs_text(), by_poll=True)).items():
            seen[k] = seen.get(k, 0) + v
    assert all(v > 0 for v in seen.values()), seen
    d = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fake_reef_2be")
    obs = open(os.path.join(d, "observations.log")).read().replace("@DIR@", d)
    check_reef_rule(obs, jobs.native_replay(obs, by_poll=True))


def check_time_slicing(obs_text, dec_text):
    """Time slicing with the repaired rule: everything runs on client 0's stream
    set (schedule_sequential, scheduler_eval.cpp:199-201, :225-227), and past the
    tenth iteration a client's record -- other than an allocation -- goes out only
    while no other client is in the middle of an iteration (the stated intent of
    :189-196 and :213-221)."""
    n = int(obs_text.split(" ", 2)[1])
    seen, iters = [0] * n, [0] * n
    exclusive = 0
    for line in dec_text.splitlines():
        p = line.split(" ")
        if p[0] == "D":
            c = int(p[1])
            assert p[2] == "0", line
            if n > 1 and iters[c] > 10 and p[3] != "m":
                assert all(seen[j] == 0 for j in range(n) if j != c), (line, seen)
                exclusive += 1
            if p[3] == "k":
                seen[c] += 1
        elif p[0] == "F":
            c = int(p[1])
            seen[c], iters[c] = 0, iters[c] + 1
    return exclusive


@settings(max_examples=60, deadline=None,
          suppress_health_check=[HealthCheck.function_scoped_fixture, HealthCheck.too_slow])
@given(seed=st.integers(0, 10_000), n_clients=st.integers(1, 4), hp_iters=st.integers(12, 30))
def test_time_slicing_never_overlaps_iterations(tmp_path_factory, seed, n_clients, hp_iters):
    tmp = str(tmp_path_factory.mktemp("job"))
    job = jobs.make_job(tmp, seed, n_clients=n_clients, algo=po.ALGO_SEQUENTIAL, hp_train=False,
                        hp_iters=hp_iters)
    _, _, rec = jobs.run_oracle(job)
    dec = jobs.native_replay(rec.obs_text())
    assert dec == rec.dec.text()
    assert check_time_slicing(rec.obs_text(), dec) > 0 or n_clients == 1


@settings(max_examples=150, deadline=None,
          suppress_health_check=[HealthCheck.function_scoped_fixture, HealthCheck.too_slow])
@given(seed=st.integers(0, 10_000), n_clients=st.integers(1, 5),
       depth=st.sampled_from([1, 20_000, 150_000, 600_000, 5_000_000]),
       hp_iters=st.integers(11, 30))
def test_orion_invariants_on_the_native_core(tmp_path_factory, seed, n_clients, depth, hp_iters):
    tmp = str(tmp_path_factory.mktemp("job"))
    job = jobs.make_job(tmp, seed, n_clients=n_clients, algo=po.ALGO_ORION, hp_train=False,
                        hp_iters=hp_iters, depth=depth)
    _, _, rec = jobs.run_oracle(job)
    obs = rec.obs_text()
    marked = jobs.native_replay(obs, by_poll=True)
    assert "".join(l + "\n" for l in marked.splitlines() if l != "P") == rec.dec.text()
    check_orion_invariants(obs, marked, depth)


@pytest.mark.parametrize("case", ["fake_orion_2be", "mi355x_kernel_pair"])
def test_orion_invariants_on_recordings_of_the_live_scheduler(case):
    """The same checks on committed recordings of the live native scheduler
    (the recording HIP stand-in, and the kernel pair on an MI355X)."""
    d = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", case)
    obs = open(os.path.join(d, "observations.log")).read().replace("@DIR@", d)
    assert " orion " in obs
    depth = int(next(l for l in obs.splitlines() if l.startswith("S ")).split(" ")[4])
    counts = check_orion_invariants(obs, jobs.native_replay(obs, by_poll=True), depth)
    assert counts["rotation"] > 0


def test_the_checks_bite(tmp_path):
    """The invariants are not vacuous: every kind fires on an ordinary job, and a
    log with one best-effort dispatch moved to the neighbouring poll fails."""
    counts = {}
    for seed in range(11, 17):
        job = jobs.make_job(str(tmp_path), seed, n_clients=3, hp_iters=25, depth=150_000)
        _, _, rec = jobs.run_oracle(job)
        obs = rec.obs_text()
        marked = jobs.native_replay(obs, by_poll=True)
        for k, v in check_orion_invariants(obs, marked, 150_000).items():
            counts[k] = counts.get(k, 0) + v
    assert all(v > 0 for v in counts.values()), counts
    lines = marked.splitlines()
    # move the first high-priority dispatch one poll later
    i = next(k for k, l in enumerate(lines) if l.startswith("D 2 "))
    j = next(k for k in range(i + 1, len(lines)) if lines[k] == "P")
    moved = lines[:i] + lines[i + 1:j + 1] + [lines[i]] + lines[j + 1:]
    try:
        check_orion_invariants(obs, "\n".join(moved) + "\n", 150_000)
    except AssertionError:
        return
    raise AssertionError("a displaced high-priority dispatch went unnoticed")
