"""The admission option O1 (ORION_ADMIT_OVERSIZED=1), hand-worked.

Not in the reference.  Its CU clause, ``size + op.sm_used <= max_sms``
(src/scheduler/scheduler_eval.cpp:339-340), takes the profiled CU need as it
comes -- un-clipped, so a kernel whose grid alone exceeds the device can never
be admitted while a high-priority inference request is in flight, and the
client stands behind it.  With the option such a kernel is let in when it is
the first best-effort kernel admitted in the poll (``size == 0``), its class
and the class of the high-priority op last dispatched are both known and
differ, and its profiled duration is at most a quarter of the duration budget;
it is placed on the smallest CU mask, and its full need closes the poll's
budget for every other client.

The expected decisions below were worked out by hand from that statement and
from the reference's loop (:277-400); the trace runs through the CPU oracle and
through the native core.  A second trace shows the same poll without the
option: the reference's rule, nothing admitted.
"""

import numpy as np

from oracle import obslog, policy_oracle as po
from tests import jobs


def op(profile, sm, dur):
    return po.OpInfo("x", profile, 0, sm, np.float32(dur))


BE0 = [op(0, 200, 2000), op(0, 200, 30000), op(1, 10, 1000)]
BE1 = [op(0, 300, 2000), op(-1, 300, 1000)]
HP = [op(1, 20, 1000), op(0, 20, 1000), op(-1, 20, 1000)]
N, NK = 3, [3, 2, 3]
MAX_SMS, MASKS = 80, "16,32,80"
BUDGET = 40000            # a quarter of it: 10000 ns


def heads_only(client):
    return "".join("k" if c == client else "." for c in range(N))


def header(tmp_path, option):
    lines = [f"J {N} {MAX_SMS} {MASKS}" + (" O1" if option else "")]
    for c, ops in enumerate((BE0, BE1, HP)):
        path = str(tmp_path / f"c{c}.csv")
        jobs.write_profile(path, ops)
        lines.append(f"K {c} {len(ops)} 1000 {int(c < N - 1)} {path}")
    return lines


def warmup():
    """Eleven iterations of every client, one client visible per poll, under a
    budget that is never reached.  A best-effort record goes out at once while
    the high-priority client is between two requests (``seen[hp] == 0``, :333),
    on the whole-GPU stream (slot 2 of 16,32,80); a high-priority record goes
    out in the poll that sees it (:311-321); the last kernel of an iteration
    completes in the poll that dispatched it (:380-420)."""
    obs, dec = ["S 1 11 orion 100000000 1 1"], ["S"]
    for it in range(11):
        for c in range(N):
            for k in range(NK[c]):
                last = k == NK[c] - 1
                obs.append(f"P 0 {heads_only(c)} {'1' if last else '-'} -")
                dec.append(f"D {c} {c} k {k} {k} {0 if c == N - 1 else 2}")
                if last:
                    dec.append(f"F {c} {it}")
    return obs + ["E"], dec + ["E"]


def replay_both(obs_lines, want_lines):
    obs = "\n".join(obs_lines) + "\n"
    want = "\n".join(want_lines) + "\n"
    for name, got in (("oracle", obslog.replay(obs)), ("native", jobs.native_replay(obs))):
        g, w = got.splitlines(), want.splitlines()
        for i, (a, b) in enumerate(zip(g, w)):
            assert a == b, f"{name}, line {i}: got {a!r}, hand-worked {b!r}"
        assert len(g) == len(w), (name, len(g), len(w))


def test_oversized_kernels_of_the_other_class_go_in_alone_on_the_smallest_mask(tmp_path):
    obs, dec = warmup()
    obs = header(tmp_path, option=True) + obs
    # every client is past its tenth iteration; a new schedule() call starts with
    # start = -1, sum = 0, no throttle, profiles[hp] = -1
    obs.append(f"S 0 0 orion {BUDGET} 1 1")
    dec.append("S")
    steps = [
        # 1. HP op 0 (compute-bound) goes out.  BE0 op 0: memory-bound, need 200
        #    of 80, 2000 ns <= 10000: nothing admitted yet in this poll -> let in,
        #    smallest mask (slot 0).  BE1 op 0 qualifies too, but size is 200 now.
        ("P 0 kkk - -", ["D 2 2 k 0 0 0", "D 0 0 k 0 0 0"]),
        # 2. no new HP record; the running HP op is still the compute-bound one.
        #    Rotation resumes after BE0: BE1 first (:323-326).  BE1 op 0 goes in
        #    alone; BE0 op 1 finds size = 300 (and lasts 30000 ns anyway).
        ("P 0 kk. - -", ["D 1 1 k 0 0 0"]),
        # 3. HP op 1 is memory-bound.  BE0 op 1: same class (and too long);
        #    BE1 op 1: class unknown.  Neither goes.
        ("P 0 kkk - -", ["D 2 2 k 1 1 0"]),
        # 4. HP op 2 has no known class: nothing oversized beside it.  It is the
        #    request's last kernel: its event is asked about (:380-395), not done.
        ("P 0 kkk 0 -", ["D 2 2 k 2 2 0"]),
        # 5. the request completes (HP is not peeked: seen == num_kernels)
        ("P 0 kk- 1 -", ["F 2 11"]),
        # 6. HP idle: the reference's first clause (:333) admits both, on the
        #    whole-GPU stream (slot 2).  Rotation: after BE1 comes BE0.  The sum of
        #    durations is 2000 + 2000 + 30000 + 1000 = 35000 <= 40000: no throttle.
        #    BE1 has dispatched both its kernels: its event is asked about.
        ("P 0 kk. 0 -", ["D 0 0 k 1 1 2", "D 1 1 k 1 1 2"]),
        # 7. every client acknowledges a stop (:383-388): BE0's last kernel still
        #    goes out first (small, HP idle); BE1 is not peeked (its iteration is
        #    fully dispatched); an acknowledged client's events are not asked about.
        ("P 7 k-. - -", ["D 0 0 k 2 2 2"]),
    ]
    for p, d in steps:
        obs.append(p)
        dec += d
    replay_both(obs + ["E"], dec + ["E"])


def test_without_the_option_the_oversized_kernel_waits(tmp_path):
    """The same first poll under the reference's rule alone (:339-340): 200 of
    80 CUs does not fit, nothing best-effort goes out beside the request."""
    obs, dec = warmup()
    obs = header(tmp_path, option=False) + obs
    obs.append(f"S 0 0 orion {BUDGET} 1 1")
    dec.append("S")
    obs.append("P 0 kkk - -")
    dec.append("D 2 2 k 0 0 0")
    # the request runs to its end with both best-effort clients waiting
    obs += ["P 0 kkk - -", "P 0 kkk 1 -"]
    dec += ["D 2 2 k 1 1 0", "D 2 2 k 2 2 0", "F 2 11"]
    # idle again: both go, whole GPU, BE0 first (start is still -1)
    obs.append("P 0 kk. - -")
    dec += ["D 0 0 k 0 0 2", "D 1 1 k 0 0 2"]
    obs.append("P 7 kk. - -")            # stops acknowledged; idle, so both go on
    dec += ["D 0 0 k 1 1 2", "D 1 1 k 1 1 2"]
    replay_both(obs + ["E"], dec + ["E"])
