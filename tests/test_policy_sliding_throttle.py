"""The throttle option T1 (ORION_SLIDING_THROTTLE=1), hand-worked.

Not in the reference.  Its duration throttle (src/scheduler/scheduler_eval.cpp
:342-359, :363-368) stops best-effort admission once the sum of the admitted
kernels' profiled durations exceeds the budget, and lets go only when the last
kernel of EVERY best-effort client has completed: the sum then restarts at zero.
With the option, the policy also takes a mark when the sum first passes half the
budget -- the latest kernel of every best-effort client, and the sum so far --
and, while throttled, asks about the marks after the reference's own question;
when they have completed, the marked part of the sum is taken off and admission
goes on.  The outstanding work stays within the budget, as in the reference, but
the best-effort streams no longer have to run empty first.

The expected decisions and event questions below were worked out by hand from
that statement and the reference's loop; the trace runs through the CPU oracle
and through the native core, and a second trace shows the reference's rule on
the same kernels.
"""

import numpy as np

from oracle import obslog, policy_oracle as po
from tests import jobs


def op(dur):
    return po.OpInfo("x", -1, 0, 10, np.float32(dur))


BE = [op(3000)] * 6
HP = [op(1000)]
N, NK = 2, [6, 1]
BUDGET = 10000            # half of it: 5000 ns


def header(tmp_path, option):
    lines = [f"J {N} 80 80" + (" T1" if option else "")]
    for c, ops in enumerate((BE, HP)):
        path = str(tmp_path / f"c{c}.csv")
        jobs.write_profile(path, ops)
        lines.append(f"K {c} {len(ops)} 1000 {int(c < N - 1)} {path}")
    return lines


def warmup():
    """Eleven iterations of both clients, one record per poll, under a budget
    that is never reached; the last kernel of an iteration completes in the poll
    that dispatched it (:380-420)."""
    obs, dec = ["S 1 11 orion 100000000 1 1"], ["S"]
    for it in range(11):
        for c in range(N):
            for k in range(NK[c]):
                last = k == NK[c] - 1
                heads = "".join("k" if x == c else "." for x in range(N))
                obs.append(f"P 0 {heads} {'1' if last else '-'} -")
                dec.append(f"D {c} {c} k {k} {k} 0")
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


def test_the_throttle_lets_go_at_the_half_way_mark(tmp_path):
    obs, dec = warmup()
    obs = header(tmp_path, option=True) + obs
    # a new schedule() call: sum = 0, not throttled, no mark.  The high-priority
    # client stays idle, so every best-effort kernel is admissible (:333) and only
    # the duration throttle decides.  Kernels last 3000 ns by profile.
    obs.append(f"S 0 0 orion {BUDGET} 1 1")
    dec.append("S")
    steps = [
        ("P 0 k. - -", ["D 0 0 k 0 0 0"]),    # sum 3000
        ("P 0 k. - -", ["D 0 0 k 1 1 0"]),    # sum 6000 > 5000: mark = kernel 1, 6000
        ("P 0 k. - -", ["D 0 0 k 2 2 0"]),    # sum 9000
        ("P 0 k. - -", ["D 0 0 k 3 3 0"]),    # sum 12000 > 10000: throttled from now on
        # kernel 4 waits.  The reference's question first: has the client's latest
        # kernel (3) completed?  No.  Then the mark: has kernel 1?  Yes: 6000 comes
        # off the sum (6000 left), the throttle is off, kernel 4 goes (9000), and
        # since no mark is standing and 9000 > 5000 a new one is taken: kernel 4, 9000
        ("P 0 k. 01 -", ["D 0 0 k 4 4 0"]),
        # kernel 5: 12000 > 10000, throttled again.  It is the iteration's last
        # kernel: the completion check asks about it (:389-395): not done
        ("P 0 k. 0 -", ["D 0 0 k 5 5 0"]),
        ("P 0 -. 1 -", ["F 0 11"]),           # done: the iteration is released
        # next iteration, still throttled (sum 12000).  The reference's question
        # finds no kernel of this iteration outstanding (:344-351 skips a client
        # with no event yet): everything has drained, the sum restarts at 0
        ("P 0 k. - -", ["D 0 0 k 0 0 0"]),    # sum 3000
        ("P 3 k. - -", ["D 0 0 k 1 1 0"]),    # both clients acknowledge a stop
    ]
    for p, d in steps:
        obs.append(p)
        dec += d
    replay_both(obs + ["E"], dec + ["E"])


def test_without_the_option_the_streams_must_drain(tmp_path):
    """The reference's rule on the same kernels: once throttled, kernel 4 goes
    only after the client's latest kernel (3) has completed, and the sum restarts
    at zero -- so kernels 4 and 5 (6000) do not throttle again."""
    obs, dec = warmup()
    obs = header(tmp_path, option=False) + obs
    obs.append(f"S 0 0 orion {BUDGET} 1 1")
    dec.append("S")
    steps = [
        ("P 0 k. - -", ["D 0 0 k 0 0 0"]),
        ("P 0 k. - -", ["D 0 0 k 1 1 0"]),
        ("P 0 k. - -", ["D 0 0 k 2 2 0"]),
        ("P 0 k. - -", ["D 0 0 k 3 3 0"]),    # sum 12000: throttled
        ("P 0 k. 1 -", ["D 0 0 k 4 4 0"]),    # kernel 3 done: sum 0 -> 3000
        ("P 0 k. 1 -", ["D 0 0 k 5 5 0", "F 0 11"]),   # sum 6000; last kernel done at once
        ("P 3 k. - -", ["D 0 0 k 0 0 0"]),
    ]
    for p, d in steps:
        obs.append(p)
        dec += d
    replay_both(obs + ["E"], dec + ["E"])
