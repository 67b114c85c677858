"""Observation and decision logs of a policy run, and their replay.

TEST INFRASTRUCTURE ONLY (see ``oracle/policy_oracle.py``).

The policy is a pure function of what it observes.  A run is therefore fixed by
(1) the job description -- profile files, kernel counts, iteration limits,
flags -- and (2) the observations every *effective* poll consumed, in order: the
stop acknowledgements, the queue heads it peeked, the answers of the event
queries it made, and the iteration wall times it read.  Polls that changed no
state are elided: replaying them or not yields the same decisions
(reference: src/scheduler/scheduler_eval.cpp:277-302 -- per-poll state `size`
and `frecords` is rebuilt on every iteration of the loop).

Both logs are line-based text, shared with the native core
(orion_amd/csrc/policy/obslog.h):

observation log
    ``J <n> <max_sms> <place_masks comma list> [L1] [R1] [O1] [T1]``  job header (L1: long
                                                    best-effort kernels confined; R1:
                                                    the high-priority op's CU need
                                                    is reserved; O1: short kernels of
                                                    the other class whose CU need
                                                    exceeds the device go in alone,
                                                    on the smallest mask; T1: the
                                                    duration throttle lets go at its
                                                    half-way mark)
    ``K <client> <num_kernels> <num_iters> <train 0|1> <profile path>``
    ``X <client> <num_kernels> <profile path>``      setup_change
    ``S <warmup 0|1> <warmup_iters> <algo> <depth> <hp_limit> <update_start>``
    ``P <acks hex> <heads> <events|-> <us comma list|->``  one effective poll
    ``E``                                            schedule() returned
  heads: one character per client -- ``-`` not peeked, ``.`` empty queue, else
  the record class (k kernel, c memcpy, m malloc, f free, s memset).
  events: the answers (0/1) of the event queries in the order they were asked.

decision log
    ``S`` / ``E`` / ``X <client>`` mirror the observation log's structure
    ``D <client> <owner> <class> <op_index> <event_slot> <cu_slot>``  a dispatch
    ``F <client> <iteration>``                      iteration released
    ``T <client>``                                  stop raised for a client
"""

import numpy as np

from oracle import policy_oracle as po


class DecisionLog:
    def __init__(self):
        self.lines = []

    def add(self, line):
        self.lines.append(line)

    def text(self):
        return "\n".join(self.lines) + ("\n" if self.lines else "")


def place_cu_slot(masks, cls, sm_used, algo, hp_active, long_kernel=False):
    """CU-mask placement of a best-effort dispatch (no reference counterpart:
    the reference has one stream per client).  ``masks`` is the ascending list
    of mask sizes a best-effort client owns; the last entry is the whole GPU.
    High-priority client idle: the whole GPU, unless the kernel alone outlasts
    the best-effort duration budget (``long_kernel``) -- a request arriving
    behind it cannot be protected in time, so it is confined to the largest
    partial mask and leaves the other CUs free.  Request in flight: the
    smallest mask that holds the kernel's profiled CU need, never the whole
    GPU when a partial mask exists.  Records that are not kernels stay where
    the client's previous op ran (-1)."""
    if cls != po.KERNEL:
        return -1
    last = len(masks) - 1
    if algo != po.ALGO_ORION or last == 0:
        return last
    if not hp_active:
        return last - 1 if long_kernel else last
    for slot in range(last):
        if sm_used <= masks[slot]:
            return slot
    return last - 1


class RecordingEnv(po.Env):
    """Wraps another Env; writes both logs while the oracle drives it."""

    def __init__(self, inner, n, masks, ops_of, algo=po.ALGO_ORION,
                 hp_active=None):
        self.hp_active = hp_active    # callable() -> bool: seen[hp] > 0
        self.inner = inner
        self.n = n
        self.masks = list(masks)
        self.ops_of = ops_of          # callable(client, op_index) -> OpInfo
        self.algo = algo
        self.budget = None            # Orion's best-effort duration budget (ns)
        self.confine_long = False     # placement option, header token L1
        self.mark_polls = False       # a "P" line before every poll's decisions
        self.obs = []
        self.dec = DecisionLog()
        self._reset_poll()

    def _reset_poll(self):
        self._acks = None
        self._heads = ["-"] * self.n
        self._events = []
        self._us = []
        self._dec = []

    # structure markers -------------------------------------------------
    def header(self, max_sms, clients, confine_long=False, reserve_hp=False,
               admit_oversized=False, sliding_throttle=False):
        self.confine_long = bool(confine_long)
        self.obs.append(f"J {self.n} {max_sms} " + ",".join(map(str, self.masks))
                        + (" L1" if confine_long else "") + (" R1" if reserve_hp else "")
                        + (" O1" if admit_oversized else "")
                        + (" T1" if sliding_throttle else ""))
        for i, (nk, ni, train, path) in enumerate(clients):
            self.obs.append(f"K {i} {nk} {ni} {int(bool(train))} {path}")

    def setup_change(self, client, num_kernels, path):
        self.obs.append(f"X {client} {num_kernels} {path}")
        self.dec.add(f"X {client}")

    def begin_schedule(self, warmup, warmup_iters, algo, depth, hp_limit,
                       update_start):
        self.algo = algo
        self.obs.append(f"S {int(bool(warmup))} {warmup_iters} {algo} {depth} "
                        f"{hp_limit} {update_start}")
        self.dec.add("S")

    def end_schedule(self):
        self.obs.append("E")
        self.dec.add("E")

    # Env ----------------------------------------------------------------
    def begin_poll(self):
        self.inner.begin_poll()
        self._reset_poll()
        self._acks = [self.inner.stop_ack(i) for i in range(self.n)]

    def end_poll(self, changed):
        if changed:
            acks = sum(1 << i for i, a in enumerate(self._acks) if a)
            ev = "".join("1" if e else "0" for e in self._events) or "-"
            us = ",".join(str(u) for u in self._us) or "-"
            self.obs.append(f"P {acks:x} {''.join(self._heads)} {ev} {us}")
            if self.mark_polls:
                self.dec.add("P")
            for line in self._dec:
                self.dec.add(line)
        else:
            assert not self._dec
        self.inner.end_poll(changed)

    def stop_ack(self, client):
        return self._acks[client]

    def peek(self, client):
        cls = self.inner.peek(client)
        self._heads[client] = "." if cls is None else cls
        return cls

    def event_done(self, owner, index):
        done = bool(self.inner.event_done(owner, index))
        self._events.append(done)
        return done

    def iteration_us(self, client):
        us = int(self.inner.iteration_us(client))
        self._us.append(us)
        return us

    def dispatch(self, client, owner, cls, op_index, event_slot, smallest_mask=False):
        if cls != po.KERNEL:
            cu_slot = -1
        elif owner == self.n - 1:      # the high-priority stream is unmasked
            cu_slot = 0
        elif smallest_mask:            # an oversized kernel let in alone (O1)
            cu_slot = 0
        else:
            op = self.ops_of(client, op_index)
            cu_slot = place_cu_slot(
                self.masks, cls, op.sm_used, self.algo, self.hp_active(),
                self.confine_long and self.budget is not None
                and float(op.duration) > float(np.float32(self.budget)))
        self._dec.append(f"D {client} {owner} {cls} {op_index} {event_slot} "
                         f"{cu_slot}")
        self.inner.dispatch(client, owner, cls, op_index, event_slot)

    def mark(self, owner, index):
        if hasattr(self.inner, "mark"):
            self.inner.mark(owner, index)

    def iteration_done(self, client, iteration):
        self._dec.append(f"F {client} {iteration}")
        self.inner.iteration_done(client, iteration)

    def set_stop(self, client):
        self._dec.append(f"T {client}")
        self.inner.set_stop(client)

    def obs_text(self):
        return "\n".join(self.obs) + "\n"


class ReplayDivergence(RuntimeError):
    pass


class ReplayEnv(po.Env):
    """Feeds the observations of one ``S``..``E`` segment back to the oracle."""

    def __init__(self, n, polls):
        self.n = n
        self.polls = polls
        self.at = -1

    def begin_poll(self):
        self.at += 1
        if self.at >= len(self.polls):
            raise ReplayDivergence("oracle wants more polls than were logged")
        acks, heads, events, us = self.polls[self.at]
        self._acks, self._heads = acks, heads
        self._events, self._us = list(events), list(us)

    def end_poll(self, changed):
        if self._events or self._us:
            raise ReplayDivergence(
                f"poll {self.at}: logged observations left unread")
        if not changed:
            raise ReplayDivergence(f"poll {self.at}: logged poll changed nothing")


    def stop_ack(self, client):
        return bool((self._acks >> client) & 1)

    def peek(self, client):
        ch = self._heads[client]
        if ch == "-":
            raise ReplayDivergence(
                f"poll {self.at}: client {client} peeked but log says it was not")
        return None if ch == "." else ch

    def event_done(self, owner, index):
        if not self._events:
            raise ReplayDivergence(f"poll {self.at}: unlogged event query")
        return self._events.pop(0)

    def iteration_us(self, client):
        if not self._us:
            raise ReplayDivergence(f"poll {self.at}: unlogged time read")
        return self._us.pop(0)

    def dispatch(self, *a, **kw):
        pass

    def iteration_done(self, *a):
        pass

    def set_stop(self, *a):
        pass


def replay(obs_text, load_profile=po.parse_profile, sequential_fix=True, mark_polls=False):
    """Run the oracle over an observation log; return its decision log text
    (with ``mark_polls``, a line ``P`` precedes every logged poll's decisions)."""
    oracle = None
    rec = None
    n = max_sms = masks = None
    confine_long = reserve_hp = admit_oversized = sliding_throttle = False
    clients = {}
    lines = obs_text.splitlines()
    i = 0
    while i < len(lines):
        parts = lines[i].split(" ")
        tag = parts[0]
        if tag == "J":
            n, max_sms = int(parts[1]), int(parts[2])
            masks = [int(x) for x in parts[3].split(",")]
            _ensure(set(parts[4:]) <= {"L1", "R1", "O1", "T1"} and len(parts) <= 8,
                    "J: 3 fields and optional L1 / R1 / O1 / T1")
            confine_long, reserve_hp = "L1" in parts[4:], "R1" in parts[4:]
            admit_oversized = "O1" in parts[4:]
            sliding_throttle = "T1" in parts[4:]
        elif tag == "K":
            clients[int(parts[1])] = (int(parts[2]), int(parts[3]),
                                      bool(int(parts[4])), " ".join(parts[5:]))
        elif tag == "X":
            _ensure(oracle is not None, "X before S")
            c = int(parts[1])
            oracle.setup_change(c, load_profile(" ".join(parts[3:])),
                                int(parts[2]))
            rec.dec.add(f"X {c}")
        elif tag == "S":
            if oracle is None:
                order = [clients[c] for c in range(n)]
                oracle = po.PolicyOracle(
                    [load_profile(c[3]) for c in order], [c[0] for c in order],
                    [c[1] for c in order], [c[2] for c in order], max_sms,
                    sequential_fix=sequential_fix, reserve_hp=reserve_hp,
                    admit_oversized=admit_oversized, sliding_throttle=sliding_throttle)
            polls = []
            i += 1
            while lines[i] != "E":
                p = lines[i].split(" ")
                _ensure(p[0] == "P", f"line {i}: expected P")
                events = [] if p[3] == "-" else [ch == "1" for ch in p[3]]
                us = [] if p[4] == "-" else [int(x) for x in p[4].split(",")]
                polls.append((int(p[1], 16), p[2], events, us))
                i += 1
            env = ReplayEnv(n, polls)
            if rec is None:
                rec = RecordingEnv(env, n, masks,
                                   lambda c, k: oracle.ops[c][k],
                                   hp_active=lambda: oracle.seen[n - 1] > 0)
            rec.inner = env
            rec.mark_polls = mark_polls
            warmup, witers, algo = bool(int(parts[1])), int(parts[2]), parts[3]
            depth, hp_limit, ustart = int(parts[4]), int(parts[5]), int(parts[6])
            rec.algo = algo
            rec.budget = depth
            rec.confine_long = confine_long
            rec.dec.add("S")
            oracle.schedule(rec, warmup, witers, algo, depth, hp_limit, ustart,
                            max_polls=len(polls) + 1)
            _ensure(env.at == len(polls) - 1,
                    "oracle finished before the logged polls ran out")
            rec.dec.add("E")
        i += 1
    return rec.dec.text() if rec else ""


def _ensure(cond, msg):
    if not cond:
        raise ReplayDivergence(msg)
