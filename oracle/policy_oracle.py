"""CPU oracle: the reference scheduler's dispatch policy, restated in Python.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this file;
it is the checker that ``tests/``, ``__graft_entry__.smoke()`` and
``bench.py``'s ``cpu_baseline`` leg hold the native policy core against.

It follows the reference scheduler statement by statement; every method cites
the lines of ``src/scheduler/scheduler_eval.cpp`` (reference tree) it restates:

* profile CSV parser ........ ``populate_kernel_info``      :498-526
* per-client setup .......... ``setup`` / ``setup_change``   :528-540, :591-601
* dispatch bookkeeping ...... ``schedule_kernel``            utils_sched.cpp:239-522
* Orion policy .............. ``busy_wait_profile``          :238-487
* REEF policy ............... ``schedule_reef``              :93-165
* time-slicing policy ....... ``schedule_sequential``        :167-236

The oracle is *pure*: everything it observes of the outside world (queue heads,
event completion, stop acknowledgements, wall-clock iteration times) arrives
through an ``Env`` object, and everything it decides leaves through the same
object.  That makes a run replayable from a log of observations.

How each part is pinned (the reference ships no tests and cannot be compiled in
this image: it needs CUDA, cuDNN and cuBLAS headers that are absent):

* parser: the reference's own 19 profile files (row counts named in its JSON
  configs, per-file maxima and duration sums) -- tests/test_profile_csv.py
* Orion admission / throttle / round-robin / completion: invariants that the
  reference text fixes, checked by brute force over small random runs, and
  hand-worked traces -- tests/test_policy_oracle.py
* fp32 ``sum`` accumulation: closed form against numpy.float32
* threshold bisection: closed form (bisection on [0, max_sms_clients[0]])
* REEF and sequential: hand-worked traces and the invariants their text fixes
  (REEF pairs a best-effort op only with duration <= and CU need >= the
  high-priority op's; sequential never runs two clients' iterations at once
  after warm-up).  No reference-produced vector exists for them: beyond those
  checks their parity is UNPINNED.
"""

from dataclasses import dataclass
import re

import numpy as np

# Record classes as the policy distinguishes them (reference: enum func_type,
# src/cuda_capture/intercept_temp.h:642-660).  Every library-op record type of
# the reference behaves like KERNEL for the policy, so one class covers them.
KERNEL = "k"
MEMCPY = "c"
MALLOC = "m"
FREE = "f"
MEMSET = "s"
MEM_CLASSES = (MALLOC, MEMCPY, MEMSET, FREE)
ALL_CLASSES = (KERNEL, MEMCPY, MALLOC, FREE, MEMSET)

INT_MAX = 2**31 - 1

ALGO_ORION = "orion"
ALGO_REEF = "reef"
ALGO_SEQUENTIAL = "sequential"


@dataclass
class OpInfo:
    """One profile row (reference: struct op_info, utils_sched.h:90-98)."""
    name: str
    profile: int      # 1 compute-bound, 0 memory-bound, -1 unknown
    mem: int
    sm_used: int
    duration: np.float32  # nanoseconds, held in fp32 like the reference


_STOI = re.compile(r"^[ \t\n\v\f\r]*([+-]?[0-9]+)")
_STOF = re.compile(
    r"^[ \t\n\v\f\r]*([+-]?(?:[0-9]+\.?[0-9]*(?:[eE][+-]?[0-9]+)?"
    r"|\.[0-9]+(?:[eE][+-]?[0-9]+)?|inf(?:inity)?|nan))", re.IGNORECASE)


def c_stoi(text):
    """std::stoi: leading whitespace, optional sign, decimal digits; the rest
    of the field is ignored (scheduler_eval.cpp:520)."""
    m = _STOI.match(text)
    if not m:
        raise ValueError(f"stoi: no conversion in {text!r}")
    value = int(m.group(1))
    if not -2**31 <= value <= INT_MAX:
        raise OverflowError(f"stoi: out of range {text!r}")
    return value


def c_stof(text):
    """std::stof: longest valid floating prefix, rounded to fp32."""
    m = _STOF.match(text)
    if not m:
        raise ValueError(f"stof: no conversion in {text!r}")
    return np.float32(float(m.group(1)))


def parse_profile(path):
    """populate_kernel_info (scheduler_eval.cpp:498-526): skip the header line,
    split every further line on ',', fields 1..4 through stoi/stoi/stoi/stof."""
    ops = []
    with open(path, "r", newline="") as f:
        text = f.read()
    lines = text.split("\n")
    if lines and lines[-1] == "":
        lines.pop()          # getline yields no empty record after a final \n
    for line in lines[1:]:   # :507 header ignored
        v = line.split(",")  # :514-518
        ops.append(OpInfo(v[0], c_stoi(v[1]), c_stoi(v[2]), c_stoi(v[3]),
                          c_stof(v[4])))   # :520
    return ops


def max_sm_used(ops):
    """setup :595-598 / setup_change :534-537 (starts from 0)."""
    best = 0
    for op in ops:
        best = max(best, op.sm_used)
    return best


class Env:
    """What the policy sees and does.  Subclasses: the virtual-time model in
    ``oracle/virtual_gpu.py`` and the log replayer in ``oracle/obslog.py``."""

    def begin_poll(self):
        """Called at the top of every poll-loop iteration."""

    def end_poll(self, changed):
        """Called at the bottom; ``changed`` says whether any state moved."""

    def stop_ack(self, client):            # client_stop_ack[i]
        raise NotImplementedError

    def peek(self, client):                # queue head class or None
        raise NotImplementedError

    def event_done(self, owner, index):    # cudaEventQuery(...) == success
        raise NotImplementedError

    def iteration_us(self, client):        # microseconds since first op seen
        raise NotImplementedError

    def dispatch(self, client, owner, cls, op_index, event_slot):
        raise NotImplementedError

    def iteration_done(self, client, iteration):   # request_status[i][it]=true
        raise NotImplementedError

    def set_stop(self, client):            # client_stop[k] = true
        raise NotImplementedError

    def mark(self, owner, index):          # sliding_throttle only: a later
        pass                               # event_done(owner, index) will come


class PolicyOracle:
    """State that the reference keeps in file-scope globals
    (scheduler_eval.cpp:6-46) and that therefore survives between
    ``schedule`` calls: seen, event_ids, cur_iters, penalty, profiles."""

    def __init__(self, profiles, num_kernels, num_iters, is_train, max_sms=80,
                 sequential_fix=False, reserve_hp=False, admit_oversized=False,
                 sliding_throttle=False):
        # sliding_throttle (not in the reference, whose throttle :342-359 lets
        # go only when every best-effort stream has drained): when the duration
        # sum first passes depth // 2 the latest kernel of every best-effort
        # client is remembered (a mark) together with the sum; while throttled
        # the marks are asked about too, and once all have completed that part
        # of the sum is taken off and admission goes on.
        self.sliding_throttle = bool(sliding_throttle)
        # admit_oversized (not in the reference, whose CU clause :339-340 can
        # never admit a kernel whose un-clipped need exceeds max_sms while a
        # high-priority inference request is in flight): such a kernel goes in
        # if nothing else has been admitted in this poll, its class and the
        # running high-priority op's are both known and differ, and its
        # duration is at most depth // 4; it is placed on the smallest mask.
        self.admit_oversized = bool(admit_oversized)
        # reserve_hp (not in the reference): best-effort kernels admitted in one
        # poll may add up to max_sms minus the CU need of the high-priority op
        # last dispatched, instead of max_sms (:339 ignores that need).
        self.reserve_hp = bool(reserve_hp)
        # sequential_fix: the reference's time-slicing policy can never
        # dispatch once a client is past its 10th iteration (see _sequential).
        # With the flag set, the evident intent is restated instead: dispatch
        # unless another client is in the middle of an iteration.
        self.sequential_fix = bool(sequential_fix)
        n = len(profiles)
        assert len(num_kernels) == len(num_iters) == len(is_train) == n
        self.n = n
        self.ops = [list(p) for p in profiles]
        self.max_sms_clients = [max_sm_used(p) for p in profiles]   # :595-598
        self.num_kernels = list(num_kernels)                        # :608
        self.max_iters = list(num_iters)                            # :609
        self.is_train = [bool(t) for t in is_train]                 # :600
        self.max_sms = int(max_sms)                                 # :20
        self.seen = [0] * n                                         # :79
        self.event_ids = [0] * n                                    # :80
        self.cur_iters = [0] * n                                    # :611
        self.penalty = 0                                            # :43
        self.stops = [False] * n                                    # :646
        # exposed for tests
        self.sm_threshold = None
        self.large_found = False
        self.sum = 0

    def setup_change(self, client, ops, num_kernels):
        """setup_change (scheduler_eval.cpp:528-540)."""
        self.ops[client] = list(ops)
        self.max_sms_clients[client] = max_sm_used(ops)
        self.num_kernels[client] = int(num_kernels)

    # -- schedule_kernel + pop_from_queue (utils_sched.cpp:239-522, :113-117)
    def _dispatch(self, env, client, owner, cls, smallest_mask=False):
        op_index = self.seen[client]
        # the event handed to schedule_kernel is events[owner][event_ids[owner]]
        # evaluated before the call, i.e. before the increment below
        if smallest_mask:       # admit_oversized only: placement is forced
            env.dispatch(client, owner, cls, op_index, self.event_ids[owner],
                         smallest_mask=True)
        else:
            env.dispatch(client, owner, cls, op_index, self.event_ids[owner])
        if cls == KERNEL:            # every kernel-like case: :246-247 etc.
            self.event_ids[owner] += 1
            self.seen[client] += 1
        self._changed = True

    # -- schedule_reef (scheduler_eval.cpp:93-165)
    def _reef(self, env, heads, depth):
        n = self.n
        if n == 1:                                           # :97-103
            if heads[0] is not None:
                self._dispatch(env, 0, 0, heads[0])
            return
        hp = n - 1
        for i in range(n):                                   # :108-116
            if heads[i] is not None:
                if (heads[i] == MALLOC or self.cur_iters[i] <= 10
                        or self.cur_iters[hp] >= self.max_iters[hp]):
                    self._dispatch(env, i, i, heads[i])
                    return
        if heads[hp] is not None:                            # :119-141
            hp_idx = self.seen[hp]
            self._dispatch(env, hp, hp, heads[hp])
            op1 = self.ops[hp][hp_idx]
            for i in range(hp):
                if heads[i] is not None:
                    op0 = self.ops[i][self.seen[i]]
                    if (op0.duration <= op1.duration
                            and op0.sm_used >= op1.sm_used):  # :131
                        self._dispatch(env, i, i, heads[i])
                        return
        else:                                                # :142-164
            for i in range(hp):
                if heads[i] is not None:
                    self.penalty += 1
                    self._changed = True
            if self.penalty >= depth:
                for i in range(hp):
                    if heads[i] is not None:
                        self._dispatch(env, i, i, heads[i])
                self.penalty = 0

    # -- schedule_sequential (scheduler_eval.cpp:167-236)
    def _sequential(self, env, heads, start):
        n = self.n
        if n == 1:                                           # :173-179
            if heads[0] is not None:
                self._dispatch(env, 0, 0, heads[0])
            return start
        hp = n - 1
        if heads[hp] is not None:                            # :184-204
            go = False
            if self.cur_iters[hp] <= 10 or heads[hp] == MALLOC:
                go = True
            else:
                # :191-197 -- `schedule` starts false and the loop can only
                # set it false again: past warm-up the branch never fires.
                go = self.sequential_fix
                for i in range(hp):
                    if self.seen[i] > 0:
                        go = False
                        break
            if go:
                self._dispatch(env, hp, 0, heads[hp])        # stream/event 0
        end = start + n                                      # :207
        for t in range(start + 1, end):
            i = t % (n - 1)
            if heads[i] is not None:
                go = False
                if self.cur_iters[i] <= 10 or heads[i] == MALLOC:
                    go = True
                else:
                    go = self.sequential_fix
                    for j in range(n):                       # :216-222
                        if i != j and self.seen[j] > 0:
                            go = False
                            break
                if go:
                    self._dispatch(env, i, 0, heads[i])
                    start = t                                # :228 (t, not i)
                    break
        return start

    # -- busy_wait_profile (scheduler_eval.cpp:238-487)
    def schedule(self, env, warmup, warmup_iters, algo=ALGO_ORION, depth=1,
                 hp_limit=1, update_start=1, max_polls=None):
        n = self.n
        reef = algo == ALGO_REEF
        seq = algo == ALGO_SEQUENTIAL
        hp = n - 1                                           # :256
        profiles = [-1] * n                                  # :254
        large_found = False                                  # :258
        total = 0          # `sum`, a C long                  :259
        start = -1                                           # :261
        low_sms = 0                                          # :265
        high_sms = self.max_sms_clients[0]                   # :266
        sm_threshold = self.max_sms_clients[0] // 2          # :267
        hp_iter_duration = np.float32(0.0)                   # :268
        hp_limit_float = np.float32(hp_limit)                # :269
        if not self.is_train[hp]:                            # :272-275
            sm_threshold = self.max_sms
            update_start = INT_MAX
        polls = 0
        hp_need = 0
        mark_index = [-1] * n        # sliding_throttle: see __init__
        mark_valid = False
        mark_sum = 0

        while True:                                          # :277
            env.begin_poll()
            self._changed = False
            heads = [None] * n
            size = 0                                         # :279
            for i in range(n):                               # :281-302
                if self.seen[i] == self.num_kernels[i]:
                    continue
                heads[i] = env.peek(i)

            if reef:
                self._reef(env, heads, depth)
            elif seq:
                start = self._sequential(env, heads, start)
            else:
                if heads[hp] is not None:                    # :311-321
                    op1 = self.ops[hp][self.seen[hp]]
                    self._dispatch(env, hp, hp, heads[hp])
                    profiles[hp] = op1.profile
                    hp_need = op1.sm_used
                room = sm_threshold
                if self.reserve_hp and not self.is_train[hp]:
                    room = max(0, sm_threshold - max(0, hp_need))
                end = start + n                              # :323
                for t in range(start + 1, end):
                    j = t % (n - 1)                          # :326
                    if heads[j] is None:
                        continue
                    op0 = self.ops[j][self.seen[j]]          # :328
                    cls = heads[j]
                    mem_op = cls in MEM_CLASSES
                    go = False
                    oversized = False
                    if n == 1 or self.seen[hp] == 0 or mem_op:          # :333
                        go = True
                    elif (self.cur_iters[j] <= 10
                          or self.cur_iters[hp] >= self.max_iters[hp]):  # :335
                        go = True
                    elif (self.seen[hp] >= update_start
                          and op0.sm_used <= sm_threshold
                          and env.event_done(hp, update_start - 1)):    # :338
                        go = True
                    elif (self.seen[hp] > 0
                          and size + op0.sm_used <= room
                          and (op0.profile == -1 or profiles[hp] == -1
                               or profiles[hp] != op0.profile)):        # :340
                        go = True
                    elif (self.admit_oversized and not self.is_train[hp]
                          and size + op0.sm_used > room and size == 0
                          and op0.sm_used > self.max_sms
                          and op0.profile != -1 and profiles[hp] != -1
                          and profiles[hp] != op0.profile
                          and float(op0.duration) <= float(np.float32(depth // 4))):
                        go = True
                        oversized = True
                    if go and large_found:                   # :342-359
                        clear = True
                        for k in range(n - 1):
                            if self.event_ids[k] >= 1:
                                if not env.event_done(k, self.event_ids[k] - 1):
                                    clear = False
                                    break
                        if clear:
                            large_found = False
                            total = 0
                            self._changed = True
                            mark_valid = False
                        elif self.sliding_throttle and mark_valid:
                            half = True
                            for k in range(n - 1):
                                if mark_index[k] >= 0:
                                    if not env.event_done(k, mark_index[k]):
                                        half = False
                                        break
                            if half:
                                total = max(0, total - mark_sum)
                                mark_valid = False
                                large_found = False
                                self._changed = True
                            else:
                                go = False
                        else:
                            go = False
                    if go:                                   # :360-375
                        size += op0.sm_used
                        if not mem_op:                       # :364-365
                            # long += float: convert, add in fp32, truncate
                            total = int(np.float32(total)
                                        + np.float32(op0.duration))
                        if (total > depth
                                and self.cur_iters[hp] < self.max_iters[hp]):
                            large_found = True               # :366-368
                        self._dispatch(env, j, j, cls, oversized)
                        start = j                            # :374
                        if (self.sliding_throttle and not mem_op and not mark_valid
                                and total > depth // 2):
                            for k in range(n - 1):
                                mark_index[k] = self.event_ids[k] - 1
                                if mark_index[k] >= 0:
                                    env.mark(k, mark_index[k])
                            mark_sum = total
                            mark_valid = True

            finished = 0                                     # :380
            for i in range(n):
                if (self.cur_iters[i] == self.max_iters[i]
                        or (warmup and self.cur_iters[i] == warmup_iters)
                        or env.stop_ack(i)):                 # :383-388
                    finished += 1
                elif self.seen[i] == self.num_kernels[i]:    # :389
                    owner = 0 if seq else i                  # :397-408
                    ready = True
                    if self.event_ids[owner] >= 1:
                        if not env.event_done(owner, self.event_ids[owner] - 1):
                            ready = False
                    if ready:                                # :409-447
                        self.seen[i] = 0
                        if seq:
                            self.event_ids[0] = 0
                        self.event_ids[i] = 0
                        mark_index[i] = -1       # nothing of it is outstanding
                        env.iteration_done(i, self.cur_iters[i])
                        self.cur_iters[i] += 1
                        self._changed = True
                        # :423-425 microseconds -> float, then /= 1000.0
                        # (read only where the value is used, :427)
                        duration = np.float32(0.0)
                        if (not reef and not seq and i == hp
                                and self.is_train[hp]):
                            duration = np.float32(
                                float(np.float32(env.iteration_us(i))) / 1000.0)
                        if (not reef and not seq and i == hp
                                and self.is_train[hp]):      # :427-445
                            hp_iter_duration = np.float32(
                                hp_iter_duration + duration)
                            if (self.cur_iters[i] % 10 == 0
                                    and low_sms != sm_threshold):
                                avg = np.float32(
                                    float(hp_iter_duration) / 10.0)
                                hp_iter_duration = np.float32(0.0)
                                if avg > hp_limit_float:
                                    high_sms = sm_threshold
                                    sm_threshold = (low_sms + high_sms) // 2
                                else:
                                    low_sms = sm_threshold
                                    sm_threshold = (low_sms + high_sms) // 2
                    if (self.cur_iters[i] == self.max_iters[i]
                            or (warmup and self.cur_iters[i] == warmup_iters)
                            or env.stop_ack(i)):             # :448-452
                        finished += 1
                        if not warmup and i == n - 1:        # :454-468
                            for k in range(n - 1):
                                if not self.stops[k]:
                                    self._changed = True
                                self.stops[k] = True
                                env.set_stop(k)

            self.sm_threshold = sm_threshold
            self.large_found = large_found
            self.sum = total
            # The poll that ends the loop counts as effective even when only an
            # observation (a stop acknowledgement) moved, so a replay ends too.
            env.end_poll(self._changed or finished == n)
            if finished == n:                                # :474
                break
            polls += 1
            if max_polls is not None and polls >= max_polls:
                raise RuntimeError("policy oracle: poll budget exhausted")
