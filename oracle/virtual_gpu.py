"""A deterministic virtual-time model of clients, queues and a GPU.

TEST INFRASTRUCTURE ONLY (see ``oracle/policy_oracle.py``).

It closes the world around the policy so that a run is a pure function of the
job description: clients hand one record at a time to their queue and wait for
it to be taken (the reference's hand-off, src/cuda_capture/utils_interc.cpp:53-64
and intercept_temp.cpp:418-458); a dispatched kernel occupies its stream for the
profiled duration; an event completes when virtual time passes the end of the
op it was recorded after.  Time is an integer count of nanoseconds.

The model is not a performance predictor.  It exists to put the policy through
every branch (warm-up gates, admission, throttle, stop protocol, phases) in a
reproducible way, and to produce observation logs the native core must replay
to the same decisions.
"""

from oracle import policy_oracle as po


class VClient:
    """One client thread of the launcher (benchmarking/launch_jobs.py:78-86).

    trace_of(iteration) -> sequence of record classes one iteration submits.
    arrivals: None for a closed loop, else a list of inter-arrival gaps (ns)
    used once the client is past its tenth iteration
    (benchmark_suite/train_imagenet.py:185-191)."""

    def __init__(self, trace_of, max_iters, gap_ns=2000, arrivals=None):
        self.trace_of = trace_of
        self.max_iters = max_iters
        self.gap_ns = gap_ns
        self.arrivals = arrivals
        self.iteration = 0
        self.trace = None
        self.pos = 0
        self.visible_at = None     # when the head record becomes visible
        self.next_arrival = 0
        self.stop_flag = False
        self.acked = False
        self.parked = True         # waiting at a launcher barrier
        self.released_upto = 0     # iterations the scheduler has released


class VirtualGpu(po.Env):
    def __init__(self, clients, duration_of, poll_ns=400, dispatch_ns=2500,
                 mem_ns=3000):
        self.clients = clients
        self.duration_of = duration_of   # callable(client, op_index) -> ns
        self.poll_ns = poll_ns
        self.dispatch_ns = dispatch_ns
        self.mem_ns = mem_ns
        self.now = 0
        self.stream_free = {}
        self.event_time = {}
        self.phase_limit = 0
        self.iter_start = [0] * len(clients)
        self.start_pending = [True] * len(clients)
        self.released = []               # (client, iteration, time)
        self.dispatched = []             # (time, client, owner, cls, op_index)

    # -- launcher side ---------------------------------------------------
    def start_phase(self, limit):
        """Release clients parked at a barrier; they may run iterations
        < limit (None = until max_iters)."""
        self.phase_limit = limit
        for c in self.clients:
            if c.parked and not c.acked and c.iteration < c.max_iters:
                if limit is None or c.iteration < limit:
                    c.parked = False
                    c.next_arrival = self.now
                    self._begin_iteration(c, self.now + c.gap_ns)

    def _begin_iteration(self, c, earliest):
        c.trace = list(c.trace_of(c.iteration))
        c.pos = 0
        start = earliest
        if c.arrivals is not None and c.iteration >= 10:
            start = max(earliest, c.next_arrival)
        c.visible_at = start if c.trace else None
        if not c.trace:
            raise ValueError("an iteration must submit at least one record")

    def _after_release(self, c):
        if c.arrivals is not None:
            if c.iteration >= 10:
                gap = c.arrivals[(c.iteration - 10) % len(c.arrivals)]
                c.next_arrival += gap
            else:
                c.next_arrival = self.now
        c.iteration += 1
        c.trace, c.visible_at = None, None
        if c.stop_flag:                      # stop() polled once per iteration
            c.acked = True
            return
        if c.iteration >= c.max_iters:
            return
        if self.phase_limit is not None and c.iteration >= self.phase_limit:
            c.parked = True
            return
        self._begin_iteration(c, self.now + c.gap_ns)

    # -- Env ---------------------------------------------------------------
    def begin_poll(self):
        self.now += self.poll_ns

    def end_poll(self, changed):
        if changed:
            return
        # Nothing moved: jump to the next instant at which something can.
        horizon = []
        for c in self.clients:
            if c.visible_at is not None and c.visible_at > self.now:
                horizon.append(c.visible_at)
        horizon += [t for t in self.event_time.values() if t > self.now]
        if horizon:
            self.now = max(self.now, min(horizon) - self.poll_ns)

    def stop_ack(self, client):
        return self.clients[client].acked

    def peek(self, client):
        c = self.clients[client]
        if c.visible_at is None or c.visible_at > self.now:
            return None
        # client_starts[i] is taken at the first record seen while seen[i] == 0
        # and the iteration's flag is still clear (scheduler_eval.cpp:290-292)
        if self.start_pending[client]:
            self.iter_start[client] = self.now
            self.start_pending[client] = False
        return c.trace[c.pos]

    def event_done(self, owner, index):
        return self.event_time[(owner, index)] <= self.now

    def iteration_us(self, client):
        return (self.now - self.iter_start[client]) // 1000

    def dispatch(self, client, owner, cls, op_index, event_slot):
        c = self.clients[client]
        assert c.visible_at is not None and c.visible_at <= self.now
        assert c.trace[c.pos] == cls
        busy = self.duration_of(client, op_index) if cls == po.KERNEL \
            else self.mem_ns
        begin = max(self.now, self.stream_free.get(owner, 0))
        self.stream_free[owner] = begin + int(busy)
        self.event_time[(owner, event_slot)] = self.stream_free[owner]
        self.dispatched.append((self.now, client, owner, cls, op_index))
        self.now += self.dispatch_ns
        c.pos += 1
        c.visible_at = self.now + c.gap_ns if c.pos < len(c.trace) else None
        # Records after the iteration's last kernel (an output copy, say) are
        # taken after the scheduler has already released the iteration
        # (scheduler_eval.cpp:389-421 holds the client's mutex meanwhile).
        if c.pos == len(c.trace) and c.released_upto > c.iteration:
            self._after_release(c)

    def iteration_done(self, client, iteration):
        c = self.clients[client]
        assert c.released_upto == iteration
        c.released_upto += 1
        self.start_pending[client] = True
        self.released.append((client, iteration, self.now))
        if c.trace is not None and c.iteration == iteration \
                and c.pos == len(c.trace):
            self._after_release(c)

    def set_stop(self, client):
        c = self.clients[client]
        c.stop_flag = True
        if c.trace is None and not c.acked:
            # idle (parked, or out of iterations): the next stop() poll acks
            c.acked = True


def run_job(oracle, env, rec, phases, setup_changes=None, algo=po.ALGO_ORION,
            depth=1, hp_limit=1, update_start=1, max_polls=2_000_000):
    """The three-phase run of the frontend (src/scheduler_frontend.py:68-94):
    one warm-up iteration, profile swap, ten warm-up iterations, measured run.
    ``phases`` is a list of (warmup, warmup_iters); ``setup_changes`` maps the
    phase index before which a swap happens to [(client, ops, nk, path)]."""
    setup_changes = setup_changes or {}
    for idx, (warmup, warmup_iters) in enumerate(phases):
        for client, ops, nk, path in setup_changes.get(idx, []):
            oracle.setup_change(client, ops, nk)
            rec.setup_change(client, nk, path)
        env.start_phase(warmup_iters if warmup else None)
        rec.begin_schedule(warmup, warmup_iters, algo, depth, hp_limit,
                           update_start)
        oracle.schedule(rec, warmup, warmup_iters, algo, depth, hp_limit,
                        update_start, max_polls=max_polls)
        rec.end_schedule()
