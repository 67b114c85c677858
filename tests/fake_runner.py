"""Drives libinttemp.so + scheduler_eval.so end to end on a host without a GPU,
against the recording HIP stand-in (tests/fakehip).  Runs in its own process
(the HIP table of a process is resolved once); prints one JSON object.

usage: python tests/fake_runner.py <workdir> <algo> <n_be> <hp_iters> [graph]

With ``graph`` the high-priority client submits each iteration's kernels as one
executable graph (hipGraphLaunch): one kernel-class record per iteration.

FAKE_RUNNER_UNTYPED=1: both libraries are called the way the reference calls
them -- ``ctypes.cdll.LoadLibrary`` and nothing else, so every entry point has
ctypes' default prototype: the scheduler handle comes back as a C int (the
pointer's low 32 bits) and is passed on as that, Python bools travel as ints
(src/scheduler_frontend.py:13,56-94; train_imagenet.py:63-68,88).  The
best-effort clients then also get a second profile, so that setup_change runs.
"""

import ctypes
import json
import os
import sys
import threading

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
os.environ["ORION_HIP_LIBRARY"] = os.path.join(ROOT, "tests", "fakehip", "libfakehip.so")

import numpy as np  # noqa: E402

from orion_amd import scheduler_frontend as fe  # noqa: E402

workdir, algo, n_be, hp_iters = sys.argv[1], sys.argv[2], int(sys.argv[3]), int(sys.argv[4])
hp_graph = len(sys.argv) > 5 and sys.argv[5] == "graph"
os.environ["ORION_RECORD_DIR"] = workdir
os.environ["ORION_QUIET"] = "1"

untyped = bool(os.environ.get("FAKE_RUNNER_UNTYPED"))
fake = ctypes.CDLL(os.environ["ORION_HIP_LIBRARY"])
cap = fe.load_capture_library()
sched = fe.load_scheduler_library()
fake.fakehip_set_costs(ctypes.c_longlong(30000), ctypes.c_longlong(4000))

SAXPY = ctypes.cast(fake.fake_kernel_saxpy, ctypes.c_void_p)
SQADD = ctypes.cast(fake.fake_kernel_sqadd, ctypes.c_void_p)
cap.hipModuleLaunchKernel.argtypes = [ctypes.c_void_p] + [ctypes.c_uint] * 7 + [
    ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p]
cap.hipMemcpyAsync.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
                               ctypes.c_int, ctypes.c_void_p]
cap.hipMalloc.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t]
cap.hipStreamSynchronize.argtypes = [ctypes.c_void_p]
cap.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]

cap.hipGraphLaunch.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
cap.hipMallocAsync.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t, ctypes.c_void_p]
cap.hipFreeAsync.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
cap.hipMemcpy2D.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_size_t,
                            ctypes.c_size_t, ctypes.c_size_t, ctypes.c_int]


if untyped:
    from orion_amd import _lib
    raw_sched = ctypes.cdll.LoadLibrary(_lib.SCHEDULER_LIB)   # no argtypes, no restype
    raw_cap = ctypes.cdll.LoadLibrary(_lib.CAPTURE_LIB)
    control = raw_cap
else:
    control = cap


class FakeGraphExec(ctypes.Structure):      # mirrors tests/fakehip/fakehip.cpp
    _fields_ = [("n", ctypes.c_int), ("fn", ctypes.c_void_p * 8),
                ("params", ctypes.POINTER(ctypes.c_void_p) * 8)]


N = 64
n_clients = n_be + 1
kernels_per_iter = [5 + c for c in range(n_clients)]      # what an iteration computes
records_per_iter = list(kernels_per_iter)                 # what the scheduler counts
if hp_graph:
    records_per_iter[-1] = 1
if os.environ.get("FAKE_RUNNER_MISCOUNT"):
    # tell the scheduler one kernel more (or, with -1, one fewer) than client 0
    # submits per iteration
    records_per_iter[0] += int(os.environ["FAKE_RUNNER_MISCOUNT"])
iters = [10_000] * n_be + [hp_iters]
# FAKE_RUNNER_MODEL_NAMES=a,b,c: the model names setup() is given, one per client
model_names = (os.environ["FAKE_RUNNER_MODEL_NAMES"].split(",")
               if os.environ.get("FAKE_RUNNER_MODEL_NAMES") else ["fake"] * n_clients)
assert len(model_names) == n_clients


def write_profile(path, nk, seed, names=None):
    rng = np.random.default_rng(seed)
    with open(path, "w") as f:
        f.write("Name,Profile,Memory_footprint,SM_usage,Duration\n")
        for i in range(nk):
            f.write(f"{names[i] if names else f'k{i}'},{int(rng.integers(-1, 2))},0,"
                    f"{int(rng.integers(1, 300))},{int(rng.integers(5000, 60000))}\n")


def kernel_names(tid):
    """FAKE_RUNNER_NAMED_PROFILE=1: profile rows carry the names of the kernels the
    client launches (row k: saxpy for even k, sqadd for odd k).  With
    FAKE_RUNNER_PROFILE_INSERT=r client 0's profile has one more row, named
    fake_extra, at row r -- a profile captured with a solver the run does not use."""
    if not os.environ.get("FAKE_RUNNER_NAMED_PROFILE"):
        return None
    names = ["fake_kernel_saxpy" if k % 2 == 0 else "fake_kernel_sqadd"
             for k in range(kernels_per_iter[tid])]
    if tid == 0 and os.environ.get("FAKE_RUNNER_PROFILE_INSERT"):
        names.insert(int(os.environ["FAKE_RUNNER_PROFILE_INSERT"]), "fake_extra")
    return names + ["fake_kernel_saxpy"] * 4      # spare rows: a profile may hold more


files = []
for c in range(n_clients):
    p = os.path.join(workdir, f"client{c}.csv")
    write_profile(p, records_per_iter[c], c, kernel_names(c))
    write_profile(p + ".steady", records_per_iter[c], 100 + c, kernel_names(c))   # setup_change's file
    files.append(p)

results = [None] * n_clients
placement = [None] * (n_clients + 1)     # (pinned cpu, allowed set) while the job runs
iters_done = [0] * n_clients
barriers = [threading.Barrier(n_clients + 1)]


def param_array(params):
    return (ctypes.c_void_p * len(params))(*[ctypes.cast(ctypes.pointer(p), ctypes.c_void_p)
                                             for p in params])


class Dim3(ctypes.Structure):
    _fields_ = [("x", ctypes.c_uint), ("y", ctypes.c_uint), ("z", ctypes.c_uint)]


cap.hipLaunchKernel.argtypes = [ctypes.c_void_p, Dim3, Dim3, ctypes.POINTER(ctypes.c_void_p),
                                ctypes.c_size_t, ctypes.c_void_p]
cap.orion_client_deferred.restype = ctypes.c_ulonglong
cap.orion_client_submitted.restype = ctypes.c_ulonglong
cap.hipStreamWriteValue32.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint,
                                      ctypes.c_uint]
HOST_FN = ctypes.CFUNCTYPE(None, ctypes.c_void_p)
cap.hipLaunchHostFunc.argtypes = [ctypes.c_void_p, HOST_FN, ctypes.c_void_p]
BUFFER_POINTER, BUFFER_SIZE, PARAM_END = 1, 2, 3      # HIP_LAUNCH_PARAM_*


def launch(func, params, form=0):
    """One kernel through one of the three launch forms a client's libraries
    use.  The arguments are private copies that are overwritten as soon as the
    call returns: a record that still pointed at them when the scheduler issues
    it later would compute garbage."""
    mine = [type(p)(p.value) for p in params]
    if form == 0:        # module launch with a kernelParams array
        rc = cap.hipModuleLaunchKernel(func, 1, 1, 1, 64, 1, 1, 0, None, param_array(mine), None)
    elif form == 1:      # hipLaunchKernel: argument sizes known to the runtime only
        # each kernel with a block of its own launch bounds (256 and 64)
        block = 256 if func.value == SAXPY.value else 64
        rc = cap.hipLaunchKernel(func, Dim3(1, 1, 1), Dim3(block, 1, 1), param_array(mine), 0, None)
    else:                # module launch with one argument buffer
        buf = bytearray()
        for p in mine:
            size = ctypes.sizeof(p)
            buf += bytes(-len(buf) % size) + bytes(p)
        raw = (ctypes.c_ubyte * len(buf)).from_buffer(buf)
        size = ctypes.c_size_t(len(buf))
        extra = (ctypes.c_void_p * 5)(BUFFER_POINTER, ctypes.addressof(raw), BUFFER_SIZE,
                                      ctypes.addressof(size), PARAM_END)
        rc = cap.hipModuleLaunchKernel(func, 1, 1, 1, 64, 1, 1, 0, None, None, extra)
        ctypes.memset(raw, 0xff, len(buf))
        size.value = 0
    assert rc == 0, rc
    # a framework's launch check: queueing the call must leave no error of the
    # library's own in this thread's last-error slot
    stale = fake.hipGetLastError()
    assert stale == 0, f"stale error {stale} after a launch"
    for p in mine:
        ctypes.memset(ctypes.byref(p), 0xff, ctypes.sizeof(p))


def client(tid):
    nk = kernels_per_iter[tid]
    host_x = np.arange(N, dtype=np.float32) / N + tid
    barriers[0].wait()
    dev_y, dev_x = ctypes.c_void_p(), ctypes.c_void_p()
    assert cap.hipMalloc(ctypes.byref(dev_y), N * 4) == 0
    assert cap.hipMalloc(ctypes.byref(dev_x), N * 4) == 0
    zeros = np.zeros(N, dtype=np.float32)
    cap.hipMemcpy(dev_y, zeros.ctypes.data, N * 4, 1)
    # stream-ordered allocation and a blocking 2-D copy: granted back to this
    # thread, on the stream the scheduler assigned
    scratch = ctypes.c_void_p()
    assert cap.hipMallocAsync(ctypes.byref(scratch), 2 * N * 4, None) == 0
    assert cap.hipMemcpy2D(scratch, N * 4, host_x.ctypes.data, N * 4, N * 4, 1, 1) == 0
    back = np.empty(N, dtype=np.float32)
    assert cap.hipMemcpy2D(back.ctypes.data, N * 4, scratch, N * 4, N * 4, 1, 2) == 0
    assert np.array_equal(back, host_x)
    assert cap.hipFreeAsync(scratch, None) == 0
    it = 0
    flag_word = ctypes.c_uint(0)
    calls = [0]

    @HOST_FN
    def bump(_):
        calls[0] += 1
    n_c, a_c = ctypes.c_int(N), ctypes.c_float(0.5)
    c_c = ctypes.c_float(0.125)
    graph = None
    if hp_graph and tid == n_clients - 1:
        graph, keep = FakeGraphExec(), []
        graph.n = nk
        for k in range(nk):
            arr = param_array([dev_y, dev_x, a_c, n_c] if k % 2 == 0 else [dev_y, c_c, n_c])
            keep.append(arr)
            graph.fn[k] = SAXPY if k % 2 == 0 else SQADD
            graph.params[k] = ctypes.cast(arr, ctypes.POINTER(ctypes.c_void_p))
    while it < iters[tid]:
        cap.hipMemcpyAsync(dev_x, host_x.ctypes.data, N * 4, 1, None)
        if graph is not None:
            assert cap.hipGraphLaunch(ctypes.byref(graph), None) == 0
        # a best-effort client reads x through a temporary it allocates, fills by a
        # device copy and frees right after the launch that reads it, relying on
        # the free to wait for the device as the runtime's does: the free must not
        # take effect before a launch that is still queued has run (the stand-in
        # fills freed memory with NaNs)
        tmp = None
        if graph is None and tid < n_clients - 1:
            tmp = ctypes.c_void_p()
            assert cap.hipMalloc(ctypes.byref(tmp), N * 4) == 0
            assert cap.hipMemcpyAsync(tmp, dev_x, N * 4, 3, None) == 0
        for k in range(nk if graph is None else 0):
            if k % 2 == 0:
                launch(SAXPY, [dev_y, tmp if (tmp and k == 0) else dev_x, a_c, n_c], (k + it) % 3)
            else:
                launch(SQADD, [dev_y, c_c, n_c], (k + it) % 3)
            if tmp and k == 0:
                assert cap.hipFree(tmp) == 0
        # a stream memory operation and a host callback on the (null) stream the
        # client names: both must follow its work to where the scheduler put it
        assert cap.hipStreamWriteValue32(None, ctypes.byref(flag_word), it + 1, 0) == 0
        assert cap.hipLaunchHostFunc(None, bump, None) == 0
        # the write is stream work: it has happened once the stream has drained
        # (the asynchronous stand-in runs it later, the immediate one at once)
        assert cap.hipStreamSynchronize(None) == 0
        assert flag_word.value == it + 1 and calls[0] == it + 1
        control.block(it)
        it += 1
        iters_done[tid] = it
        if it == 1:
            placement[tid] = (cap.orion_pinned_cpu(), sorted(os.sched_getaffinity(0)))
            if tid == n_clients - 1:      # the scheduler thread, seen from outside
                placement[n_clients] = sorted(os.sched_getaffinity(sched_tid[0]))
        if it in (1, 10):
            barriers[0].wait()
        if control.stop():
            break
    barriers[0].wait()
    out = np.empty(N, dtype=np.float32)
    cap.hipMemcpy(out.ctypes.data, dev_y, N * 4, 2)
    results[tid] = out


def expected(tid, n_iters):
    nk = kernels_per_iter[tid]
    x = np.arange(N, dtype=np.float32) / N + tid
    y = np.zeros(N, dtype=np.float32)
    with np.errstate(over="ignore"):
        for _ in range(n_iters):
            for k in range(nk):
                if k % 2 == 0:
                    y = np.float32(0.5) * x + y
                else:
                    y = y * y + np.float32(0.125)
    return y


threads = [threading.Thread(target=client, args=(c,)) for c in range(n_clients)]
for t in threads:
    t.start()
tids = [t.native_id for t in threads]
py = fe.PyScheduler(sched, n_clients)
sched_tid = []
sched_after = []


handle_seen = []


def run_sched_untyped():
    """The reference front end's calls, in its order and with its argument
    objects (src/scheduler_frontend.py:13, :39-60, :72, :78, :85, :91)."""
    sched_tid.append(threading.get_native_id())
    n = n_clients
    handle = raw_sched.sched_init()          # default restype: a C int
    handle_seen.append(handle)
    IntAr, CharAr, BoolAr = ctypes.c_int * n, ctypes.c_char_p * n, ctypes.c_bool * n
    tids_ar, nk_ar, ni_ar = IntAr(*tids), IntAr(*records_per_iter), IntAr(*iters)
    names_ar = CharAr(*[m.encode() for m in model_names])
    files_ar = CharAr(*[f.encode("utf-8") for f in files])
    train = [True] * n_be + [False]
    train_ar = BoolAr(*train)
    reef, seq = algo == "reef", algo == "sequential"
    depth = 8 if reef else 100_000
    raw_sched.setup(handle, n, tids_ar, names_ar, files_ar, nk_ar, ni_ar, train_ar, reef)
    barriers[0].wait()
    raw_sched.schedule(handle, n, True, 0, True, 1, reef, seq, depth, 1, 1)
    for j in range(n):
        if train[j]:
            raw_sched.setup_change(handle, j, (files[j] + ".steady").encode("utf-8"),
                                   records_per_iter[j])
    barriers[0].wait()
    raw_sched.schedule(handle, n, True, 0, True, 10, reef, seq, depth, 1, 1)
    barriers[0].wait()
    raw_sched.schedule(handle, n, True, 0, False, 0, reef, seq, depth, 1, 1)
    barriers[0].wait()
    sched_after.extend(sorted(os.sched_getaffinity(0)))


def run_sched():
    if untyped:
        return run_sched_untyped()
    sched_tid.append(threading.get_native_id())
    py.run_scheduler(barriers, tids, model_names, files,
                     [None] * n_clients, records_per_iter, [None] * n_clients,
                     iters, True, True, algo == "reef", algo == "sequential",
                     8 if algo == "reef" else 100_000, 1, 1, [True] * n_be + [False])
    sched_after.extend(sorted(os.sched_getaffinity(0)))


st = threading.Thread(target=run_sched)
st.start()
for t in threads:
    t.join(timeout=120)
st.join(timeout=120)
alive = [t.is_alive() for t in threads] + [st.is_alive()]

log = []
kind, sid, tid_, a, b = (ctypes.c_int(), ctypes.c_int(), ctypes.c_int(),
                         ctypes.c_ulonglong(), ctypes.c_ulonglong())
for i in range(fake.fakehip_log_size()):
    fake.fakehip_log_get(i, ctypes.byref(kind), ctypes.byref(sid), ctypes.byref(tid_),
                         ctypes.byref(a), ctypes.byref(b))
    log.append((kind.value, sid.value, tid_.value))
launch_tids = sorted({t for k, s, t in log if k == 0})
launch_streams = sorted({s for k, s, t in log if k == 0})
masks = {s: fake.fakehip_stream_mask_bits(s) for s in launch_streams}

ok_outputs = []
for c in range(n_clients):
    want = expected(c, iters_done[c])
    ok_outputs.append(bool(results[c] is not None and np.array_equal(results[c], want)))

_reloads, _touches = ctypes.c_ulonglong(), ctypes.c_ulonglong()
cap.orion_tls_fresh_stats(ctypes.byref(_reloads), ctypes.byref(_touches))

print(json.dumps({
    "alive": alive, "iters_done": iters_done, "handle": handle_seen,
    "tls_fresh": {"reloads": int(_reloads.value), "touches": int(_touches.value)},
    "deferred": [int(cap.orion_client_deferred(c)) for c in range(n_clients)],
    "submitted": [int(cap.orion_client_submitted(c)) for c in range(n_clients)],
    "holder_sets": sum(1 for k, s, t in log if k == 8),
    # host callbacks and stream memory operations: [stream id, thread] each
    "stream_ops": [[s, t] for k, s, t in log if k == 9], "outputs_equal": ok_outputs,
    "async_allocs": [[s, t] for k, s, t in log if k == 3 and s != 0],
    "async_frees": [[s, t] for k, s, t in log if k == 4 and s != 0],
    "placement": placement[:n_clients], "scheduler_placement": placement[n_clients],
    "scheduler_mask_after": sched_after, "allowed_cpus": sorted(os.sched_getaffinity(0)),
    "launch_tids": launch_tids, "sched_tid": sched_tid, "client_tids": tids,
    "launch_stream_masks": masks, "n_launches": sum(1 for k, s, t in log if k == 0),
    "launch_streams_by_tid": {str(t): sorted({s for k, s, tt in log if k == 0 and tt == t})
                              for t in launch_tids},
    "launches_by_tid": {str(t): sum(1 for k, s, tt in log if k == 0 and tt == t)
                        for t in launch_tids},
}))
sys.stdout.flush()
os._exit(0 if not any(alive) else 3)
