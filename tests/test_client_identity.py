"""Which client an intercepted call belongs to (the reference's get_idx,
src/cuda_capture/utils_interc.cpp:3-51: OS thread id -> client index, the
scheduler's own thread and strangers pass through).  Here the lookup is cached
per thread, and calls from unregistered threads (autograd workers) are routed by
the stream they name.  Runs in a child process: arming is process-global."""

import os
import subprocess
import sys
import textwrap

from orion_amd import _lib

CHILD = textwrap.dedent("""
    import ctypes, threading, sys
    cap = ctypes.CDLL(sys.argv[1])
    cap.orion_client_of_stream.argtypes = [ctypes.c_void_p]
    cap.orion_register_stream.argtypes = [ctypes.c_void_p]
    N = 3
    go, armed, done = threading.Barrier(N + 3), threading.Barrier(N + 3), threading.Barrier(N + 3)
    tids, seen = {}, {}
    STREAM_OF = {0: 0x1000, 1: 0x2000, 2: 0x3000}

    def client(i):
        tids[i] = threading.get_native_id()
        go.wait(); armed.wait()
        seen[("idx", i)] = cap.orion_client_index()
        seen[("cpu", i)] = cap.orion_pinned_cpu()
        cap.orion_register_stream(STREAM_OF[i])
        cap.orion_thread_passthrough(1)
        seen[("bypass", i)] = cap.orion_client_index()
        cap.orion_thread_passthrough(0)
        seen[("again", i)] = cap.orion_client_index()
        done.wait(); done.wait()

    def scheduler():
        tids["sched"] = threading.get_native_id()
        go.wait(); armed.wait(); done.wait()
        # the scheduler's own calls never queue, whatever stream they name
        seen["sched"] = [cap.orion_client_index()] + [cap.orion_client_of_stream(s)
                                                      for s in STREAM_OF.values()]
        done.wait()

    def stranger():
        tids["stranger"] = threading.get_native_id()
        go.wait(); armed.wait(); done.wait()
        seen["stranger"] = [cap.orion_client_index(), cap.orion_client_of_stream(None),
                            cap.orion_client_of_stream(0x9999)] + [
                            cap.orion_client_of_stream(s) for s in STREAM_OF.values()]
        # the first client it worked for (client 0) decides where it runs
        import os
        seen["stranger_cpu"] = [cap.orion_pinned_cpu(), sorted(os.sched_getaffinity(0))]
        cap.orion_register_thread(1)          # an adopted helper thread
        seen["adopted"] = [cap.orion_client_index(), cap.orion_client_of_stream(0x1000)]
        done.wait()

    ts = [threading.Thread(target=client, args=(i,)) for i in range(N)]
    ts += [threading.Thread(target=scheduler), threading.Thread(target=stranger)]
    for t in ts: t.start()
    seen["before"] = cap.orion_client_index()
    go.wait()
    arr = (ctypes.c_int * N)(*[tids[i] for i in range(N)])
    cap.orion_capture_arm(N, arr, tids["sched"])
    armed.wait(); done.wait(); done.wait()
    for t in ts: t.join()
    seen["main"] = cap.orion_client_index()
    cap.orion_capture_disarm()
    seen["after"] = cap.orion_client_of_stream(0x1000)
    print(repr(sorted((str(k), v) for k, v in seen.items())))
""")


def test_thread_and_stream_identity():
    out = subprocess.run([sys.executable, "-c", CHILD, _lib.CAPTURE_LIB],
                         capture_output=True, text=True, timeout=60,
                         env=dict(os.environ, ORION_PIN_THREADS="1"))
    assert out.returncode == 0, out.stderr
    seen = dict(eval(out.stdout.strip().splitlines()[-1]))
    for i in range(3):
        assert seen[str(("idx", i))] == i
        assert seen[str(("bypass", i))] < 0       # pass-through beats identity
        assert seen[str(("again", i))] == i
    assert seen["before"] < 0 and seen["main"] < 0 and seen["after"] < 0
    assert all(v < 0 for v in seen["sched"])
    # stranger: no identity of its own, none for a null or foreign stream, the
    # owner's for each registered stream
    assert all(v < 0 for v in seen["stranger"][:3])
    assert seen["stranger"][3:] == [0, 1, 2]
    # an adopted thread is its client whatever stream it names
    assert seen["adopted"] == [1, 1]
    # a thread that works for a client by naming its stream runs on that client's
    # CPU from then on (reference: utils_interc.cpp:28-49), when threads are pinned
    cpu0 = seen[str(("cpu", 0))]
    if cpu0 >= 0:
        assert seen["stranger_cpu"] == [cpu0, [cpu0]]
        assert len({seen[str(("cpu", i))] for i in range(3)}) == 3
    else:
        assert seen["stranger_cpu"][0] < 0


def test_rearming_remaps_cached_threads():
    child = textwrap.dedent("""
        import ctypes, threading, sys
        cap = ctypes.CDLL(sys.argv[1])
        me = threading.get_native_id()
        out = []
        for order in ([me, 1], [1, me], [1, 2]):
            cap.orion_capture_arm(2, (ctypes.c_int * 2)(*order), 7)
            out.append(cap.orion_client_index())
        cap.orion_capture_disarm()
        out.append(cap.orion_client_index())
        print(out)
    """)
    out = subprocess.run([sys.executable, "-c", child, _lib.CAPTURE_LIB],
                         capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stderr
    got = eval(out.stdout.strip().splitlines()[-1])
    assert got[0] == 0 and got[1] == 1 and got[2] < 0 and got[3] < 0
