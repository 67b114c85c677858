"""Client threads are kept on the dynamic loader's fast path for thread-local
accesses (orion_amd/csrc/capture/tls_fresh.h).  Host-only: the stand-in runtime
and a native probe; no counterpart in the reference."""

import json
import os
import subprocess

import pytest

from tests.test_capture_scheduler_host import run_child

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CAPTURE = os.path.join(ROOT, "orion_amd", "libinttemp.so")


def test_every_client_thread_calls_into_a_fresh_copy(tmp_path):
    res = run_child(str(tmp_path), "orion", 2, 30)
    assert all(res["outputs_equal"]), res
    fresh = res["tls_fresh"]
    assert fresh["reloads"] >= 1
    # three client threads and the scheduler thread, once each per reload at least
    assert fresh["touches"] >= 4, fresh


def test_it_can_be_switched_off(tmp_path):
    res = run_child(str(tmp_path), "orion", 1, 20, extra_env={"ORION_TLS_REFRESH": "0"})
    assert all(res["outputs_equal"]), res
    assert res["tls_fresh"] == {"reloads": 0, "touches": 0}


def _build(tmp_path):
    for name in "ab":
        src = tmp_path / f"lib{name}.c"
        src.write_text(f"static __thread long v;\nlong touch_{name}(void) {{ return ++v; }}\n")
        subprocess.run(["gcc", "-O2", "-fPIC", "-ftls-model=global-dynamic", "-shared", str(src),
                        "-o", str(tmp_path / f"lib{name}.so")], check=True)
    probe = tmp_path / "probe"
    subprocess.run(["gcc", "-O2", os.path.join(ROOT, "tests", "native", "tls_fresh_probe.c"),
                    "-o", str(probe), "-ldl"], check=True)
    return probe


def test_a_stale_thread_is_cured(tmp_path):
    """A thread whose newest touched library is older than the newest loaded one
    pays for every thread-local access on glibc before 2.39; after the capture
    library's check it does not.  On a C library without that behaviour there is
    nothing to cure, and the test only checks that the mechanism ran."""
    probe = _build(tmp_path)
    env = dict(os.environ, ORION_HIP_LIBRARY=os.path.join(ROOT, "tests", "fakehip", "libfakehip.so"))
    best = None
    for _ in range(3):      # timing on a shared machine: the clearest of three runs
        out = subprocess.run([str(probe), CAPTURE, str(tmp_path / "liba.so"),
                              str(tmp_path / "libb.so")], check=True, capture_output=True,
                             text=True, env=env, timeout=120).stdout
        res = json.loads(out.strip().splitlines()[-1])
        assert res["reloads"] >= 1 and res["touches"] >= 1, res
        if best is None or res["stale_ns"] / res["fresh_ns"] > best["stale_ns"] / best["fresh_ns"]:
            best = res
    if best["stale_ns"] < 1.3 * best["fresh_ns"]:
        pytest.skip(f"this C library shows no slow path for stale threads: {best}")
    # back to within a fraction of the gap
    gap = best["stale_ns"] - best["fresh_ns"]
    assert best["cured_ns"] < best["fresh_ns"] + 0.4 * gap, best


def test_an_unscheduled_thread_can_ask_for_the_same(tmp_path):
    """orion_tls_fresh_check(): what a plain-stream client calls once per request
    under ORION_PLAIN_TLS_REFRESH=1 (benchmark_suite/client_common.py Backend)."""
    code = (
        "import ctypes, json, sys\n"
        f"sys.path.insert(0, {ROOT!r})\n"
        "from orion_amd import scheduler_frontend as fe\n"
        "lib = fe.load_capture_library()\n"
        "r, t = ctypes.c_ulonglong(), ctypes.c_ulonglong()\n"
        "lib.orion_tls_fresh_stats(ctypes.byref(r), ctypes.byref(t)); before = (r.value, t.value)\n"
        "lib.orion_tls_fresh_check(); lib.orion_tls_fresh_check()\n"
        "lib.orion_tls_fresh_stats(ctypes.byref(r), ctypes.byref(t))\n"
        "print(json.dumps({'before': before, 'after': (r.value, t.value)}))\n")
    env = dict(os.environ, ORION_HIP_LIBRARY=os.path.join(ROOT, "tests", "fakehip", "libfakehip.so"))
    out = subprocess.run([os.sys.executable, "-c", code], check=True, capture_output=True,
                         text=True, env=env, timeout=120).stdout
    res = json.loads(out.strip().splitlines()[-1])
    assert res["before"] == [0, 0]
    # one reload (nothing was loaded between the two calls), one call into it
    assert res["after"] == [1, 1], res


def test_a_missing_helper_library_is_reported_once_and_nothing_else_changes(tmp_path):
    proc_env = {"ORION_TLS_REFRESH_LIBRARY": str(tmp_path / "no_such_library.so")}
    res = run_child(str(tmp_path), "orion", 1, 20, extra_env=proc_env)
    assert all(res["outputs_equal"]), res
    assert res["iters_done"][-1] == 20
    assert res["tls_fresh"]["touches"] == 0 and res["tls_fresh"]["reloads"] >= 1
