"""The interception layer and the scheduler under ThreadSanitizer (host only).

The reference shares plain ints and `volatile bool`s between the client threads
and the scheduler thread (src/cuda_capture/intercept_temp.cpp:16-19,
src/scheduler/scheduler_eval.cpp:24,36); the hand-off here is built on C++11
atomics, and this test is what holds it to that: every library source is
compiled with -fsanitize=thread into one stress program (client threads pushing
records, scheduler thread running the three-phase schedule against the
recording HIP stand-in), which must finish with the right outputs and without
a reported race.
"""

import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "orion_amd", "csrc")


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_capture_and_scheduler_are_race_free(tmp_path):
    exe = str(tmp_path / "stress_tsan")
    fake = str(tmp_path / "libfakehip_tsan.so")
    common = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=thread", "-fPIC", "-pthread",
              "-I" + os.path.join(ROOT, "include"), "-I/opt/rocm/include",
              "-I" + os.path.join(CSRC, "policy")]
    subprocess.run(common + ["-shared", os.path.join(ROOT, "tests", "fakehip", "fakehip.cpp"),
                             "-o", fake], check=True)
    srcs = [os.path.join(CSRC, p) for p in (
        "capture/capture.cpp", "capture/tls_fresh.cpp", "common/hip_api.cpp", "policy/policy.cpp",
        "policy/obslog.cpp",
        "scheduler/scheduler_eval.cpp", "scheduler/profile_capture.cpp")]
    subprocess.run(common + srcs + [os.path.join(ROOT, "tests", "native", "stress_capture.cpp"),
                                    fake, "-Wl,-rpath," + str(tmp_path), "-ldl", "-o", exe],
                   check=True)
    # the thread-local helper library is loaded once here; reloading it while
    # clients run is left to the un-sanitized run below (the sanitizer's own
    # bookkeeping of dynamically allocated thread-local blocks does not survive a
    # library being unloaded and loaded again: it aborts inside its
    # __tls_get_addr interceptor, not in the code under test)
    helper = str(tmp_path / "liborion_tlsfresh.so")
    subprocess.run(["gcc", "-O2", "-fPIC", "-ftls-model=global-dynamic", "-shared",
                    os.path.join(CSRC, "capture", "tls_fresh_helper.c"), "-o", helper], check=True)
    env = dict(os.environ, ORION_HIP_LIBRARY=fake, ORION_QUIET="1",
               ORION_TLS_REFRESH_LIBRARY=helper, STRESS_EXPECT_TLS_RELOADS="1",
               TSAN_OPTIONS="halt_on_error=1 exitcode=66 second_deadlock_stack=1")
    env.pop("LD_PRELOAD", None)
    # both hand-offs of the high-priority client: issuing its own calls and
    # queueing notices (default), and the synchronous hand-off of every record
    # and both hand-offs of the best-effort clients: every record waited for
    # (default), and records that carry their arguments queued ahead
    # and both ways the stand-in runtime executes: at the call, and later on a
    # thread of its own, the streams in an order it draws at random
    # (the last: hipLaunchKernel left synchronous among records queued ahead)
    for clients, direct, ahead, later, holders in (
            (2, "1", "1", "0", "1"), (4, "1", "1", "0", "1"), (3, "0", "1", "0", "1"),
            (3, "1", "0", "0", "1"), (4, "1", "1", "1", "1"), (3, "1", "0", "1", "1"),
            (3, "1", "1", "1", "0")):
        proc = subprocess.run([exe, str(tmp_path), str(clients), "40"],
                              env=dict(env, ORION_HP_DIRECT=direct, ORION_BE_RUN_AHEAD=ahead,
                                       FAKEHIP_ASYNC=later, ORION_BE_RUN_AHEAD_HOLDERS=holders),
                              capture_output=True, text=True, timeout=600)
        assert "WARNING: ThreadSanitizer" not in proc.stderr, proc.stderr[-4000:]
        assert proc.returncode == 0, proc.stdout + proc.stderr[-4000:]


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_order_and_lifetime_on_the_asynchronous_runtime(tmp_path):
    """The same stress program, optimised and without the sanitizer, against the
    stand-in runtime in its asynchronous mode: launches return at once, an
    executor thread runs each stream in order and the streams against each other
    in a random order, a free waits for the device and fills the block with NaNs.
    Work issued without the cross-stream edge, the wait or the postponed release
    it needs computes a different result (checked by taking each of them out)."""
    exe = str(tmp_path / "stress")
    fake = str(tmp_path / "libfakehip_async.so")
    common = ["g++", "-std=c++17", "-O2", "-g", "-fPIC", "-pthread",
              "-I" + os.path.join(ROOT, "include"), "-I/opt/rocm/include",
              "-I" + os.path.join(CSRC, "policy")]
    subprocess.run(common + ["-shared", os.path.join(ROOT, "tests", "fakehip", "fakehip.cpp"),
                             "-o", fake], check=True)
    srcs = [os.path.join(CSRC, p) for p in (
        "capture/capture.cpp", "capture/tls_fresh.cpp", "common/hip_api.cpp", "policy/policy.cpp",
        "policy/obslog.cpp",
        "scheduler/scheduler_eval.cpp", "scheduler/profile_capture.cpp")]
    subprocess.run(common + srcs + [os.path.join(ROOT, "tests", "native", "stress_capture.cpp"),
                                    fake, "-Wl,-rpath," + str(tmp_path), "-ldl", "-o", exe],
                   check=True)
    # a small library with thread-local storage that the stress program keeps
    # loading and unloading, so that the interception library reloads its helper
    # every few milliseconds while client threads are calling into it
    helper = str(tmp_path / "liborion_tlsfresh.so")
    subprocess.run(["gcc", "-O2", "-fPIC", "-ftls-model=global-dynamic", "-shared",
                    os.path.join(CSRC, "capture", "tls_fresh_helper.c"), "-o", helper], check=True)
    churn_src = tmp_path / "churn.c"
    churn_src.write_text("static __thread long v;\nlong churn_touch(void) { return ++v; }\n")
    churn = str(tmp_path / "libchurn.so")
    subprocess.run(["gcc", "-O2", "-fPIC", "-shared", str(churn_src), "-o", churn], check=True)
    env = dict(os.environ, ORION_HIP_LIBRARY=fake, ORION_QUIET="1", FAKEHIP_ASYNC="1",
               ORION_TLS_REFRESH_LIBRARY=helper, STRESS_DLOPEN=churn,
               STRESS_EXPECT_TLS_RELOADS="2")
    env.pop("LD_PRELOAD", None)
    for seed in range(4):
        for clients, ahead in ((3, "0"), (3, "1"), (4, "1")):
            proc = subprocess.run([exe, str(tmp_path), str(clients), "60"],
                                  env=dict(env, ORION_BE_RUN_AHEAD=ahead, FAKEHIP_SEED=str(seed + 1)),
                                  capture_output=True, text=True, timeout=600)
            assert proc.returncode == 0, (seed, clients, ahead, proc.stdout + proc.stderr[-4000:])


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_capture_and_scheduler_under_address_and_undefined_behaviour_sanitizers(tmp_path):
    """The same stress program with AddressSanitizer and UBSan (host code only),
    the thread-local helper being reloaded under churn while clients run: a record
    read after its slot was reused, an argument copy past its buffer or a call into
    an unloaded helper copy would be reported here."""
    exe = str(tmp_path / "stress_asan")
    fake = str(tmp_path / "libfakehip_asan.so")
    common = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined",
              "-fno-omit-frame-pointer", "-fPIC", "-pthread",
              "-I" + os.path.join(ROOT, "include"), "-I/opt/rocm/include",
              "-I" + os.path.join(CSRC, "policy")]
    subprocess.run(common + ["-shared", os.path.join(ROOT, "tests", "fakehip", "fakehip.cpp"),
                             "-o", fake], check=True)
    srcs = [os.path.join(CSRC, p) for p in (
        "capture/capture.cpp", "capture/tls_fresh.cpp", "common/hip_api.cpp", "policy/policy.cpp",
        "policy/obslog.cpp",
        "scheduler/scheduler_eval.cpp", "scheduler/profile_capture.cpp")]
    subprocess.run(common + srcs + [os.path.join(ROOT, "tests", "native", "stress_capture.cpp"),
                                    fake, "-Wl,-rpath," + str(tmp_path), "-ldl", "-o", exe],
                   check=True)
    helper = str(tmp_path / "liborion_tlsfresh.so")
    subprocess.run(["gcc", "-O2", "-fPIC", "-ftls-model=global-dynamic", "-shared",
                    os.path.join(CSRC, "capture", "tls_fresh_helper.c"), "-o", helper], check=True)
    churn_src = tmp_path / "churn.c"
    churn_src.write_text("static __thread long v;\nlong churn_touch(void) { return ++v; }\n")
    churn = str(tmp_path / "libchurn.so")
    subprocess.run(["gcc", "-O2", "-fPIC", "-shared", str(churn_src), "-o", churn], check=True)
    env = dict(os.environ, ORION_HIP_LIBRARY=fake, ORION_QUIET="1",
               ORION_TLS_REFRESH_LIBRARY=helper, STRESS_DLOPEN=churn,
               STRESS_EXPECT_TLS_RELOADS="2",
               ASAN_OPTIONS="detect_leaks=0 abort_on_error=0 exitcode=67",
               UBSAN_OPTIONS="halt_on_error=1 exitcode=68 print_stacktrace=1")
    env.pop("LD_PRELOAD", None)
    for clients, ahead, later in ((3, "1", "0"), (4, "1", "1"), (3, "0", "1")):
        proc = subprocess.run([exe, str(tmp_path), str(clients), "40"],
                              env=dict(env, ORION_BE_RUN_AHEAD=ahead, FAKEHIP_ASYNC=later),
                              capture_output=True, text=True, timeout=600)
        assert "ERROR: AddressSanitizer" not in proc.stderr, proc.stderr[-4000:]
        assert "runtime error:" not in proc.stderr, proc.stderr[-4000:]
        assert proc.returncode == 0, proc.stdout + proc.stderr[-4000:]
