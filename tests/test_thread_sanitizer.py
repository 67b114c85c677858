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
        "capture/capture.cpp", "common/hip_api.cpp", "policy/policy.cpp", "policy/obslog.cpp",
        "scheduler/scheduler_eval.cpp", "scheduler/profile_capture.cpp")]
    subprocess.run(common + srcs + [os.path.join(ROOT, "tests", "native", "stress_capture.cpp"),
                                    fake, "-Wl,-rpath," + str(tmp_path), "-ldl", "-o", exe],
                   check=True)
    env = dict(os.environ, ORION_HIP_LIBRARY=fake, ORION_QUIET="1",
               TSAN_OPTIONS="halt_on_error=1 exitcode=66 second_deadlock_stack=1")
    env.pop("LD_PRELOAD", None)
    # both hand-offs of the high-priority client: issuing its own calls and
    # queueing notices (default), and the synchronous hand-off of every record
    for clients, direct in ((2, "1"), (4, "1"), (3, "0")):
        proc = subprocess.run([exe, str(tmp_path), str(clients), "40"],
                              env=dict(env, ORION_HP_DIRECT=direct),
                              capture_output=True, text=True, timeout=600)
        assert "WARNING: ThreadSanitizer" not in proc.stderr, proc.stderr[-4000:]
        assert proc.returncode == 0, proc.stdout + proc.stderr[-4000:]
