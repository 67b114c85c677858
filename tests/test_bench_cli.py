"""bench.py's command-line contract and its housekeeping, without a GPU."""

import importlib.util
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                          capture_output=True, text=True, timeout=120)
    assert proc.returncode != 0
    assert "one GPU" in (proc.stdout + proc.stderr) or "1 GPU" in (proc.stdout + proc.stderr)


def test_children_still_alive_at_the_end_are_ended_by_process_id():
    bench = _bench()
    assert bench.own_children() == []
    child = subprocess.Popen(["sleep", "100"])
    try:
        assert bench.own_children() == [child.pid]
        assert bench.end_own_children(grace_s=1.0) == 1
        assert bench.own_children() == []
    finally:
        if child.poll() is None:
            child.kill()
    assert bench.end_own_children() == 0
