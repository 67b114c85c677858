"""The replay command line on committed recordings (tests/golden/)."""

import json
import os
import shutil
import subprocess
import sys

from orion_amd import replay

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden")


def _materialise(case, tmp_path):
    """A copy of a recording with its profile paths pointing at the copy."""
    d = tmp_path / case
    shutil.copytree(os.path.join(GOLDEN, case), d)
    obs = (d / "observations.log").read_text().replace("@DIR@", str(d))
    (d / "observations.log").write_text(obs)
    return str(d)


def test_replay_reproduces_a_recording_and_summarises_it(tmp_path):
    d = _materialise("mi355x_kernel_pair", tmp_path)
    proc = subprocess.run([sys.executable, "-m", "orion_amd.replay", d], cwd=ROOT,
                          capture_output=True, text=True, timeout=60)
    assert proc.returncode == 0, proc.stderr
    out = json.loads(proc.stdout)
    assert out["equals_recorded"] is True and out["algo"] == "orion" and out["clients"] == 2
    dec = open(os.path.join(d, "decisions.log")).read().splitlines()
    assert out["decisions"] == sum(1 for l in dec if l[:1] in "DFT")
    hp, be = out["per_client"][1], out["per_client"][0]
    assert hp["kernels"] == sum(1 for l in dec if l.startswith("D 1 1 k"))
    assert set(hp["by_cu_slot"]) == {"whole GPU"}
    assert sum(be["by_cu_slot"].values()) == be["kernels"] > 0
    assert be["stopped"] and not hp["stopped"]
    assert hp["iterations"] == sum(1 for l in dec if l.startswith("F 1 "))


def test_by_poll_output_lines_up_with_the_observation_log(tmp_path):
    d = _materialise("fake_orion_2be", tmp_path)
    proc = subprocess.run([sys.executable, "-m", "orion_amd.replay", d, "--by-poll"], cwd=ROOT,
                          capture_output=True, text=True, timeout=60)
    assert proc.returncode == 0, proc.stderr
    obs = open(os.path.join(d, "observations.log")).read()
    assert proc.stdout.splitlines().count("P") == sum(l.startswith("P ") for l in obs.splitlines())


def test_moved_profiles_and_a_tampered_log(tmp_path):
    d = _materialise("fake_reef_2be", tmp_path)
    moved = tmp_path / "elsewhere"
    moved.mkdir()
    for f in os.listdir(d):
        if f.endswith(".csv"):
            shutil.move(os.path.join(d, f), moved / f)
    obs, replayed, recorded = replay.check(d, profile_dir=str(moved))
    assert replayed == recorded
    # without the profiles the replay says what is missing
    proc = subprocess.run([sys.executable, "-m", "orion_amd.replay", d], cwd=ROOT,
                          capture_output=True, text=True, timeout=60)
    assert proc.returncode == 2 and "replay failed" in proc.stderr
    # a recorded decision log that differs is reported with exit status 1
    with open(os.path.join(d, "decisions.log"), "a") as f:
        f.write("T 0\n")
    proc = subprocess.run([sys.executable, "-m", "orion_amd.replay", d, "--profiles", str(moved)],
                          cwd=ROOT, capture_output=True, text=True, timeout=60)
    assert proc.returncode == 1 and json.loads(proc.stdout)["equals_recorded"] is False
