"""Committed recordings of the live native scheduler (tests/golden/, written by
tests/golden/make_recordings.py: three policies on the recording HIP stand-in
and one run of the kernel pair on an MI355X) replayed by the CPU oracle and by
the native policy core: both must reproduce the recorded decisions byte for
byte, from the recorded observations and the profile files alone."""

import glob
import os

import pytest

from oracle import obslog
from tests import jobs

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
CASES = sorted(os.path.basename(os.path.dirname(p))
               for p in glob.glob(os.path.join(GOLDEN, "*", "observations.log")))


def test_fixtures_are_present():
    assert {"fake_orion_2be", "fake_reef_2be", "fake_sequential_1be",
            "mi355x_kernel_pair"} <= set(CASES)


@pytest.mark.parametrize("case", CASES)
def test_recording_replays_bit_exactly(case):
    d = os.path.join(GOLDEN, case)
    obs = open(os.path.join(d, "observations.log")).read().replace("@DIR@", d)
    dec = open(os.path.join(d, "decisions.log")).read()
    assert dec.count("\nD ") > 50
    assert obslog.replay(obs) == dec
    assert jobs.native_replay(obs) == dec


def test_a_changed_observation_changes_the_decisions():
    """The replay really depends on the log: completing one event earlier in the
    MI355X recording moves a release or a dispatch."""
    d = os.path.join(GOLDEN, "mi355x_kernel_pair")
    lines = open(os.path.join(d, "observations.log")).read().replace("@DIR@", d).splitlines()
    dec = open(os.path.join(d, "decisions.log")).read()
    changed = 0
    for i, line in enumerate(lines):
        p = line.split(" ")
        if p[0] == "P" and "0" in p[3] and p[3] != "-":
            lines[i] = " ".join(p[:3] + [p[3].replace("0", "1", 1)] + p[4:])
            try:
                if obslog.replay("\n".join(lines) + "\n") != dec:
                    changed += 1
            except obslog.ReplayDivergence:
                changed += 1
            break
    assert changed == 1
