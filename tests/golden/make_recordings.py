"""Writes the fixtures under tests/golden/: observation and decision logs that
the *live* native scheduler recorded, with the profile files they name.

    python tests/golden/make_recordings.py            # host-only recordings
    python tests/golden/make_recordings.py --gpu      # + the MI355X recording

* fake_<algo>_<n>be: the job protocol on the recording HIP stand-in
  (tests/fake_runner.py), one directory per policy;
* mi355x_kernel_pair: the small GEMM/triad pair through the real hot path on an
  MI355X (orion_amd/kernel_pair.py), profiles captured on the same GPU.

Directory names inside the logs are replaced by the token @DIR@ so that the
fixtures can be replayed from wherever the repository lies.
tests/test_golden_recordings.py replays every one of them with the CPU oracle and
with the native policy core and expects the recorded decisions, byte for byte.
"""

import os
import shutil
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)


def store(name, record_dir, profile_paths):
    out = os.path.join(HERE, name)
    shutil.rmtree(out, ignore_errors=True)
    os.makedirs(out)
    obs = open(os.path.join(record_dir, "observations.log")).read()
    for path in profile_paths:
        shutil.copyfile(path, os.path.join(out, os.path.basename(path)))
        # logs may name the file through a symlinked spelling of the same place
        for spelled in {path, os.path.realpath(path)}:
            obs = obs.replace(spelled, "@DIR@/" + os.path.basename(path))
    for line in obs.splitlines():
        if line[:2] in ("K ", "X ") and "@DIR@/" not in line:
            raise SystemExit(f"{name}: profile path not rewritten: {line}")
    open(os.path.join(out, "observations.log"), "w").write(obs)
    shutil.copyfile(os.path.join(record_dir, "decisions.log"),
                    os.path.join(out, "decisions.log"))
    print(name, len(obs.splitlines()), "observation lines")


def profiles_named(record_dir):
    names = []
    for line in open(os.path.join(record_dir, "observations.log")):
        parts = line.rstrip("\n").split(" ")
        if parts[0] == "K":
            names.append(" ".join(parts[5:]))
        elif parts[0] == "X":
            names.append(" ".join(parts[3:]))
    return sorted(set(names))


def main():
    for algo, n_be in (("orion", 2), ("reef", 2), ("sequential", 1)):
        with tempfile.TemporaryDirectory() as work:
            subprocess.run([sys.executable, os.path.join(ROOT, "tests", "fake_runner.py"),
                            work, algo, str(n_be), "14"], check=True,
                           stdout=subprocess.DEVNULL)
            store(f"fake_{algo}_{n_be}be", work, profiles_named(work))
    if "--gpu" in sys.argv:
        from orion_amd import kernel_pair
        with tempfile.TemporaryDirectory() as work:
            res = kernel_pair.run_child(small=True, check=True, workdir=work, hp_iters=30)
            assert res["outputs_match"]
            rec = os.path.join(work, "out_co")
            store("mi355x_kernel_pair", rec, profiles_named(rec))


if __name__ == "__main__":
    main()
