"""Replay of a recorded scheduler run through the native policy core.

A run with ``ORION_RECORD_DIR=<dir>`` leaves ``observations.log`` (what every
effective poll of the scheduler saw: stop acknowledgements, queue heads, event
answers, iteration times) and ``decisions.log`` (what it dispatched, released
and stopped).  The policy is a pure function of the observations, so the run
can be re-decided offline, on any host, from the log and the profile files it
names:

    python -m orion_amd.replay <dir>            # check + summary
    python -m orion_amd.replay <dir> --by-poll  # print decisions poll by poll

The reference has no counterpart (its loop, scheduler_eval.cpp:277-487, keeps no
trace); the formats are described in ``orion_amd/csrc/policy/obslog.h``.
"""

import argparse
import ctypes
import json
import os
import sys

from . import _lib


class ReplayError(RuntimeError):
    pass


def native_replay(observations, by_poll=False, sequential_fix=True):
    """Decision log (text) the native core produces for an observation log."""
    lib = _lib.load(_lib.POLICY_LIB)
    fn = lib.orion_policy_replay_by_poll if by_poll else lib.orion_policy_replay
    fn.argtypes = [ctypes.c_char_p, ctypes.c_int, ctypes.POINTER(ctypes.c_void_p),
                   ctypes.POINTER(ctypes.c_void_p)]
    fn.restype = ctypes.c_int
    lib.orion_policy_free.argtypes = [ctypes.c_void_p]
    lib.orion_policy_free.restype = None
    out, err = ctypes.c_void_p(), ctypes.c_void_p()
    rc = fn(observations.encode(), int(sequential_fix), ctypes.byref(out), ctypes.byref(err))
    try:
        if rc != 0:
            raise ReplayError(ctypes.string_at(err).decode() if err else f"status {rc}")
        return ctypes.string_at(out).decode()
    finally:
        lib.orion_policy_free(out)
        lib.orion_policy_free(err)


def summarise(observations, decisions):
    """Counts per client of a decision log: dispatches by record class and by
    CU slot, iterations released, stops raised; and the number of logged polls."""
    lines = observations.splitlines()
    header = lines[0].split(" ")
    n, masks = int(header[1]), [int(m) for m in header[3].split(",")]
    clients = [{"kernels": 0, "memory_records": 0, "by_cu_slot": {}, "iterations": 0,
                "stopped": False} for _ in range(n)]
    for line in decisions.splitlines():
        p = line.split(" ")
        if p[0] == "D":
            c = clients[int(p[1])]
            if p[3] == "k":
                c["kernels"] += 1
                width = masks[int(p[6])] if 0 <= int(p[6]) < len(masks) else None
                key = "whole GPU" if int(p[1]) == n - 1 else f"{width} CUs"
                c["by_cu_slot"][key] = c["by_cu_slot"].get(key, 0) + 1
            else:
                c["memory_records"] += 1
        elif p[0] == "F":
            clients[int(p[1])]["iterations"] += 1
        elif p[0] == "T":
            clients[int(p[1])]["stopped"] = True
    segments = [l.split(" ") for l in lines if l.startswith("S ")]
    return {"clients": n, "max_sms": int(header[2]), "be_cu_masks": masks,
            "algo": segments[0][3] if segments else None,
            "budget": int(segments[0][4]) if segments else None,
            "schedule_calls": len(segments),
            "polls": sum(1 for l in lines if l.startswith("P ")),
            "decisions": sum(1 for l in decisions.splitlines() if l[:1] in "DFT"),
            "per_client": clients}


def check(record_dir, profile_dir=None):
    """Replays ``record_dir`` and compares with what the live scheduler wrote.
    ``profile_dir``: where the profile files are now, if they have moved."""
    with open(os.path.join(record_dir, "observations.log")) as f:
        obs = f.read()
    if profile_dir:
        moved = []
        for line in obs.splitlines():
            p = line.split(" ")
            if p[0] == "K":
                p[5] = os.path.join(profile_dir, os.path.basename(" ".join(p[5:])))
                line = " ".join(p[:6])
            elif p[0] == "X":
                p[3] = os.path.join(profile_dir, os.path.basename(" ".join(p[3:])))
                line = " ".join(p[:4])
            moved.append(line)
        obs = "\n".join(moved) + "\n"
    replayed = native_replay(obs)
    recorded_path = os.path.join(record_dir, "decisions.log")
    recorded = open(recorded_path).read() if os.path.exists(recorded_path) else None
    return obs, replayed, recorded


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("record_dir")
    ap.add_argument("--profiles", help="directory the profile files are in now")
    ap.add_argument("--by-poll", action="store_true",
                    help="print the decisions with a line P before every poll's")
    a = ap.parse_args(argv)
    try:
        obs, replayed, recorded = check(a.record_dir, a.profiles)
    except ReplayError as e:
        print(f"replay failed: {e}", file=sys.stderr)
        return 2
    if a.by_poll:
        sys.stdout.write(native_replay(obs, by_poll=True))
        return 0
    out = summarise(obs, replayed)
    out["equals_recorded"] = None if recorded is None else recorded == replayed
    print(json.dumps(out, indent=1))
    return 0 if recorded is None or recorded == replayed else 1


if __name__ == "__main__":
    sys.exit(main())
