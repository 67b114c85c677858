"""Profile CSV parsing: oracle and native core against the reference's own
profile files (read in place when the reference tree is mounted) and against
the quirks std::stoi / std::stof have (reference:
src/scheduler/scheduler_eval.cpp:498-526)."""

import ctypes
import json
import os

import numpy as np
import pytest

from oracle import policy_oracle as po
from tests import jobs

# num_kernels the reference's own job files name for each profile
# (artifact_evaluation/fig7/config_files/*.json, benchmarking/*.json): the row
# count the scheduler must find.  max(SM_usage) and the duration sums are the
# per-file figures of the structural survey of the reference.
EXPECTED_ROWS = {
    "resnet50_4_fwd": 175, "mobilenetv2_4_fwd": 152, "resnet50_32_fb1": 946,
    "resnet50_32_fb0": 624, "mobilenetv2_64_fb1": 890, "bert_8_fb1": 4777,
    "bert_2_fwd": 572,
}
EXPECTED_MAX_SM = {"resnet50_4_fwd": 392, "resnet50_32_fb1": 12544,
                   "mobilenetv2_4_fwd": 882}
EXPECTED_SUM_MS = {"resnet50_4_fwd": 6.498, "mobilenetv2_4_fwd": 2.263,
                   "resnet50_32_fb1": 95.28, "mobilenetv2_64_fb1": 74.90,
                   "bert_8_fb1": 190.77, "bert_2_fwd": 48.63}


def native_stats(path):
    lib = jobs.policy_lib()
    rows, mx = ctypes.c_int(), ctypes.c_int()
    total, err = ctypes.c_double(), ctypes.c_void_p()
    rc = lib.orion_profile_stats(path.encode(), ctypes.byref(rows),
                                 ctypes.byref(mx), ctypes.byref(total),
                                 ctypes.byref(err))
    msg = ctypes.string_at(err).decode() if err else ""
    lib.orion_policy_free(err)
    return rc, rows.value, mx.value, total.value, msg


def native_row(path, row):
    lib = jobs.policy_lib()
    name = ctypes.create_string_buffer(256)
    prof, mem, sm = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    dur = ctypes.c_float()
    rc = lib.orion_profile_row(path.encode(), row, name, 256, ctypes.byref(prof),
                               ctypes.byref(mem), ctypes.byref(sm),
                               ctypes.byref(dur))
    return rc, name.value.decode(), prof.value, mem.value, sm.value, dur.value


def test_reference_profile_files(reference_root):
    d = os.path.join(reference_root, "benchmarking", "model_kernels")
    files = sorted(os.listdir(d))
    assert len(files) == 19
    for name in files:
        path = os.path.join(d, name)
        ops = po.parse_profile(path)
        rc, rows, mx, total, msg = native_stats(path)
        assert rc == 0, msg
        assert rows == len(ops)
        assert mx == po.max_sm_used(ops)
        assert total == pytest.approx(sum(float(o.duration) for o in ops), rel=1e-12)
        if name in EXPECTED_ROWS:
            assert rows == EXPECTED_ROWS[name], name
        if name in EXPECTED_MAX_SM:
            assert mx == EXPECTED_MAX_SM[name], name
        if name in EXPECTED_SUM_MS:
            assert total / 1e6 == pytest.approx(EXPECTED_SUM_MS[name], abs=6e-3), name
        for r in (0, len(ops) // 2, len(ops) - 1):
            rc, nm, prof, mem, sm, dur = native_row(path, r)
            o = ops[r]
            assert (rc, nm, prof, mem, sm) == (0, o.name, o.profile, o.mem, o.sm_used)
            assert np.float32(dur) == o.duration
    # first-iteration placeholder files: every row is -1,1,1,7
    for o in po.parse_profile(os.path.join(d, "resnet50_32_fb0")):
        assert (o.profile, o.mem, o.sm_used, float(o.duration)) == (-1, 1, 1, 7.0)


def test_reference_job_files_name_existing_row_counts(reference_root):
    """Every kernel_file/num_kernels pair of the reference's fig7 configs
    matches the row count of the profile of the same base name."""
    cfg_dir = os.path.join(reference_root, "artifact_evaluation", "fig7",
                           "config_files")
    prof_dir = os.path.join(reference_root, "benchmarking", "model_kernels")
    checked = 0
    for f in sorted(os.listdir(cfg_dir)):
        if not f.endswith(".json"):
            continue
        with open(os.path.join(cfg_dir, f)) as fh:
            cfg = json.load(fh)
        for entry in cfg:
            for key_file, key_n in (("kernel_file", "num_kernels"),
                                    ("additional_kernel_file",
                                     "additional_num_kernels")):
                if key_file not in entry:
                    continue
                path = os.path.join(prof_dir, os.path.basename(entry[key_file]))
                if not os.path.exists(path):
                    continue
                assert len(po.parse_profile(path)) == entry[key_n], (f, path)
                checked += 1
    assert checked >= 10


def test_field_conversion_quirks(tmp_path):
    p = str(tmp_path / "q.csv")
    with open(p, "w") as f:
        f.write("Name,Profile,Memory_footprint,SM_usage,Duration\n")
        f.write("void at::native::kernel<int, float>(x),1,0,98,100480\n".replace(
            "<int, float>", "<int>"))
        f.write("a, -1 ,  7,12abc,3.5e3xyz\n")      # stoi/stof take a prefix
        f.write("b,+0,0,16777217,16777217\n")       # fp32 rounds the duration
        f.write("c,1,2,3,.25,extra,columns\n")
    ops = po.parse_profile(p)
    assert [o.profile for o in ops] == [1, -1, 0, 1]
    assert [o.mem for o in ops] == [0, 7, 0, 2]
    assert [o.sm_used for o in ops] == [98, 12, 16777217, 3]
    assert [float(o.duration) for o in ops] == [100480.0, 3500.0, 16777216.0, 0.25]
    rc, rows, mx, total, msg = native_stats(p)
    assert (rc, rows, mx) == (0, 4, 16777217)
    for r, o in enumerate(ops):
        got = native_row(p, r)
        assert got[1:5] == (o.name, o.profile, o.mem, o.sm_used)
        assert np.float32(got[5]) == o.duration


def test_malformed_profiles_are_rejected_not_guessed(tmp_path):
    p = str(tmp_path / "bad.csv")
    with open(p, "w") as f:
        f.write("Name,Profile,Memory_footprint,SM_usage,Duration\nconv,1,0\n")
    rc, *_rest, msg = native_stats(p)
    assert rc == 2 and "row 2" in msg
    rc, *_rest, msg = native_stats(str(tmp_path / "missing.csv"))
    assert rc == 2 and "cannot open" in msg
    with pytest.raises((IndexError, ValueError)):
        po.parse_profile(p)


def test_cu_slot_placement_matches_oracle():
    from oracle import obslog
    lib = jobs.policy_lib()
    masks = [32, 64, 128, 256]
    arr = (ctypes.c_int * 4)(*masks)
    cls_id = {po.KERNEL: 0, po.MEMCPY: 1, po.MALLOC: 2, po.FREE: 3, po.MEMSET: 4}
    for algo_id, algo in enumerate([po.ALGO_ORION, po.ALGO_REEF,
                                    po.ALGO_SEQUENTIAL]):
        for cls in po.ALL_CLASSES:
            for sm in [0, 1, 32, 33, 64, 65, 128, 129, 256, 257, 12544]:
                for active in (False, True):
                    for long_k in (False, True):
                        want = obslog.place_cu_slot(masks, cls, sm, algo, active, long_k)
                        got = lib.orion_place_cu_slot(arr, 4, cls_id[cls], sm, algo_id,
                                                      int(active), int(long_k))
                        assert got == want
    # hand-worked: idle -> whole GPU; active -> smallest mask that holds the
    # need, capped below the whole GPU; a single mask leaves no choice
    place = obslog.place_cu_slot
    assert place(masks, po.KERNEL, 33, po.ALGO_ORION, False) == 3
    assert place(masks, po.KERNEL, 33, po.ALGO_ORION, True) == 1
    # a kernel that alone outlasts the duration budget never gets every CU
    assert place(masks, po.KERNEL, 33, po.ALGO_ORION, False, True) == 2
    assert place(masks, po.KERNEL, 33, po.ALGO_ORION, True, True) == 1
    assert place([256], po.KERNEL, 33, po.ALGO_ORION, False, True) == 0
    assert place(masks, po.KERNEL, 33, po.ALGO_REEF, False, True) == 3
    assert place(masks, po.KERNEL, 4000, po.ALGO_ORION, True) == 2
    assert place(masks, po.KERNEL, 1, po.ALGO_ORION, True) == 0
    assert place(masks, po.MEMCPY, 1, po.ALGO_ORION, True) == -1
    assert place([256], po.KERNEL, 4000, po.ALGO_ORION, True) == 0
    assert place(masks, po.KERNEL, 1, po.ALGO_REEF, True) == 3
