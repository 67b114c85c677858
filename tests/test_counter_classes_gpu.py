"""Bound classes from hardware counters on the GPU: the rocprofv3 passes
(`orion_amd.profiling.rocprof.collect`) over the two hand-written kernels as
stand-alone clients, merged into their captured profiles with the name table
switched off.  The streaming triad must come out memory-bound (0) and the bf16
MFMA GEMM compute-bound (1) from the counters alone (reference: the class
column that profiling/postprocessing/roofline_analysis.py:37-71 derives from
Nsight Compute metrics)."""

import json
import os

import pytest

pytestmark = pytest.mark.gpu


def test_triad_and_gemm_classes_from_counters_alone(tmp_path):
    from orion_amd.profiling import capture_profile, rocprof
    work = str(tmp_path)
    # sizes that fill the GPU: 256 MiB per triad array, a 4096^3 GEMM (256 tiles)
    job = [
        {"arch": "triad_f32", "kernel_file": "", "num_kernels": 0, "num_iters": 6,
         "args": {"batchsize": 1 << 26, "rps": 0, "uniform": False, "dummy_data": True,
                  "train": True, "per_iter": 2}},
        {"arch": "gemm_bf16", "kernel_file": "", "num_kernels": 0, "num_iters": 6,
         "args": {"batchsize": 4096, "rps": 0, "uniform": False, "dummy_data": True,
                  "train": False, "per_iter": 2}},
    ]
    cfg = os.path.join(work, "job.json")
    with open(cfg, "w") as f:
        json.dump(job, f)
    filled = capture_profile.fill_job(cfg, os.path.join(work, "profiles"),
                                      os.path.join(work, "filled.json"), quiet=True)
    want = {0: 0, 1: 1}
    for idx, entry in enumerate(filled):
        profile = entry.get("additional_kernel_file", entry["kernel_file"])
        rdir = os.path.join(work, f"rocprof{idx}")
        rocprof.collect(cfg, idx, rdir, iters=6, timeout=120)
        out = os.path.join(work, f"merged{idx}")
        stats = rocprof.merge(profile, rdir, out, use_name_hints=False)
        assert stats["from_counters"] == stats["rows"] == 2 and stats["from_names"] == 0, stats
        rows = [l.split(",") for l in open(out).read().splitlines()[1:]]
        assert [int(r[1]) for r in rows] == [want[idx]] * 2, (rows, stats)
        classes = json.load(open(out + ".classes.json"))
        (name, fam), = classes.items()
        if idx == 0:      # the triad moves 12 bytes per element and computes one FMA
            assert fam["memory_fraction"] > 0.5 > fam["valu_fraction"] and fam["mfma_fraction"] == 0
        else:             # the GEMM keeps the matrix cores busy
            assert fam["mfma_fraction"] > 0.5 > fam["memory_fraction"]
        report_dir = os.environ.get("ORION_TEST_REPORT_DIR")
        if report_dir and os.path.isdir(report_dir):
            with open(os.path.join(report_dir, "counter_classes.jsonl"), "a") as f:
                f.write(json.dumps({"client": entry["arch"], "kernel": name, **fam, **stats}) + "\n")
