"""Profile generation for gfx950: CU need, bound class, and the order-join of a
rocprofv3 trace with a captured profile.  Closed-form cases; the reference's
counterparts are profiling/postprocessing/get_num_blocks.py:34-52 and
roofline_analysis.py:37-71."""

import os

import pytest

from orion_amd.profiling import cu_need, rocprof


def test_workgroups_per_cu_closed_forms():
    # 256 threads = 4 waves; 32 wave slots per CU -> 8 workgroups
    assert cu_need.workgroups_per_cu(256) == 8
    # 128 VGPRs -> 512/128 = 4 waves per SIMD -> 16 waves -> 4 workgroups of 4 waves
    assert cu_need.workgroups_per_cu(256, regs_per_thread=128) == 4
    # 512 registers (256 arch + 256 acc): one wave per SIMD -> one workgroup
    assert cu_need.workgroups_per_cu(256, regs_per_thread=512) == 1
    # LDS: 128 KiB per workgroup of the 160 KiB -> one workgroup
    assert cu_need.workgroups_per_cu(256, lds_per_block=128 * 1024) == 1
    assert cu_need.workgroups_per_cu(256, lds_per_block=40 * 1024) == 4
    # single-wave workgroups are capped by the 32 workgroup slots
    assert cu_need.workgroups_per_cu(64) == 32
    # 1024 threads = 16 waves -> two workgroups
    assert cu_need.workgroups_per_cu(1024) == 2


def test_cu_needed_closed_forms():
    assert cu_need.cu_needed(2048, 256) == 256          # the triad's chunked grid
    assert cu_need.cu_needed(1024, 256, 512, 131072) == 1024   # the GEMM: one tile per CU
    assert cu_need.cu_needed(1, 64) == 1
    assert cu_need.cu_needed(33, 64) == 2
    assert cu_need.cu_needed(0, 256) == 1               # never below one


def test_classify_by_counters_and_by_name():
    assert cu_need.classify("whatever", hbm_fraction=0.7, mfma_fraction=0.0) == 0
    assert cu_need.classify("whatever", hbm_fraction=0.1, mfma_fraction=0.65) == 1
    assert cu_need.classify("whatever", hbm_fraction=0.1, mfma_fraction=0.1) == -1
    assert cu_need.classify("igemm_fwd_gtcx35_nhwc_bf16") == 1
    assert cu_need.classify("void at::native::vectorized_elementwise_kernel") == 0
    assert cu_need.classify("mystery") == -1


def test_classify_roofline_closed_forms():
    # the two co-location kernels at their benchmark sizes
    triad = cu_need.classify_roofline(bytes_moved=3 * 2 ** 30,
                                      vector_fp32_flops=2.0 * 2 ** 28)
    gemm = cu_need.classify_roofline(bytes_moved=402.7e6, mfma_bf16_flops=2.0 * 8192 ** 3)
    assert (triad, gemm) == (0, 1)
    # exactly at the bf16 knee (2.5e15 / 8e12 = 312.5 flop/byte): not right of it
    assert cu_need.classify_roofline(1.0e6, mfma_bf16_flops=312.5e6) == 0
    assert cu_need.classify_roofline(1.0e6, mfma_bf16_flops=313.0e6) == 1
    # no floating point at all: utilisation decides, else unknown
    assert cu_need.classify_roofline(1e6, hbm_fraction=0.8, mfma_fraction=0.0) == 0
    assert cu_need.classify_roofline(1e6, hbm_fraction=0.2, mfma_fraction=0.0) == -1


def test_short_name_matches_the_capture_layer():
    f = rocprof.short_name
    assert f("void at::native::(anonymous namespace)::max_pool_forward_nchw<float>(int)") == \
        "void at::native::max_pool_forward_nchw"
    assert f("igemm_fwd_gtcx35_nhwc_bf16_bx0") == "igemm_fwd_gtcx35_nhwc_bf16_bx0"
    assert f("void k<a, b>(c)") == "void k"


def _write_csv(path, header, rows):
    os.makedirs(os.path.dirname(path), exist_ok=True)
    with open(path, "w") as f:
        f.write(",".join(f'"{h}"' for h in header) + "\n")
        for r in rows:
            f.write(",".join(f'"{x}"' for x in r) + "\n")


def test_order_join_of_trace_and_profile(tmp_path):
    names = ["void at::native::vectorized_elementwise_kernel", "Cijk_gemm", "copy_k"]
    prof = tmp_path / "p_fwd"
    prof.write_text("Name,Profile,Memory_footprint,SM_usage,Duration\n" +
                    "".join(f"{n},-1,0,1,1000\n" for n in names))
    hdr = ["Kind", "Dispatch_Id", "Kernel_Name", "Start_Timestamp", "End_Timestamp",
           "LDS_Block_Size", "VGPR_Count", "Accum_VGPR_Count", "Workgroup_Size_X",
           "Workgroup_Size_Y", "Workgroup_Size_Z", "Grid_Size_X", "Grid_Size_Y", "Grid_Size_Z"]
    full = ["void at::native::vectorized_elementwise_kernel<4, f>(int)", "Cijk_gemm", "copy_k(float*)"]
    rows, d, t = [], 0, 0
    rows.append(["KERNEL_DISPATCH", (d := d + 1), "warmup_only_kernel", 0, 10, 0, 8, 0, 64, 1, 1, 64, 1, 1])
    for it in range(3):
        for k, n in enumerate(full):
            rows.append(["KERNEL_DISPATCH", (d := d + 1), n, t, t + 1000 * (k + 1) + it, 0,
                         32, 0, 256, 1, 1, 256 * 100, 1, 1])
            t += 10_000
            if k == 0:   # a runtime-internal fill between user kernels is ignored
                rows.append(["KERNEL_DISPATCH", (d := d + 1), "__amd_rocclr_fillBufferAligned",
                             t, t + 5, 0, 8, 0, 256, 1, 1, 256, 1, 1])
    _write_csv(str(tmp_path / "r" / "trace" / "t_kernel_trace.csv"), hdr, rows)
    stats = rocprof.merge(str(prof), str(tmp_path / "r"), str(tmp_path / "out"))
    assert stats["iterations_joined"] == 3 and stats["rows"] == 3
    out = (tmp_path / "out").read_text().splitlines()
    assert out[0] == "Name,Profile,Memory_footprint,SM_usage,Duration"
    # median duration over the three iterations; CU need = 100 workgroups / 8 per CU
    assert out[1] == f"{names[0]},0,0,13,1001"
    assert out[2] == f"{names[1]},1,0,13,2001"
    assert out[3].startswith(f"{names[2]},0,0,13,3001")


TRACE_HDR = ["Kind", "Dispatch_Id", "Kernel_Name", "Start_Timestamp", "End_Timestamp",
             "LDS_Block_Size", "VGPR_Count", "Accum_VGPR_Count", "Workgroup_Size_X",
             "Workgroup_Size_Y", "Workgroup_Size_Z", "Grid_Size_X", "Grid_Size_Y", "Grid_Size_Z"]
COUNTER_HDR = ["Dispatch_Id", "Kernel_Name", "Counter_Name", "Counter_Value"]


def _counter_runs(tmp_path, kernels, iterations=2):
    """kernels: [(name, duration_ns, fetch_units, write_units, mfma %, valu %)] per
    iteration, written as the five rocprofv3 runs ``merge`` reads."""
    trace, t, d = [], 0, 0
    counters = {"fetch": [], "write": [], "mfma": [], "valu": []}
    for _ in range(iterations):
        for name, ns, fetch, write, mfma, valu in kernels:
            d += 1
            trace.append(["KERNEL_DISPATCH", d, name, t, t + ns, 0, 32, 0, 256, 1, 1, 25600, 1, 1])
            t += ns + 1000
            for key, cname, value in (("fetch", "FETCH_SIZE", fetch), ("write", "WRITE_SIZE", write),
                                      ("mfma", "MfmaUtil", mfma), ("valu", "VALUBusy", valu)):
                counters[key].append([d, name, cname, value])
    root = tmp_path / "r"
    _write_csv(str(root / "trace" / "t_kernel_trace.csv"), TRACE_HDR, trace)
    for key, rows in counters.items():
        _write_csv(str(root / key / "t_counter_collection.csv"), COUNTER_HDR, rows)
    return str(root)


def test_classes_from_counters_per_kernel_name(tmp_path):
    """Closed forms.  The class of a row is the class of its kernel NAME over all
    its dispatches: traffic / time against 8000 B/ns on one side, the matrix-core
    busy fraction on the other; the vector-ALU busy fraction counts only for a
    convolution or GEMM family (by name)."""
    kernels = [
        # 1 ms moving 4 GB (fetch unit 2 KiB, write unit 1 KiB): 0.5 of HBM; MFMA 10 % -> memory
        ("stream_k", 1_000_000, 1_000_000, 1_952_125, 10.0, 3.0),
        # MFMA 82 % against 0.3 of HBM -> compute
        ("gemm_k", 1_000_000, 1_000_000, 352_000, 82.0, 25.0),
        # no matrix cores, vector ALUs 87 %, almost no traffic, and a name that says
        # nothing: busy vector ALUs alone decide nothing -> unknown
        ("valu_k", 100_000, 10, 10, 0.0, 87.0),
        # the same figures under a convolution's name -> compute
        ("naive_conv_k", 100_000, 10, 10, 0.0, 87.0),
        # a tiny dispatch of stream_k with nothing measurable on its own: it takes
        # the class of its family
        ("stream_k", 2_000, 0, 0, 0.0, 0.0),
        # neither resource reaches 5 % -> unknown
        ("idle_k", 50_000, 100, 100, 1.0, 2.0),
    ]
    prof = tmp_path / "p_fwd"
    prof.write_text("Name,Profile,Memory_footprint,SM_usage,Duration\n" +
                    "".join(f"{k[0]},-1,0,1,1\n" for k in kernels))
    rdir = _counter_runs(tmp_path, kernels)
    stats = rocprof.merge(str(prof), rdir, str(tmp_path / "out"), use_name_hints=False)
    out = [l.split(",") for l in (tmp_path / "out").read_text().splitlines()[1:]]
    assert [int(r[1]) for r in out] == [0, 1, -1, 1, 0, -1]
    assert stats["from_counters"] == 6 and stats["from_names"] == 0 and stats["unknown"] == 2
    assert abs(stats["unknown_time_fraction"] - 150_000 / 2_252_000) < 1e-9
    import json
    classes = json.loads((tmp_path / "out.classes.json").read_text())
    fam = classes["stream_k"]
    assert fam["dispatches"] == 2 and fam["source"] == "counters"
    want = (1_000_000 * 2048.0 + 1_952_125 * 1024.0) / 1_002_000 / 8000.0
    assert abs(fam["memory_fraction"] - want) < 1e-12
    assert abs(fam["mfma_fraction"] - 0.10 * 1_000_000 / 1_002_000) < 1e-12
    # the table built from this profile alone says the same
    table = rocprof.build_table([str(tmp_path / "out.classes.json")], str(tmp_path / "table.json"))
    assert {k: v["class"] for k, v in table.items()} == {
        "stream_k": 0, "gemm_k": 1, "valu_k": -1, "naive_conv_k": 1, "idle_k": -1}


def test_class_boundaries():
    f = rocprof.classify_utilisation
    assert f(0.049, 0.049) == -1            # neither roof within reach
    assert f(0.05, 0.0) == 0 and f(0.0, 0.05) == 1
    assert f(0.30, 0.30) == 0               # a tie is not "right of the knee"
    assert f(0.30, 0.31) == 1


def test_busy_vector_alus_alone_do_not_make_a_kernel_compute_bound():
    """VALUBusy counts address arithmetic and issue time: data movers reach
    0.3-0.6 of it.  With the matrix cores idle it decides only for convolution
    and GEMM families (by name); the fractions below are the ones measured on
    the MI355X and kept in the committed table."""
    import json
    f = rocprof.classify_utilisation
    table = json.load(open(cu_need.CLASS_TABLE_PATH))
    movers = ["void at::native::CatArrayBatchedCopy", "void at::native::indexFuncLargeIndex",
              "void at::native::max_pool_backward_nchw", "void at::native::max_pool_forward_nchw",
              "void at::native::vectorized_layer_norm_kernel"]
    for name in movers:
        e = table[name]
        assert e["valu_fraction"] > e["memory_fraction"] and e["mfma_fraction"] == 0.0, name
        assert f(e["memory_fraction"], e["mfma_fraction"], e["valu_fraction"], name) == 0, name
        assert e["class"] == 0, name
    # MIOpen's Winograd and naive convolutions do their FMAs on the vector ALUs
    for name in ("miopenSp3AsmConv_v30_3_1_gfx9_fp32_f3x2_stride2",
                 "naive_conv_ab_nonpacked_fwd_nchw_float_double_float"):
        e = table[name]
        assert e["mfma_fraction"] == 0.0 and e["class"] == 1, name
        assert f(e["memory_fraction"], e["mfma_fraction"], e["valu_fraction"], name) == 1
    # no name, or a name outside those families: the vector ALUs do not count
    assert f(0.28, 0.0, 0.57) == 0 and f(0.02, 0.0, 0.57, "some_copy_kernel") == -1
    # every entry of the table carries the class its own fractions give
    for name, e in table.items():
        if "memory_fraction" in e:
            assert e["class"] == f(e["memory_fraction"], e["mfma_fraction"],
                                   e["valu_fraction"], name), name


def test_the_flop_counter_pass_is_refused(tmp_path):
    """Eight SQ counters in one pass over a training client hung the profiler on
    the MI355X box: neither collected nor consumed."""
    with pytest.raises(ValueError, match="made no progress"):
        rocprof.collect("job.json", 0, str(tmp_path), passes=["flops"])
    with pytest.raises(ValueError, match="unknown pass"):
        rocprof.collect("job.json", 0, str(tmp_path), passes=["everything"])
    prof = tmp_path / "p"
    prof.write_text("Name,Profile,Memory_footprint,SM_usage,Duration\nA,-1,0,1,1\n")
    os.makedirs(tmp_path / "r" / "flops")
    with pytest.raises(ValueError, match="flops/ directory is not used"):
        rocprof.merge(str(prof), str(tmp_path / "r"), str(tmp_path / "o"))


def test_measured_class_table_comes_before_name_hints(tmp_path, monkeypatch):
    import json
    table = tmp_path / "t.json"
    table.write_text(json.dumps({"void at::native::vectorized_elementwise_kernel": {"class": 1},
                                 "mystery": {"class": 0}}))
    monkeypatch.setattr(cu_need, "CLASS_TABLE_PATH", str(table))
    monkeypatch.setattr(cu_need, "_class_table", None)
    assert cu_need.classify_source("mystery") == (0, "counters")
    assert cu_need.classify_source("void at::native::vectorized_elementwise_kernel") == (1, "counters")
    assert cu_need.classify_source("Cijk_gemm") == (1, "name")
    assert cu_need.classify_source("nothing_known") == (-1, "none")
    monkeypatch.setattr(cu_need, "_class_table", None)


def test_order_join_refuses_a_different_kernel_sequence(tmp_path):
    prof = tmp_path / "p_fwd"
    prof.write_text("Name,Profile,Memory_footprint,SM_usage,Duration\nA,-1,0,1,1\nB,-1,0,1,1\n")
    hdr = ["Kind", "Dispatch_Id", "Kernel_Name", "Start_Timestamp", "End_Timestamp",
           "LDS_Block_Size", "VGPR_Count", "Accum_VGPR_Count", "Workgroup_Size_X",
           "Workgroup_Size_Y", "Workgroup_Size_Z", "Grid_Size_X", "Grid_Size_Y", "Grid_Size_Z"]
    rows = [["KERNEL_DISPATCH", 1, "A", 0, 1, 0, 8, 0, 64, 1, 1, 64, 1, 1],
            ["KERNEL_DISPATCH", 2, "C", 2, 3, 0, 8, 0, 64, 1, 1, 64, 1, 1]]
    _write_csv(str(tmp_path / "r" / "trace" / "t_kernel_trace.csv"), hdr, rows)
    with pytest.raises(RuntimeError, match="does not end with"):
        rocprof.merge(str(prof), str(tmp_path / "r"), str(tmp_path / "out"))


def test_trace_summary_cuts_requests_from_the_end(tmp_path):
    """Closed form: a thread with 2 + 100 x 3 kernels of 1, 2, 3 us per request
    (the first two are start-up), another thread with 5 kernels."""
    from orion_amd.profiling import trace_summary
    path = tmp_path / "kt_kernel_trace.csv"
    rows = ["Kind,Agent_Id,Queue_Id,Stream_Id,Thread_Id,Dispatch_Id,Kernel_Id,Kernel_Name,"
            "Correlation_Id,Start_Timestamp,End_Timestamp"]
    t = 1000
    for d in (50_000, 60_000):                      # start-up kernels, cut off
        rows.append(f"KERNEL_DISPATCH,0,1,0,77,0,0,k,0,{t},{t + d}")
        t += d + 100
    for req in range(100):
        for d in (1000, 2000, 3000):
            rows.append(f"KERNEL_DISPATCH,0,{1 + req % 2},0,77,0,0,k,0,{t},{t + d}")
            t += d + 500
    for i in range(5):
        rows.append(f"KERNEL_DISPATCH,0,4,0,88,0,0,k,0,{i * 10},{i * 10 + 7}")
    path.write_text("\n".join(rows) + "\n")
    s = trace_summary.summarise(str(path), per_request=3, last=40)
    assert s["77"]["kernels"] == 302 and s["77"]["queues"] == [1, 2]
    assert s["77"]["groups"] == 40
    assert s["77"]["kernel_ms"] == {"p50": 0.006, "p99": 0.006, "mean": 0.006}
    assert s["77"]["span_ms"]["p50"] == 0.007        # 6 us of kernels + two 0.5 us gaps
    assert abs(s["77"]["sum_ms"] - (0.11 + 100 * 0.006)) < 1e-9
    assert s["88"] == {"kernels": 5, "sum_ms": 35 / 1e6, "mean_us": 0.007, "queues": [4]}


def test_profile_names_keep_clients_apart():
    """Two clients of one job share a profile only when they submit the same
    records: a HIP-graph client (one record per request) and the eager client of
    the same model, batch and dtype do not."""
    from orion_amd.profiling import capture_profile as cp
    eager = {"arch": "resnet50", "args": {"model_name": "resnet50", "batchsize": 4,
                                          "dtype": "bf16", "train": False}}
    graph = {"arch": "resnet50", "args": dict(eager["args"], hip_graph=True)}
    train = {"arch": "resnet50", "args": dict(eager["args"], train=True)}
    names = {cp.profile_name(e) for e in (eager, graph, train)}
    assert len(names) == 3 and cp.profile_name(eager) == "resnet50_4_bf16_inf"
    assert cp.profile_name({"arch": "bert", "args": {"batchsize": 8, "train": True}}) == \
        "bert_8_fp32_train"
