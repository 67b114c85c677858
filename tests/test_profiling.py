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
