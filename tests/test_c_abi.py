"""Every function the public headers declare is exported by the library that
is supposed to hold it, and the libraries load on a host without a GPU."""

import ctypes
import os
import re

import pytest

from orion_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DECL = re.compile(r"^\s*(?:int|void\*?|void \*|bool)\s*\*?\s*([a-z_][a-z0-9_]*)\s*\(", re.M)


def declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(DECL.findall(text)))


CAPTURE_SYMBOLS = {"block", "stop", "orion_register_thread", "orion_register_stream",
                   "orion_client_index", "orion_client_of_stream", "orion_pinned_cpu",
                   "orion_thread_passthrough"}


def test_kernels_header():
    names = declared("orion_kernels.h")
    assert names == ["orion_gemm_bf16_nt", "orion_stream_create", "orion_stream_destroy",
                     "orion_triad_f32"]
    lib = _lib.load(_lib.KERNELS_LIB)
    for n in names:
        assert hasattr(lib, n)


def test_policy_header():
    names = declared("orion_policy.h")
    assert "orion_policy_replay" in names and "orion_policy_replay_by_poll" in names and len(names) == 6
    lib = _lib.load(_lib.POLICY_LIB)
    for n in names:
        assert hasattr(lib, n)


def test_scheduler_header():
    names = declared("orion_scheduler.h")
    for required in ("sched_init", "setup", "setup_change", "schedule", "reset",
                     "block", "stop"):      # the reference's own entry points
        assert required in names
    cap = _lib.load(_lib.CAPTURE_LIB)
    sched = _lib.load(_lib.SCHEDULER_LIB)
    for n in names:
        holder = cap if n in CAPTURE_SYMBOLS else sched
        assert hasattr(holder, n), n


def test_interposed_hip_symbols_are_exported():
    cap = _lib.load(_lib.CAPTURE_LIB)
    for n in ("hipLaunchKernel", "hipExtLaunchKernel", "hipModuleLaunchKernel",
              "hipExtModuleLaunchKernel", "hipHccModuleLaunchKernel",
              "hipModuleLaunchCooperativeKernel", "hipLaunchCooperativeKernel",
              "hipGraphLaunch",
              "hipMalloc", "hipFree", "hipMallocAsync", "hipFreeAsync", "hipMemcpy2D",
              "hipMemcpy", "hipMemcpyAsync",
              "hipMemcpyWithStream", "hipMemcpy2DAsync", "hipMemset",
              "hipMemsetAsync", "hipMemsetD32Async", "hipMemsetD16Async",
              "hipMemsetD8Async", "hipStreamSynchronize", "hipStreamQuery",
              "hipEventRecord", "hipStreamWaitEvent", "hipDeviceSynchronize",
              "hipLaunchHostFunc", "hipStreamWriteValue32", "hipStreamWriteValue64",
              "hipStreamWaitValue32", "hipStreamWaitValue64", "hipMemcpyToSymbol",
              "hipMemcpyToSymbolAsync", "hipMemcpyFromSymbol", "hipMemcpyFromSymbolAsync",
              "hipModuleUnload", "hipHostFree", "hipFreeHost"):
        assert hasattr(cap, n), n


def test_capture_library_does_not_link_a_hip_runtime():
    """It must bind to whatever runtime the process already carries."""
    import subprocess
    out = subprocess.run(["readelf", "-d", _lib.CAPTURE_LIB], capture_output=True,
                         text=True).stdout
    assert "libamdhip64" not in out
    out = subprocess.run(["readelf", "-d", _lib.SCHEDULER_LIB], capture_output=True,
                         text=True).stdout
    assert "libamdhip64" not in out and "libinttemp.so" in out


def test_missing_library_fails_loudly(tmp_path):
    with pytest.raises(_lib.NativeLibraryMissing):
        _lib.load(str(tmp_path / "nope.so"))


def test_control_calls_are_noops_when_not_armed():
    cap = _lib.load(_lib.CAPTURE_LIB)
    cap.block.argtypes = [ctypes.c_int]
    cap.block(0)               # returns at once: nothing is armed
    assert cap.stop() == 0
    assert cap.orion_client_index() == -1


def test_profiler_detection_counts_the_tool_library_only(monkeypatch):
    """The kernel library is unloaded at exit only under a profiler.  The HIP
    runtime maps librocprofiler-register.so in every process, so that library
    must not count as one (it did: the kernel library was then unloaded at the
    end of every run and never showed among the process's libraries)."""
    import torch  # noqa: F401  (maps the HIP runtime and what it depends on)
    from orion_amd import kernels
    monkeypatch.delenv("ROCP_TOOL_LIBRARIES", raising=False)
    monkeypatch.delenv("LD_PRELOAD", raising=False)
    assert not kernels._profiler_attached()
    monkeypatch.setenv("ROCP_TOOL_LIBRARIES", "/opt/rocm/lib/rocprofiler-sdk/librocprofiler-sdk-tool.so")
    assert kernels._profiler_attached()
