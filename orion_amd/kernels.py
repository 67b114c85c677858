"""ctypes bindings of liborion_kernels.so (the hand-written gfx950 kernels).

torch is used only as the owner of device memory and streams; the arithmetic
runs in the HIP kernels behind the C ABI declared in ``include/orion_kernels.h``.
"""

import atexit
import ctypes

import torch

from . import _lib

STATUS = {0: "ok", 1: "bad argument", 2: "shape not a multiple of the tile",
          3: "pointer not 16-byte aligned", 4: "launch rejected"}


class KernelError(RuntimeError):
    def __init__(self, name, code):
        super().__init__(f"{name}: {STATUS.get(code, code)}")
        self.code = code


def lib():
    handle = _lib.load(_lib.KERNELS_LIB)
    if not getattr(handle, "_orion_typed", False):
        handle.orion_triad_f32.argtypes = [
            ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float,
            ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p]
        handle.orion_triad_f32.restype = ctypes.c_int
        handle.orion_gemm_bf16_nt.argtypes = [
            ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
            ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
        handle.orion_gemm_bf16_nt.restype = ctypes.c_int
        handle.orion_stream_create.argtypes = [ctypes.c_int, ctypes.POINTER(ctypes.c_void_p)]
        handle.orion_stream_create.restype = ctypes.c_int
        handle.orion_stream_destroy.argtypes = [ctypes.c_void_p]
        handle.orion_stream_destroy.restype = ctypes.c_int
        handle._orion_typed = True
    return handle


_streams = []          # raw handles of the streams made here, destroyed at exit


def cu_masked_stream(cu_count, device=0):
    """A ``torch.cuda.ExternalStream`` over a stream limited to ``cu_count``
    compute units (the whole GPU for ``cu_count <= 0``)."""
    out = ctypes.c_void_p()
    rc = lib().orion_stream_create(int(cu_count), ctypes.byref(out))
    if rc != 0:
        raise KernelError("orion_stream_create", rc)
    _streams.append(out.value)
    return torch.cuda.ExternalStream(out.value, device=device)


def _profiler_attached():
    """True when a rocprofiler *tool* library is in this process: rocprofv3
    names it in ROCP_TOOL_LIBRARIES and LD_PRELOAD and it shows in the process's
    maps.  (``librocprofiler-register.so`` does not count: the HIP runtime maps
    it in every process, profiled or not.)"""
    import os
    named = os.environ.get("ROCP_TOOL_LIBRARIES", "") + ":" + os.environ.get("LD_PRELOAD", "")
    if "rocprofiler-sdk-tool" in named:
        return True
    try:
        with open("/proc/self/maps") as f:
            return any("rocprofiler-sdk-tool" in line for line in f)
    except OSError:
        return False


@atexit.register
def _shutdown():
    """Gives back what this module took from the HIP runtime while the runtime
    is still up: waits for the device and destroys the streams made here.  Under
    a profiler the kernel library is unloaded as well (which un-registers its
    code object): left to process exit, the library's own finaliser then runs
    after the interpreter and the profiler's hooks have shut down, and the
    process dies in it.  Without a profiler the library stays mapped until the
    process ends, so that whoever lists the process's libraries at exit sees it."""
    handle = _lib.loaded(_lib.KERNELS_LIB)
    if handle is None:
        return
    if torch.cuda.is_initialized():
        torch.cuda.synchronize()
    while _streams:
        handle.orion_stream_destroy(ctypes.c_void_p(_streams.pop()))
    if _profiler_attached():
        _lib.unload(_lib.KERNELS_LIB)


def _stream_ptr(stream):
    if stream is None:
        stream = torch.cuda.current_stream()
    return ctypes.c_void_p(stream.cuda_stream)


def _check_device(*tensors):
    for t in tensors:
        if not t.is_cuda:
            raise ValueError("orion_amd kernels take device tensors only")
        if not t.is_contiguous():
            raise ValueError("orion_amd kernels take contiguous tensors only")


def triad(a, b, c, s, grid_blocks=0, stream=None):
    """a = b + s * c (fp32, one FMA per element), in place into ``a``."""
    _check_device(a, b, c)
    if not (a.dtype == b.dtype == c.dtype == torch.float32):
        raise ValueError("triad is fp32")
    if not (a.numel() == b.numel() == c.numel()):
        raise ValueError("triad operands differ in length")
    rc = lib().orion_triad_f32(a.data_ptr(), b.data_ptr(), c.data_ptr(),
                               ctypes.c_float(s), a.numel(), grid_blocks,
                               _stream_ptr(stream))
    if rc != 0:
        raise KernelError("orion_triad_f32", rc)
    return a


def gemm_bf16_nt(a, b, out=None, out_dtype=torch.bfloat16, stream=None):
    """out[M,N] = a[M,K] @ b[N,K].T with bf16 inputs and fp32 accumulation."""
    _check_device(a, b)
    if a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16:
        raise ValueError("gemm_bf16_nt takes bf16 operands")
    if a.dim() != 2 or b.dim() != 2 or a.shape[1] != b.shape[1]:
        raise ValueError("gemm_bf16_nt wants a[M,K] and b[N,K]")
    m, k = a.shape
    n = b.shape[0]
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=a.device)
    _check_device(out)
    if out.shape != (m, n) or out.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError("gemm_bf16_nt output must be [M,N] bf16 or fp32")
    rc = lib().orion_gemm_bf16_nt(a.data_ptr(), b.data_ptr(), out.data_ptr(),
                                  m, n, k, int(out.dtype == torch.float32),
                                  _stream_ptr(stream))
    if rc != 0:
        raise KernelError("orion_gemm_bf16_nt", rc)
    return out
