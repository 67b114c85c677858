"""Python front end of the scheduler: ctypes marshalling and the phase protocol.

Mirror of the reference's ``src/scheduler_frontend.py`` (class ``PyScheduler``,
``run_scheduler``): same constructor and ``run_scheduler`` argument list, same
three-phase run -- one warm-up iteration, profile swap for training clients,
ten warm-up iterations, measured run -- with the same rendezvous points on
``barriers[0]`` (scheduler_frontend.py:68-94).  Unlike the reference it declares
``argtypes``/``restype`` for every entry point (the reference assigns them to
the library object, scheduler_frontend.py:56, which has no effect).
"""

from ctypes import (POINTER, c_bool, c_char_p, c_float, c_int, c_ulonglong, c_void_p)
import time

from . import _lib


def load_scheduler_library(path=None):
    """``scheduler_eval.so`` with typed entry points."""
    lib = _lib.load(path or _lib.SCHEDULER_LIB)
    if getattr(lib, "_orion_typed", False):
        return lib
    lib.sched_init.argtypes = []
    lib.sched_init.restype = c_void_p
    lib.setup.argtypes = [c_void_p, c_int, POINTER(c_int), POINTER(c_char_p),
                          POINTER(c_char_p), POINTER(c_int), POINTER(c_int),
                          POINTER(c_bool), c_bool]
    lib.setup.restype = None
    lib.setup_change.argtypes = [c_void_p, c_int, c_char_p, c_int]
    lib.setup_change.restype = None
    lib.schedule.argtypes = [c_void_p, c_int, c_bool, c_int, c_bool, c_int,
                             c_bool, c_bool, c_int, c_int, c_int]
    lib.schedule.restype = c_void_p
    lib.reset.argtypes = [c_void_p, c_int]
    lib.reset.restype = c_void_p
    lib.orion_client_stream.argtypes = [c_int]
    lib.orion_client_stream.restype = c_void_p
    lib.orion_sched_num_cus.argtypes = []
    lib.orion_sched_num_cus.restype = c_int
    lib.orion_sched_iteration_ms.argtypes = [c_int, POINTER(c_float), c_int]
    lib.orion_sched_iteration_ms.restype = c_int
    lib.orion_sched_teardown.argtypes = []
    lib.orion_sched_teardown.restype = None
    lib._orion_typed = True
    return lib


def load_capture_library(path=None):
    """``libinttemp.so`` (already in the process when it was LD_PRELOADed)."""
    lib = _lib.load(path or _lib.CAPTURE_LIB)
    if getattr(lib, "_orion_typed", False):
        return lib
    lib.block.argtypes = [c_int]
    lib.block.restype = None
    lib.stop.argtypes = []
    lib.stop.restype = c_int
    lib.orion_register_thread.argtypes = [c_int]
    lib.orion_register_thread.restype = None
    lib.orion_register_stream.argtypes = [c_void_p]
    lib.orion_register_stream.restype = None
    lib.orion_client_index.argtypes = []
    lib.orion_client_index.restype = c_int
    lib.orion_thread_passthrough.argtypes = [c_int]
    lib.orion_thread_passthrough.restype = None
    lib.orion_client_deferred.argtypes = [c_int]
    lib.orion_client_deferred.restype = c_ulonglong
    lib.orion_client_submitted.argtypes = [c_int]
    lib.orion_client_submitted.restype = c_ulonglong
    lib.orion_thread_time_in_calls_ns.argtypes = []
    lib.orion_thread_time_in_calls_ns.restype = c_ulonglong
    lib.orion_thread_calls.argtypes = []
    lib.orion_thread_calls.restype = c_ulonglong
    lib.orion_tls_fresh_check.argtypes = []
    lib.orion_tls_fresh_check.restype = None
    lib.orion_tls_fresh_stats.argtypes = [POINTER(c_ulonglong), POINTER(c_ulonglong)]
    lib.orion_tls_fresh_stats.restype = None
    lib._orion_typed = True
    return lib


class PyScheduler:
    """reference: src/scheduler_frontend.py:8-15."""

    def __init__(self, sched_lib, num_clients):
        try:    # reference :12 -- device 0 is the only device used
            import torch
            if torch.cuda.is_available():
                torch.cuda.set_device(0)
        except ImportError:
            pass
        self._sched_lib = sched_lib
        self._scheduler = sched_lib.sched_init()
        self._num_clients = num_clients

    def run_scheduler(self, barriers, tids, model_names, kernel_files,
                      additional_kernel_files, num_kernels,
                      additional_num_kernels, num_iters, profile, run_eval,
                      reef, sequential, reef_depth, hp_limit, update_start,
                      train):
        """reference: src/scheduler_frontend.py:17-94 (the run_eval branch; the
        per-iteration branch :96-127 depends on a library, scheduler.so, that the
        reference does not contain)."""
        n = self._num_clients
        if not (len(tids) == len(model_names) == len(kernel_files)
                == len(num_kernels) == len(num_iters) == len(train) == n):
            raise ValueError("per-client lists must have one entry per client")
        if not run_eval:
            raise NotImplementedError(
                "run_eval=False needs scheduler.so/schedule_one, which the "
                "reference never shipped")
        lib = self._sched_lib
        IntAr = c_int * n
        CharAr = c_char_p * n
        BoolAr = c_bool * n
        # The arrays must outlive every schedule() call below; they do, as
        # locals of this frame (the reference borrows them, too: :608-609).
        tids_ar = IntAr(*tids)
        num_kernels_ar = IntAr(*num_kernels)
        num_iters_ar = IntAr(*num_iters)
        names_ar = CharAr(*[m.encode("utf-8") for m in model_names])
        files_ar = CharAr(*[f.encode("utf-8") for f in kernel_files])
        train_ar = BoolAr(*[bool(t) for t in train])

        lib.setup(self._scheduler, n, tids_ar, names_ar, files_ar,
                  num_kernels_ar, num_iters_ar, train_ar, bool(reef))
        if not profile:
            return
        self._sync = _device_synchronize
        barriers[0].wait()
        # one iteration to warm up; training clients run on a placeholder profile
        lib.schedule(self._scheduler, n, True, 0, True, 1, bool(reef),
                     bool(sequential), reef_depth, hp_limit, update_start)
        self._sync()
        for j in range(n):
            if additional_kernel_files[j] is not None:
                lib.setup_change(self._scheduler, j,
                                 additional_kernel_files[j].encode("utf-8"),
                                 additional_num_kernels[j])
        barriers[0].wait()
        lib.schedule(self._scheduler, n, True, 0, True, 10, bool(reef),
                     bool(sequential), reef_depth, hp_limit, update_start)
        self._sync()
        barriers[0].wait()
        start = time.time()
        lib.schedule(self._scheduler, n, True, 0, False, 0, bool(reef),
                     bool(sequential), reef_depth, hp_limit, update_start)
        barriers[0].wait()
        self._sync()
        self.total_time = time.time() - start
        print(f"Total time is {self.total_time}")

    def iteration_times_ms(self, client):
        """Per-iteration wall times the scheduler measured for a client."""
        lib = self._sched_lib
        count = lib.orion_sched_iteration_ms(client, None, 0)
        if count <= 0:
            return []
        buf = (c_float * count)()
        lib.orion_sched_iteration_ms(client, buf, count)
        return list(buf)


def _device_synchronize():
    try:
        import torch
        if torch.cuda.is_available():
            torch.cuda.synchronize()
    except ImportError:
        pass
