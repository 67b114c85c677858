"""Launcher: a JSON job file -> one thread per client + the scheduler thread.

Counterpart of the reference's ``benchmarking/launch_jobs.py``: same command
line (:126-138), same JSON schema (:68-75; the LAST entry is the high-priority
client), same thread layout (:78-110).  Run it with the interception library
preloaded, as the reference is (artifact_evaluation/README.md:75)::

    LD_PRELOAD=<pkg>/libinttemp.so python -m orion_amd.launch_jobs \\
        --algo orion --config_file job.json --orion_max_be_duration 160000

``python -m orion_amd.launch_jobs --print-preload`` prints the library path.
"""

import argparse
import ctypes
import json
import os
import sys
import threading

from . import _lib
from . import scheduler_frontend as fe


def _function_dict():
    # imported lazily: the model code needs torch, the argument parser does not
    from .benchmark_suite.bert_trainer import bert_loop
    from .benchmark_suite.train_imagenet import imagenet_loop
    from .benchmark_suite.transformer_trainer import transformer_loop
    from .kernel_pair import gemm_loop, triad_loop
    return {
        "gemm_bf16": gemm_loop,
        "triad_f32": triad_loop,
        "resnet50": imagenet_loop,
        "resnet101": imagenet_loop,
        "mobilenet_v2": imagenet_loop,
        "bert": bert_loop,
        "transformer": transformer_loop,
    }


def check_preloaded():
    """The interception library only sees the clients' HIP calls when the
    dynamic linker put it first; refuse to run a job without it."""
    # A preloaded library sits in the global symbol scope; one that was only
    # dlopen()ed later does not, and would not interpose anything either.
    try:
        ctypes.CDLL(None).orion_capture_arm
    except AttributeError:
        raise RuntimeError(
            "libinttemp.so is not preloaded: start the launcher with "
            f"LD_PRELOAD={_lib.CAPTURE_LIB} (append to any value already set)")


def job_lists(config_dict_list):
    """The per-client lists the scheduler front end takes, from a job file
    (reference: launch_jobs.py:68-75).  The LAST entry is the high-priority
    client (scheduler_eval.cpp:256)."""
    for c in config_dict_list:
        for key in ("arch", "kernel_file", "num_kernels", "num_iters", "args"):
            if key not in c:
                raise KeyError(f"job entry lacks {key!r}: {c}")
        if "train" not in c["args"]:
            raise KeyError("job entry args lack 'train'")
    # "deterministic" switches MIOpen's solver choice for the whole process, so a
    # client that asks for it changes the kernels -- and the kernel count -- of
    # every other client of the job, whose profile was captured without it
    takes_flag = [c for c in config_dict_list
                  if c["arch"] in ("resnet50", "resnet101", "mobilenet_v2", "bert", "transformer")]
    if len({bool(c["args"].get("deterministic")) for c in takes_flag}) > 1:
        raise ValueError("'deterministic' must be set for all model clients of a job or for none: "
                         "it selects the convolution solvers of the whole process")
    # ORION_BE_RUN_AHEAD=1 (best-effort clients queue their launches ahead of the
    # dispatch) has faulted an MI355X with framework trainers as best-effort
    # clients, cause not found: refused for them, with no override.  (The
    # scheduler library never clears such a client for it either.)
    framework_be = [c for c in config_dict_list[:-1] if c in takes_flag]
    if os.environ.get("ORION_BE_RUN_AHEAD", "0") not in ("", "0") and framework_be:
        raise RuntimeError(
            "ORION_BE_RUN_AHEAD=1 with a framework model as a best-effort client has ended in "
            "GPU faults on an MI355X (ResNet-50 training beside ResNet-50 inference); it is "
            "supported for the kernel-pair clients (gemm_bf16, triad_f32) only.  Unset it.")
    return {
        "model_names": [c["arch"] for c in config_dict_list],
        "model_files": [c["kernel_file"] for c in config_dict_list],
        "additional_model_files": [c.get("additional_kernel_file") for c in config_dict_list],
        "num_kernels": [c["num_kernels"] for c in config_dict_list],
        "num_iters": [c["num_iters"] for c in config_dict_list],
        "train_list": [c["args"]["train"] for c in config_dict_list],
        "additional_num_kernels": [c.get("additional_num_kernels") for c in config_dict_list],
    }


class _UnscheduledRendezvous:
    """``barriers[0]`` of the ``streams`` baseline.  Under the scheduler every
    client meets the scheduler thread before it builds its model, after its
    iterations 1 and 10, and at the end of its run; without one the clients meet
    each other the first three times, and the fourth wait -- the end of a run --
    returns at once, the high-priority client's after raising the stop flag the
    best-effort clients poll."""

    def __init__(self, num_clients):
        self.barrier = threading.Barrier(num_clients)
        self.hp_name = f"orion-client-{num_clients - 1}"
        self.waits = {}

    def wait(self):
        me = threading.current_thread().name
        self.waits[me] = self.waits.get(me, 0) + 1
        if self.waits[me] <= 3:
            self.barrier.wait()
            return
        if me == self.hp_name:
            from .benchmark_suite import client_common
            client_common.UNSCHEDULED_STOP.set()


def launch_unscheduled(config_dict_list, function_dict=None):
    """The clients as plain threads on streams of their own, no interception and
    no scheduler: what the reference measures as its "streams" baseline with the
    ``*_torch.py`` variants of its client loops
    (benchmarking/benchmark_suite/train_imagenet_torch.py and siblings).  Same
    loops, same result files."""
    from .benchmark_suite.client_common import seed_everything
    seed_everything(42)
    function_dict = function_dict or _function_dict()
    num_clients = len(config_dict_list)
    rendezvous = _UnscheduledRendezvous(num_clients)
    barriers = [rendezvous] * num_clients
    client_barrier = threading.Barrier(num_clients)
    threads, results = [], [None] * num_clients
    for i, config_dict in enumerate(config_dict_list):
        kwargs = dict(config_dict["args"])
        kwargs.update({"num_iters": config_dict["num_iters"], "local_rank": 0,
                       "barriers": barriers, "client_barrier": client_barrier, "tid": i})

        def target(func=function_dict[config_dict["arch"]], kwargs=kwargs, i=i):
            try:
                results[i] = func(**kwargs)
            except BaseException:
                import traceback
                traceback.print_exc()
                print(f"orion: client {i} failed; aborting the job", flush=True)
                os._exit(1)

        thread = threading.Thread(target=target, name=f"orion-client-{i}")
        thread.start()
        threads.append(thread)
    for thread in threads:
        thread.join()
    print("--------- all threads joined!", flush=True)
    return results


def launch_jobs(config_dict_list, input_args, run_eval=True, function_dict=None,
                require_preload=True):
    """reference: launch_jobs.py:44-122."""
    if getattr(input_args, "algo", None) == "streams":
        return launch_unscheduled(config_dict_list, function_dict)
    from .benchmark_suite.client_common import seed_everything
    seed_everything(42)
    # All clients are threads of this interpreter and share its GIL.  The switch
    # interval can be shortened from the environment; on the measured pairs it
    # made no difference (clients release the GIL at every operator call).
    interval = float(os.environ.get("ORION_GIL_SWITCH_INTERVAL_S", "0"))
    if interval > 0:
        sys.setswitchinterval(interval)
    if require_preload:
        check_preloaded()
    function_dict = function_dict or _function_dict()
    num_clients = len(config_dict_list)
    barriers = [threading.Barrier(num_clients + 1) for _ in range(num_clients)]
    client_barrier = threading.Barrier(num_clients)
    sched_lib = fe.load_scheduler_library()
    py_scheduler = fe.PyScheduler(sched_lib, num_clients)

    lists = job_lists(config_dict_list)
    model_names, model_files = lists["model_names"], lists["model_files"]
    additional_model_files = lists["additional_model_files"]
    num_kernels, num_iters = lists["num_kernels"], lists["num_iters"]
    train_list = lists["train_list"]
    additional_num_kernels = lists["additional_num_kernels"]

    tids, threads, results = [], [], [None] * num_clients
    for i, config_dict in enumerate(config_dict_list):
        func = function_dict[config_dict["arch"]]
        model_args = dict(config_dict["args"])
        model_args.update({"num_iters": num_iters[i], "local_rank": 0,
                           "barriers": barriers, "client_barrier": client_barrier,
                           "tid": i})

        def target(func=func, kwargs=model_args, i=i):
            try:
                results[i] = func(**kwargs)
            except BaseException:
                # A dead client would leave the scheduler polling for records
                # that never come (the reference hangs): end the job loudly.
                import traceback
                traceback.print_exc()
                print(f"orion: client {i} failed; aborting the job", flush=True)
                os._exit(1)

        thread = threading.Thread(target=target, name=f"orion-client-{i}")
        thread.start()
        tids.append(thread.native_id)
        threads.append(thread)

    algo = input_args.algo
    sched_thread = threading.Thread(
        target=py_scheduler.run_scheduler, name="orion-scheduler",
        args=(barriers, tids, model_names, model_files, additional_model_files,
              num_kernels, additional_num_kernels, num_iters, True, run_eval,
              algo == "reef", algo == "sequential",
              input_args.reef_depth if algo == "reef" else input_args.orion_max_be_duration,
              input_args.orion_hp_limit, input_args.orion_start_update, train_list))
    sched_thread.start()
    for thread in threads:
        thread.join()
    sched_thread.join()
    print("--------- all threads joined!", flush=True)
    return results


def build_parser():
    parser = argparse.ArgumentParser()
    parser.add_argument("--algo", type=str, required=False, default="orion",
                        help="choose one of orion | reef | sequential (or streams: "
                             "the clients on plain streams, no scheduler, as a baseline)")
    parser.add_argument("--config_file", type=str,
                        help="path to the experiment configuration file")
    parser.add_argument("--reef_depth", type=int, default=1,
                        help="If reef is used, this stands for the queue depth")
    parser.add_argument("--orion_max_be_duration", type=int, default=1,
                        help="If orion is used, the maximum aggregate duration "
                             "(ns) of on-the-fly best-effort kernels")
    parser.add_argument("--orion_start_update", type=int, default=1,
                        help="If orion is used and the high priority job is training, "
                             "the kernel id after which the update phase starts")
    parser.add_argument("--orion_hp_limit", type=int, default=1,
                        help="If orion is used and the high priority job is training, "
                             "the maximum tolerated training iteration time")
    parser.add_argument("--print-preload", action="store_true",
                        help="print the path of the library to LD_PRELOAD and exit")
    return parser


def main(argv=None):
    args = build_parser().parse_args(argv)
    if args.print_preload:
        print(_lib.CAPTURE_LIB)
        return 0
    if args.algo not in ("orion", "reef", "sequential", "streams"):
        raise SystemExit("--algo must be one of orion | reef | sequential | streams")
    if not args.config_file:
        raise SystemExit("--config_file is required")
    import torch
    torch.cuda.set_device(0)
    with open(args.config_file) as f:
        config = json.load(f)
    launch_jobs(config, args, True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
