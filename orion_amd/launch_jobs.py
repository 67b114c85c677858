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
    return {
        "model_names": [c["arch"] for c in config_dict_list],
        "model_files": [c["kernel_file"] for c in config_dict_list],
        "additional_model_files": [c.get("additional_kernel_file") for c in config_dict_list],
        "num_kernels": [c["num_kernels"] for c in config_dict_list],
        "num_iters": [c["num_iters"] for c in config_dict_list],
        "train_list": [c["args"]["train"] for c in config_dict_list],
        "additional_num_kernels": [c.get("additional_num_kernels") for c in config_dict_list],
    }


def launch_jobs(config_dict_list, input_args, run_eval=True, function_dict=None,
                require_preload=True):
    """reference: launch_jobs.py:44-122."""
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
                        help="choose one of orion | reef | sequential")
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
    if args.algo not in ("orion", "reef", "sequential"):
        raise SystemExit("--algo must be one of orion | reef | sequential")
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
