"""Run one client of a job file alone, with no scheduler and no interception:
the program to put after ``rocprofv3 ... --`` when collecting hardware counters
for a profile.  The client runs the same loop as under the scheduler (so it
launches the same kernels per iteration); ``block``/``stop`` are no-ops because
nothing is armed, and one-party barriers never wait.

    rocprofv3 --kernel-trace --output-format csv -d out -o t -- \\
        python3 -m orion_amd.profiling.standalone --config job.json --client 1 --iters 12
"""

import argparse
import json
import os
import threading


def main(argv=None):
    p = argparse.ArgumentParser()
    p.add_argument("--config", required=True)
    p.add_argument("--client", type=int, default=0)
    p.add_argument("--iters", type=int, default=12)
    a = p.parse_args(argv)
    import torch
    torch.cuda.set_device(0)
    from ..launch_jobs import _function_dict
    with open(a.config) as f:
        entry = json.load(f)[a.client]
    kwargs = dict(entry["args"])
    kwargs.update({"num_iters": a.iters, "local_rank": 0,
                   "barriers": [threading.Barrier(1)],
                   "client_barrier": threading.Barrier(1), "tid": 0})
    kwargs["rps"] = 0
    os.environ.setdefault("ORION_RESULT_DIR", "/tmp")
    _function_dict()[entry["arch"]](**kwargs)
    torch.cuda.synchronize()


if __name__ == "__main__":
    main()
