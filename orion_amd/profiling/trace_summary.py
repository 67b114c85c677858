"""Per-thread summary of a rocprofv3 kernel trace (``*_kernel_trace.csv``) of a
job that ran through the interception layer.

    python -m orion_amd.profiling.trace_summary --trace kt_kernel_trace.csv --per-request 371

With the default hand-off a high-priority inference client issues its own
kernels, so its kernels carry its thread id; every best-effort kernel carries
the scheduler thread's.  For each launching thread: kernel count, summed and
mean kernel duration, the hardware queues used.  With ``--per-request N`` the
kernels of every thread that launched at least 100 x N of them are also cut into
consecutive groups of N, counted from the end of the trace (the steady state),
and the distribution of the summed kernel time and of the first-start-to-last-end
span per group is reported over the last ``--last`` groups: run on the trace of
the client alone and of the co-located job, the two tell how much the
high-priority kernels themselves were slowed down.
"""

import argparse
import collections
import csv
import json

import numpy as np


def summarise(path, per_request=0, last=150):
    by_thread = collections.defaultdict(list)
    with open(path, newline="") as f:
        for r in csv.DictReader(f):
            by_thread[int(r["Thread_Id"])].append(
                (int(r["Start_Timestamp"]), int(r["End_Timestamp"]), int(r.get("Queue_Id") or 0)))
    out = {}
    for tid, rows in sorted(by_thread.items()):
        rows.sort()
        start = np.array([r[0] for r in rows], dtype=np.int64)
        end = np.array([r[1] for r in rows], dtype=np.int64)
        dur = end - start
        s = {"kernels": int(len(rows)), "sum_ms": float(dur.sum() / 1e6),
             "mean_us": float(dur.mean() / 1e3), "queues": sorted({r[2] for r in rows})}
        if per_request and len(rows) >= 100 * per_request:
            k = len(rows) // per_request
            cut = len(rows) - k * per_request
            sums = dur[cut:].reshape(k, per_request).sum(axis=1)[-last:] / 1e6
            span = (end[cut:].reshape(k, per_request)[:, -1]
                    - start[cut:].reshape(k, per_request)[:, 0])[-last:] / 1e6
            s["groups"] = int(len(sums))
            for name, v in (("kernel_ms", sums), ("span_ms", span)):
                s[name] = {"p50": float(np.percentile(v, 50)), "p99": float(np.percentile(v, 99)),
                           "mean": float(v.mean())}
        out[str(tid)] = s
    return out


def main(argv=None):
    p = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    p.add_argument("--trace", required=True)
    p.add_argument("--per-request", type=int, default=0)
    p.add_argument("--last", type=int, default=150)
    a = p.parse_args(argv)
    print(json.dumps(summarise(a.trace, a.per_request, a.last), indent=1))


if __name__ == "__main__":
    main()
