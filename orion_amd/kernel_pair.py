"""The kernel-pair microbenchmark: a high-priority bf16 GEMM (MFMA-bound) beside
a best-effort fp32 streaming triad (HBM-bound), both hand-written gfx950
kernels.

Two ways to run the pair:

* ``measure_*``: directly on two streams of this process (the best-effort one
  CU-masked), timing every launch with HIP events -- what each kernel achieves
  alone and next to the other, per CU-mask size;
* ``gemm_loop`` / ``triad_loop``: as clients of the scheduler, through the
  interception layer (``run_child`` starts a launcher with the library
  preloaded), the configuration the reference calls a toy co-location pair
  (benchmarking/benchmark_suite/toy_models/, conv_trainer.py / bnorm_trainer.py
  loops of 25 ops per iteration).
"""

import json
import os
import subprocess
import sys

import torch

from . import _lib, kernels
from .benchmark_suite import client_common as cc

GEMM_N = 8192
TRIAD_ELEMS = 1 << 28          # 1 GiB per array
HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0


def _inputs_gemm(n, device, seed=0):
    g = torch.Generator(device=device).manual_seed(seed)
    a = (torch.rand(n, n, device=device, generator=g) * 2 - 1).to(torch.bfloat16)
    b = (torch.rand(n, n, device=device, generator=g) * 2 - 1).to(torch.bfloat16)
    return a, b


def _inputs_triad(n, device, seed=1):
    g = torch.Generator(device=device).manual_seed(seed)
    b = torch.rand(n, device=device, generator=g) * 2 - 1
    c = torch.rand(n, device=device, generator=g) * 2 - 1
    return b, c


def _time_launches(stream, launch, reps, warmup=2):
    """Average milliseconds per launch, from HIP events recorded on ``stream``."""
    with torch.cuda.stream(stream):
        for _ in range(warmup):
            launch(stream)
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record(stream)
        for _ in range(reps):
            launch(stream)
        end.record(stream)
    end.synchronize()
    return start.elapsed_time(end) / reps


def measure_alone(gemm_n=GEMM_N, triad_elems=TRIAD_ELEMS, masks=(32, 64, 128, 0),
                  reps=10, device="cuda:0", warmup=2):
    """Each kernel alone: GEMM on the whole GPU, triad per CU-mask size."""
    a, b = _inputs_gemm(gemm_n, device)
    c = torch.empty(gemm_n, gemm_n, device=device, dtype=torch.bfloat16)
    tb, tc = _inputs_triad(triad_elems, device)
    ta = torch.empty_like(tb)
    full = kernels.cu_masked_stream(0)
    out = {}
    # The GEMM holds the GPU at its power limit; after an idle period the clocks
    # overshoot, dip and settle within ~50 launches.  "burst" is the first 20
    # launches, the headline figure follows 100 untimed ones.
    launch_gemm = lambda s: kernels.gemm_bf16_nt(a, b, out=c, stream=s)
    torch.cuda.synchronize()
    burst = _time_launches(full, launch_gemm, 20, warmup=0)
    ms = _time_launches(full, launch_gemm, max(reps, 100), warmup=100)
    out["gemm"] = {"ms": ms, "tflops": 2 * gemm_n ** 3 / ms / 1e9,
                   "frac_of_peak": 2 * gemm_n ** 3 / ms / 1e9 / MFMA_BF16_PEAK_TFLOPS,
                   "burst_ms": burst, "burst_tflops": 2 * gemm_n ** 3 / burst / 1e9}
    out["triad"] = {}
    for m in masks:
        s = kernels.cu_masked_stream(m)
        ms = _time_launches(s, lambda st: kernels.triad(ta, tb, tc, 1.7, stream=st), reps,
                            warmup=warmup)
        gbs = 12 * triad_elems / ms / 1e6
        out["triad"][str(m or 256)] = {"ms": ms, "gbs": gbs, "frac_of_peak": gbs / HBM_PEAK_GBS}
    return out


def measure_pair(mask, gemm_n=GEMM_N, triad_elems=TRIAD_ELEMS, reps=10, device="cuda:0"):
    """Both kernels at once: GEMM stream over the whole GPU, triad stream over
    ``mask`` CUs.  A short pilot run finds how long each kernel takes next to
    the other; the measured run then queues as many triads as the GEMMs need,
    so both averages are taken under contention from end to end (and after the
    clocks have settled, like ``measure_alone``)."""
    a, b = _inputs_gemm(gemm_n, device)
    c = torch.empty(gemm_n, gemm_n, device=device, dtype=torch.bfloat16)
    tb, tc = _inputs_triad(triad_elems, device)
    ta = torch.empty_like(tb)
    sg = kernels.cu_masked_stream(0)
    st = kernels.cu_masked_stream(mask)

    def run(n_gemm, n_triad):
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
        # head: start the other stream first so the timed window is overlapped
        for _ in range(3):
            kernels.triad(ta, tb, tc, 1.7, stream=st)
        ev[0].record(sg)
        ev[2].record(st)
        # interleave the submissions so neither queue runs dry
        done_t = 0
        for i in range(n_gemm):
            kernels.gemm_bf16_nt(a, b, out=c, stream=sg)
            want_t = (i + 1) * n_triad // n_gemm
            while done_t < want_t:
                kernels.triad(ta, tb, tc, 1.7, stream=st)
                done_t += 1
        ev[1].record(sg)
        ev[3].record(st)
        torch.cuda.synchronize()
        return ev[0].elapsed_time(ev[1]) / n_gemm, ev[2].elapsed_time(ev[3]) / max(done_t, 1)

    torch.cuda.synchronize()
    g_ms, t_ms = run(30, 90)                      # pilot; also settles the clocks
    g_ms, t_ms = run(30, max(30, int(30 * g_ms / t_ms)))
    reps = max(reps, 60)
    gemm_ms, triad_ms = run(reps, max(reps, int(reps * g_ms / t_ms)))
    return {"mask": mask or 256, "gemm_ms": gemm_ms,
            "gemm_tflops": 2 * gemm_n ** 3 / gemm_ms / 1e9,
            "triad_ms": triad_ms, "triad_gbs": 12 * triad_elems / triad_ms / 1e6}


# ---------------------------------------------------------------------------
# the pair as scheduler clients

def _pair_client(kind, size, num_iters, rps, uniform, barriers, tid, per_iter):
    cc.seed_everything(42)
    backend = cc.Backend()
    sleep_times = cc.arrival_gaps(rps, uniform, num_iters, "", 42)
    barriers[0].wait()
    device = torch.device("cuda", 0)
    stream = torch.cuda.Stream(device=device)
    backend.register_stream(stream)
    state = {}
    with torch.cuda.stream(stream):
        with cc.uncaptured(backend):
            if kind == "gemm":
                a, b = _inputs_gemm(size, device)
                out = torch.empty(size, size, device=device, dtype=torch.bfloat16)
            else:
                tb, tc = _inputs_triad(size, device)
                out = torch.empty_like(tb)

        def step(batch_idx):
            for _ in range(per_iter):
                if kind == "gemm":
                    kernels.gemm_bf16_nt(a, b, out=out, stream=stream)
                else:
                    kernels.triad(out, tb, tc, 1.7, stream=stream)

        def extra():
            save_dir = os.environ.get("ORION_SAVE_OUTPUT_DIR")
            if save_dir:
                torch.save(out[:4096].float().cpu() if kind == "triad" else out[:8].float().cpu(),
                           os.path.join(save_dir, f"client_{tid}_output.pt"))
            return {}

        with cc.uncaptured(backend):
            step(-1)
        res = cc.run_client(tid, kind == "triad", num_iters, sleep_times, barriers,
                            step, backend, extra=extra)
    return res


def gemm_loop(batchsize, train, num_iters, rps, uniform, dummy_data, local_rank,
              barriers, client_barrier, tid, per_iter=1):
    """High-priority client: ``per_iter`` GEMMs of size ``batchsize``^3 a request."""
    return _pair_client("gemm", batchsize, num_iters, rps, uniform, barriers, tid, per_iter)


def triad_loop(batchsize, train, num_iters, rps, uniform, dummy_data, local_rank,
               barriers, client_barrier, tid, per_iter=8):
    """Best-effort client: ``per_iter`` triads over ``batchsize`` elements."""
    return _pair_client("triad", batchsize, num_iters, rps, uniform, barriers, tid, per_iter)


def pair_job(small=False, hp_iters=60, rps=0):
    gemm_n = 1024 if small else GEMM_N
    elems = (1 << 22) if small else TRIAD_ELEMS
    return [
        {"arch": "triad_f32", "kernel_file": "", "num_kernels": 0, "num_iters": 1_000_000,
         "args": {"batchsize": elems, "rps": 0, "uniform": False, "dummy_data": True,
                  "train": True}},
        {"arch": "gemm_bf16", "kernel_file": "", "num_kernels": 0, "num_iters": hp_iters,
         "args": {"batchsize": gemm_n, "rps": rps, "uniform": False, "dummy_data": True,
                  "train": False}},
    ]


def run_child(small=False, check=False, workdir=None, hp_iters=60, masks=None,
              max_be_duration=1_000_000, algo="orion", reef_depth=12, rps=0,
              confine_long=False):
    """Profile both clients and run the pair isolated and co-located, in child
    processes with the interception library preloaded.  Returns the experiment
    summary (see ``colocate.experiment``) plus ``outputs_match`` when ``check``."""
    import tempfile
    from . import colocate
    workdir = workdir or tempfile.mkdtemp(prefix="orion_pair_")
    os.makedirs(workdir, exist_ok=True)
    cfg = os.path.join(workdir, "pair.json")
    with open(cfg, "w") as f:
        json.dump(pair_job(small, hp_iters, rps), f)
    filled = os.path.join(workdir, "pair_filled.json")
    env = colocate.preload_env({"ORION_RESULT_DIR": workdir})
    subprocess.run([sys.executable, "-m", "orion_amd.profiling.capture_profile", "--config",
                    cfg, "--fill", filled, "--out-dir", os.path.join(workdir, "profiles")],
                   check=True, env=env, cwd=os.path.dirname(_lib.PKG_DIR),
                   stdout=subprocess.DEVNULL)
    with open(filled) as f:
        job = json.load(f)
    extra_env = {}
    if masks:
        extra_env["ORION_BE_CU_MASKS"] = masks
    if confine_long:
        extra_env["ORION_CONFINE_LONG_BE"] = "1"
    if check:
        os.makedirs(os.path.join(workdir, "out_iso"), exist_ok=True)
        os.makedirs(os.path.join(workdir, "out_co"), exist_ok=True)
    res = {}
    e = dict(extra_env)
    if check:
        e["ORION_SAVE_OUTPUT_DIR"] = os.path.join(workdir, "out_iso")
    iso = colocate.experiment(job[-1:], workdir=os.path.join(workdir, "iso"), env=e,
                              max_be_duration=max_be_duration)
    res["hp_isolated"] = iso["hp_isolated"]
    be = dict(job[0])
    be["num_iters"] = 40
    res["be_isolated"] = colocate.run_job([be], "orion", os.path.join(workdir, "be_iso"),
                                          max_be_duration, env=extra_env)[0]
    e = dict(extra_env)
    if check:
        e["ORION_SAVE_OUTPUT_DIR"] = os.path.join(workdir, "out_co")
        e["ORION_RECORD_DIR"] = os.path.join(workdir, "out_co")
    co = colocate.run_job(job, algo, os.path.join(workdir, "co"), max_be_duration,
                          reef_depth=reef_depth, env=e)
    res["hp_colocated"], res["be_colocated"] = co[-1], co[0]
    res["be_retained"] = co[0]["throughput"] / res["be_isolated"]["throughput"]
    if check:
        iso_out = torch.load(os.path.join(workdir, "out_iso", "client_0_output.pt"),
                             weights_only=True)
        co_out = torch.load(os.path.join(workdir, "out_co", "client_1_output.pt"),
                            weights_only=True)
        res["outputs_match"] = bool(torch.equal(iso_out, co_out))
    res["workdir"] = workdir
    return res
