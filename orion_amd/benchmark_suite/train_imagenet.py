"""Vision client (ResNet-50 / ResNet-101 / MobileNetV2): training or open-loop
inference on synthetic images.

Counterpart of the reference's ``imagenet_loop``
(benchmarking/benchmark_suite/train_imagenet.py:71-241): same keyword
arguments, same loop and barrier protocol, same ``client_{tid}.json``.  Extra,
optional keys of a job's ``args``: ``dtype`` ("fp32" | "bf16"), ``momentum``,
``lr`` (0.1, the reference's, :116), ``seed``, ``deterministic``, ``hip_graph``.  Synthetic data follows the job description: images N(0,1), labels
uniform over the classes (the reference uses U(0,1) images and all-ones labels,
:36-37).
"""

import os
import threading

import torch

from . import client_common as cc
from .vision_models import MODELS


class DummyDataLoader:
    """:33-44 -- one pinned batch, reused for every iteration."""

    def __init__(self, batchsize, seed):
        g = torch.Generator().manual_seed(seed)
        pin = torch.cuda.is_available()
        self.data = torch.randn([batchsize, 3, 224, 224], generator=g)
        self.target = torch.randint(0, 1000, [batchsize], generator=g)
        if pin:
            self.data, self.target = self.data.pin_memory(), self.target.pin_memory()

    def __iter__(self):
        return self

    def __next__(self):
        return self.data, self.target


def imagenet_loop(model_name, batchsize, train, num_iters, rps, uniform,
                  dummy_data, local_rank, barriers, client_barrier, tid,
                  input_file="", dtype="fp32", momentum=0.9, seed=42,
                  deterministic=False, hip_graph=False, lr=0.1):
    cc.seed_everything(seed)
    if deterministic:
        # keep MIOpen off solvers that accumulate with atomics (split-K), whose
        # results differ in the last bit from run to run.  The switch is the
        # process's, not the client's: every model client of a job must agree
        # on it (the launcher checks), because it changes which kernels -- and how
        # many -- the others submit
        torch.backends.cudnn.deterministic = True
    if hip_graph and train:
        raise ValueError("hip_graph is for inference clients")
    backend = cc.Backend()
    sleep_times = cc.arrival_gaps(rps, uniform, num_iters, input_file, seed)
    if not dummy_data:
        raise NotImplementedError("only synthetic data is available offline")
    barriers[0].wait()                       # released by the scheduler (:102)
    print(f"-------------- client {tid} thread id: {threading.get_native_id()}",
          flush=True)

    device = torch.device("cuda", local_rank)
    tdtype = {"fp32": torch.float32, "bf16": torch.bfloat16}[dtype]
    stream = torch.cuda.Stream(device=device)
    backend.register_stream(stream)
    losses = []
    with torch.cuda.stream(stream), torch.autograd.set_multithreading_enabled(False):
        with cc.uncaptured(backend):
            with cc.MODEL_INIT_LOCK:
                cc.seed_everything(seed)
                model = MODELS[model_name](num_classes=1000)
            model = model.to(device)
            if train:
                model.train()
                optimizer = torch.optim.SGD(model.parameters(), lr=lr, momentum=momentum)
                criterion = torch.nn.CrossEntropyLoss().to(device)
            else:
                model.eval()
                model = model.to(tdtype)
        loader = DummyDataLoader(batchsize, seed)
        data, target = next(loader)
        state = {}

        def step(batch_idx):
            if train:
                gpu_data = data.to(device, non_blocking=True)
                gpu_target = target.to(device, non_blocking=True)
                optimizer.zero_grad()
                with torch.autocast("cuda", dtype=torch.bfloat16, enabled=dtype == "bf16"):
                    output = model(gpu_data)
                    loss = criterion(output, gpu_target)
                loss.backward()
                optimizer.step()
                state["loss"] = loss
                cc.keep_loss(state, batch_idx, loss)
            elif "graph" in state:
                # one copy record and one graph record per request
                state["graph_in"].copy_(data, non_blocking=True)
                state["graph"].replay()
                state["output"] = state["graph_out"]
            else:
                with torch.no_grad():
                    gpu_data = data.to(device, non_blocking=True).to(tdtype)
                    state["output"] = model(gpu_data)

        def extra():
            out = {}
            save_dir = os.environ.get("ORION_SAVE_OUTPUT_DIR")
            if save_dir and "output" in state:
                torch.save(state["output"].float().cpu(),
                           os.path.join(save_dir, f"client_{tid}_output.pt"))
            if "loss" in state:
                out["final_loss"] = float(state["loss"].detach().float().cpu())
            out.update(cc.loss_checkpoint_report(state))
            return out

        with cc.uncaptured(backend):
            for i in range(cc.UNCAPTURED_STEPS):
                step(-1 - i)
            if hip_graph:
                # The request is launch-bound (hundreds of short kernels): capture
                # the forward pass once, un-captured by the scheduler, and replay
                # it per request as a single hipGraphLaunch record.
                torch.cuda.synchronize()
                state["graph_in"] = torch.zeros(data.shape, dtype=data.dtype, device=device)
                graph = torch.cuda.CUDAGraph()
                # thread_local: what the other clients' threads do meanwhile
                # (allocations, pinning) is not part of this capture
                with torch.no_grad(), torch.cuda.graph(graph, stream=stream,
                                                       capture_error_mode="thread_local"):
                    state["graph_out"] = model(state["graph_in"].to(tdtype))
                torch.cuda.synchronize()
                state["graph"] = graph
                for i in range(2):
                    step(-10 - i)
                torch.cuda.synchronize()
        result = cc.run_client(tid, train, num_iters, sleep_times, barriers, step,
                               backend, extra=extra)
    print(f"Client {tid} finished: {cc.brief(result)}", flush=True)
    return result
