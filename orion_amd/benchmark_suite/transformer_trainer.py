"""Transformer-XL client: the 16-layer, d_model 512 language model over the
WikiText-103 vocabulary, 192 target tokens with a 192-token memory, training
with LAMB or open-loop inference.

Counterpart of the reference's ``transformer_loop``
(benchmarking/benchmark_suite/transformer_trainer.py:43-200): the model
configuration is the one written there (:63-86), the memory returned by one
step feeds the next (:121, :144), the training loss is the mean of the
per-token losses (:122), the optimiser is LAMB with lr 0.1 (:97).  The reference
never clears gradients (its ``zero_grad`` is commented out, :120), so they
accumulate from step to step; here they are cleared.  Synthetic inputs: token
ids and targets uniform over the vocabulary (the reference uses all ones, which
never leaves the first softmax cluster).
"""

import os
import threading

import torch

from . import client_common as cc
from .transformer_xl import Lamb, MemTransformerLM

TGT_LEN = 192

MODEL_CONFIG = {
    "n_token": 267735, "n_layer": 16, "n_head": 8, "d_model": 512, "d_head": 64,
    "d_inner": 2048, "dropout": 0.1, "dropatt": 0.0, "dtype": None, "tie_weight": True,
    "d_embed": 512, "div_val": 1, "tie_projs": [False, True, True, True],
    "pre_lnorm": False, "tgt_len": TGT_LEN, "ext_len": 0, "mem_len": 192,
    "cutoffs": [19997, 39997, 199997], "same_length": False, "attn_type": 0,
    "clamp_len": -1, "sample_softmax": -1,
}


class DummyDataLoader:
    def __init__(self, batchsize, seed, n_token=MODEL_CONFIG["n_token"]):
        g = torch.Generator().manual_seed(seed)
        self.data = torch.randint(0, n_token, (TGT_LEN, batchsize), generator=g)
        self.target = torch.randint(0, n_token, (TGT_LEN, batchsize), generator=g)
        if torch.cuda.is_available():
            self.data, self.target = self.data.pin_memory(), self.target.pin_memory()

    def batch(self):
        return self.data, self.target


def transformer_loop(batchsize, train, num_iters, rps, uniform, dummy_data, local_rank,
                     barriers, client_barrier, tid, input_file="", dtype="fp32", seed=42,
                     model_config=None):
    cc.seed_everything(seed)
    backend = cc.Backend()
    sleep_times = cc.arrival_gaps(rps, uniform, num_iters, input_file, seed)
    barriers[0].wait()
    print(f"-------------- client {tid} thread id: {threading.get_native_id()}",
          flush=True)

    config = dict(MODEL_CONFIG, **(model_config or {}))
    device = torch.device("cuda", local_rank)
    tdtype = {"fp32": torch.float32, "bf16": torch.bfloat16}[dtype]
    stream = torch.cuda.Stream(device=device)
    backend.register_stream(stream)
    with torch.cuda.stream(stream), torch.autograd.set_multithreading_enabled(False):
        with cc.uncaptured(backend):
            with cc.MODEL_INIT_LOCK:
                cc.seed_everything(seed)
                model = MemTransformerLM(**config)
            model = model.to(device)
            if train:
                model.train()
                optimizer = Lamb(model.parameters(), lr=0.1)
            else:
                model.eval()
                model = model.to(tdtype)
        host = DummyDataLoader(batchsize, seed, config["n_token"]).batch()
        state = {"mems": None}

        def step(batch_idx):
            data, target = [t.to(device, non_blocking=True) for t in host]
            if train:
                optimizer.zero_grad()
                with torch.autocast("cuda", dtype=torch.bfloat16, enabled=dtype == "bf16"):
                    loss, state["mems"] = model(data, target, state["mems"])
                    loss = loss.float().mean()
                loss.backward()
                optimizer.step()
                state["loss"] = loss
            else:
                with torch.no_grad():
                    state["output"], state["mems"] = model(data, target, state["mems"])

        def extra():
            res = {}
            save_dir = os.environ.get("ORION_SAVE_OUTPUT_DIR")
            if save_dir and "output" in state:
                torch.save(state["output"].float().cpu(),
                           os.path.join(save_dir, f"client_{tid}_output.pt"))
            if "loss" in state:
                res["final_loss"] = float(state["loss"].detach().float().cpu())
            return res

        with cc.uncaptured(backend):
            # the first step runs without a memory and the second with one: both
            # shapes are past before the scheduler counts kernels
            for i in range(cc.UNCAPTURED_STEPS):
                step(-1 - i)
        result = cc.run_client(tid, train, num_iters, sleep_times, barriers, step, backend,
                               extra=extra)
    print(f"Client {tid} finished: {cc.brief(result)}", flush=True)
    return result
