"""BERT client: BERT-base training (12 x 768 x 12 heads) or BERT-large
inference (24 x 1024 x 16 heads), sequence length 384, question-answering head.

Counterpart of the reference's ``bert_loop``
(benchmarking/benchmark_suite/bert_trainer_mock.py:49-234): the model size is
chosen by ``train`` exactly as there (:69-96), the vocabulary is padded to a
multiple of 8 (:99-100), the loss is the mean of the start and end
cross-entropies (:146-150).  The reference builds the model from NVIDIA's
DeepLearningExamples and optimises with its BertAdam; here the architecture
comes from a local ``transformers.BertConfig`` (nothing is downloaded) and the
optimiser is AdamW with the same weight-decay grouping (:109-118).  Synthetic
inputs follow the job description: token ids uniform over the vocabulary, span
labels uniform over the sequence (the reference uses all-ones ids).
"""

import os
import threading

import torch

from . import client_common as cc

SEQ_LEN = 384
VOCAB = 30522


def bert_config(train):
    with cc.MODEL_INIT_LOCK:   # re-entrant; transformers' lazy imports are not thread-safe
        from transformers import BertConfig
    vocab = VOCAB + (8 - VOCAB % 8) % 8
    if train:
        return BertConfig(vocab_size=vocab, hidden_size=768, num_hidden_layers=12,
                          num_attention_heads=12, intermediate_size=3072,
                          max_position_embeddings=512, type_vocab_size=2)
    return BertConfig(vocab_size=vocab, hidden_size=1024, num_hidden_layers=24,
                      num_attention_heads=16, intermediate_size=4096,
                      max_position_embeddings=512, type_vocab_size=2)


class DummyDataLoader:
    def __init__(self, batchsize, seed):
        g = torch.Generator().manual_seed(seed)
        shape = (batchsize, SEQ_LEN)
        self.input_ids = torch.randint(0, VOCAB, shape, generator=g)
        self.segment_ids = torch.zeros(shape, dtype=torch.int64)
        self.input_mask = torch.ones(shape, dtype=torch.int64)
        self.start_positions = torch.randint(0, SEQ_LEN, (batchsize,), generator=g)
        self.end_positions = torch.randint(0, SEQ_LEN, (batchsize,), generator=g)
        if torch.cuda.is_available():
            for k, v in list(vars(self).items()):
                setattr(self, k, v.pin_memory())

    def batch(self):
        return (self.input_ids, self.segment_ids, self.input_mask,
                self.start_positions, self.end_positions)


def bert_loop(batchsize, train, num_iters, rps, uniform, dummy_data, local_rank,
              barriers, client_barrier, tid, dtype="fp32", seed=42, deterministic=False):
    with cc.MODEL_INIT_LOCK:   # transformers' lazy imports are not thread-safe
        from transformers import BertForQuestionAnswering
    cc.seed_everything(seed)
    if deterministic:   # process-wide, see train_imagenet.imagenet_loop
        torch.backends.cudnn.deterministic = True
    backend = cc.Backend()
    sleep_times = cc.arrival_gaps(rps, uniform, num_iters, "", seed)
    barriers[0].wait()
    print(f"-------------- client {tid} thread id: {threading.get_native_id()}",
          flush=True)

    device = torch.device("cuda", local_rank)
    tdtype = {"fp32": torch.float32, "bf16": torch.bfloat16}[dtype]
    stream = torch.cuda.Stream(device=device)
    backend.register_stream(stream)
    with torch.cuda.stream(stream), torch.autograd.set_multithreading_enabled(False):
        with cc.uncaptured(backend):
            with cc.MODEL_INIT_LOCK:
                cc.seed_everything(seed)
                model = BertForQuestionAnswering(bert_config(train))
            model = model.to(device)
            if train:
                model.train()
                named = [(n, p) for n, p in model.named_parameters() if "pooler" not in n]
                no_decay = ["bias", "LayerNorm.bias", "LayerNorm.weight"]
                groups = [
                    {"params": [p for n, p in named if not any(nd in n for nd in no_decay)],
                     "weight_decay": 0.01},
                    {"params": [p for n, p in named if any(nd in n for nd in no_decay)],
                     "weight_decay": 0.0}]
                optimizer = torch.optim.AdamW(groups, lr=5e-5)
            else:
                model.eval()
                model = model.to(tdtype)
        host = DummyDataLoader(batchsize, seed).batch()
        state = {}

        def step(batch_idx):
            ids, seg, mask, sp, ep = [t.to(device, non_blocking=True) for t in host]
            if train:
                optimizer.zero_grad()
                with torch.autocast("cuda", dtype=torch.bfloat16, enabled=dtype == "bf16"):
                    out = model(input_ids=ids, token_type_ids=seg, attention_mask=mask)
                    ignored = out.start_logits.size(1)
                    loss_fct = torch.nn.CrossEntropyLoss(ignore_index=ignored)
                    loss = (loss_fct(out.start_logits, sp) + loss_fct(out.end_logits, ep)) / 2
                loss.backward()
                optimizer.step()
                state["loss"] = loss
                cc.keep_loss(state, batch_idx, loss)
            else:
                with torch.no_grad():
                    out = model(input_ids=ids, token_type_ids=seg, attention_mask=mask)
                    state["output"] = torch.stack([out.start_logits, out.end_logits])

        def extra():
            res = {}
            save_dir = os.environ.get("ORION_SAVE_OUTPUT_DIR")
            if save_dir and "output" in state:
                torch.save(state["output"].float().cpu(),
                           os.path.join(save_dir, f"client_{tid}_output.pt"))
            if "loss" in state:
                res["final_loss"] = float(state["loss"].detach().float().cpu())
            res.update(cc.loss_checkpoint_report(state))
            return res

        with cc.uncaptured(backend):
            for i in range(cc.UNCAPTURED_STEPS):
                step(-1 - i)
        # the reference drops 50 requests for BERT inference (:213-214)
        result = cc.run_client(tid, train, num_iters, sleep_times, barriers, step,
                               backend, drop=50 if not train and num_iters > 60 else 10,
                               extra=extra)
    print(f"Client {tid} finished: {cc.brief(result)}", flush=True)
    return result
