"""The three co-location configurations of the job description, in their stated
form, through the whole hot path on the GPU (about 40 high-priority requests
each; bench.py measures the same jobs at length):

* configs[2]: ResNet-50 inference bs4 bf16 at Poisson 80 req/s beside
  ResNet-50 training bs32, SGD momentum 0.9;
* configs[3]: MobileNetV2 inference bs4 bf16 at Poisson 100 req/s beside
  BERT-base training (12 x 768 x 12), seq 384, bs8, AdamW;
* configs[4]: BERT-large inference (24 x 1024 x 16), seq 384, bs8, closed loop,
  beside ResNet-50 bs32, MobileNetV2 bs64 and BERT-base bs8 training.

Checked for each: the high-priority client's output tensor against its
isolated run and against the PyTorch CPU fp32 reference of the same model and
input; the decision log the live scheduler recorded, replayed bit-exactly by
the CPU oracle and by the native policy core (and the reference loop's per-poll
rules on it); every best-effort client made progress.

Tolerances.  The job description's 1e-3 (relative to the largest reference
value) is what an fp32 client meets (tests/test_colocation_gpu.py).  These
clients compute in bf16 -- 8 significand bits, unit roundoff 2^-9 = 2.0e-3 per
rounding -- so against an fp32 reference the bound is the accumulated rounding
of the network's depth, the *_RTOL values below: one and a half times what was
measured on an MI355X -- 7.7e-3 (ResNet-50; 5.1e-3 with deterministic solvers),
2.6e-2 (MobileNetV2, whose depthwise layers have short accumulations that do
not average the roundings out) and 3.4e-2 (BERT-large, 24 layers) -- and
measured values are appended to a file in the directory ORION_TEST_REPORT_DIR
names, when it is set.  Between the isolated and the
co-located run of the same bf16 client only the order of atomic accumulations
can differ (split-K convolution and GEMM solvers).  configs[2] and configs[3]
therefore run twice: with the libraries' default solvers -- the kernels bench.py
measures -- where the two runs may differ by that rounding (bounded by
DEFAULT_SOLVER_DRIFT, a bf16 roundoff or two of the largest output), and with
deterministic solvers, where the two outputs must be equal to the bit.

The best-effort trainers are compared with their own run alone at fixed points:
the loss of scheduled iteration 0 and of iteration 11, which depends on every
update before it.  Measured on the MI355X (ResNet-50 bs32, nine checkpoints):
alone, alone again and on a plain stream the trainer reproduces every loss to
the bit, with either solver set; beside the inference client it does so in some
runs and departs in the last bits from iteration 2 on in others, with either
solver set -- PyTorch's own max-pool backward kernel accumulates with atomics,
whose order follows the compute units the kernel lands on, and the scheduler
moves best-effort kernels between CU masks.  From there the trajectory is as
ill-conditioned as training on random labels is: at the reference's learning
rate of 0.1 the last-bit difference grows to tens of percent within ten
iterations (so do two runs alone under the default solvers).  The tests
therefore train with lr = 0.001 (the job description fixes the optimizer and
its momentum, not the rate; the kernels are the same) and assert: iteration 0
equal to the bit under deterministic solvers (the forward pass of the first
scheduled iteration, after a warm-up that runs alone), the later one within
TRAINER_LOSS_RTOL (measured: up to 2e-3) under both.
"""

import copy
import json
import os

import pytest
import torch

import bench
from tests.test_colocation_gpu import _check_replay

pytestmark = pytest.mark.gpu

RESNET_RTOL = 1.2e-2      # bf16 client against the CPU fp32 reference, per model:
MOBILENET_RTOL = 4e-2     # 1.5 x the error measured on an MI355X
BERT_LARGE_RTOL = 5e-2    # (7.7e-3, 2.6e-2 and 3.4e-2 with the default solvers)
# default solvers: the same bf16 client, alone and co-located, may differ by the
# order of atomic accumulations -- a few bf16 roundoffs (2^-9 each) of the largest
# output value; measured 3.9e-3 (ResNet-50) and 6.8e-3 (MobileNetV2)
DEFAULT_SOLVER_DRIFT = 1.2e-2
REQUESTS = 50
LOSS_ITERATION = 11       # past the ten warm-up iterations of the job protocol
TRAINER_LOSS_RTOL = 2e-2  # trainer's loss at LOSS_ITERATION, beside the client vs alone
TRAINER_LR = 0.001


@pytest.fixture(scope="module")
def profile_dir(tmp_path_factory):
    """One profile directory for the three jobs: they share two trainers."""
    return str(tmp_path_factory.mktemp("profiles"))


def _run(work, job, budget, profiles, be_alone=()):
    """Runs the high-priority client alone and the whole job.  ``be_alone``:
    indices of best-effort trainers that are also run alone (25 iterations), for
    their loss at LOSS_ITERATION; returned as the last element, index -> result."""
    from orion_amd import colocate
    from orion_amd.profiling import capture_profile
    cfg = os.path.join(work, "job.json")
    with open(cfg, "w") as f:
        json.dump(job, f)
    filled = capture_profile.fill_job(cfg, profiles, os.path.join(work, "filled.json"),
                                      quiet=True, reuse=True)
    iso_dir, co_dir = os.path.join(work, "iso_out"), os.path.join(work, "co_out")
    os.makedirs(iso_dir)
    os.makedirs(co_dir)
    loss_env = {"ORION_LOSS_AT_ITERATION": f"0,{LOSS_ITERATION}"}
    colocate.run_job([copy.deepcopy(filled[-1])], "orion", os.path.join(work, "iso"), budget,
                     env={"ORION_SAVE_OUTPUT_DIR": iso_dir})
    co = colocate.run_job(copy.deepcopy(filled), "orion", os.path.join(work, "co"), budget,
                          env=dict(loss_env, ORION_SAVE_OUTPUT_DIR=co_dir,
                                   ORION_RECORD_DIR=co_dir))
    alone = {}
    for k in be_alone:
        entry = copy.deepcopy(filled[k])
        entry["num_iters"] = LOSS_ITERATION + 13
        alone[k] = colocate.run_job([entry], "orion", os.path.join(work, f"be{k}_alone"), budget,
                                    env=loss_env)[0]
    hp = len(job) - 1
    iso_out = torch.load(os.path.join(iso_dir, "client_0_output.pt"), weights_only=True)
    co_out = torch.load(os.path.join(co_dir, f"client_{hp}_output.pt"), weights_only=True)
    return filled, co, iso_out, co_out, co_dir, alone


def _report(name, **values):
    report_dir = os.environ.get("ORION_TEST_REPORT_DIR")
    if report_dir and os.path.isdir(report_dir):
        with open(os.path.join(report_dir, "stated_configs_errors.jsonl"), "a") as f:
            f.write(json.dumps({"config": name, **values}) + "\n")


def _vision_reference(model_name, batch):
    from orion_amd.benchmark_suite import client_common as cc
    from orion_amd.benchmark_suite.train_imagenet import DummyDataLoader
    from orion_amd.benchmark_suite.vision_models import MODELS
    with cc.MODEL_INIT_LOCK:
        cc.seed_everything(42)
        model = MODELS[model_name](num_classes=1000).eval()
    data, _ = next(DummyDataLoader(batch, 42))
    with torch.no_grad():
        return model(data.float())


def _rel(a, b, ref):
    return float((a - b).abs().max() / ref.abs().max())


def _trainer_losses(co_result, alone_result, bit_exact_first):
    """[iteration, alone, co-located] per checkpoint, after the assertions."""
    co, alone = co_result["loss_at_iteration"], alone_result["loss_at_iteration"]
    last = str(LOSS_ITERATION)
    assert set(co) == set(alone) == {"0", last}, (co, alone)
    if bit_exact_first:
        assert co["0"][1] == alone["0"][1], (co["0"], alone["0"])
    for it in ("0", last):
        assert abs(co[it][0] - alone[it][0]) <= TRAINER_LOSS_RTOL * abs(alone[it][0]), \
            (it, co[it], alone[it])
    return [[int(it), alone[it][0], co[it][0]] for it in ("0", last)]


def _c3_job():
    job = bench.c3_job(REQUESTS + 10)
    assert job[0]["args"] == {"batchsize": 32, "rps": 0, "uniform": False, "dummy_data": True,
                              "train": True, "dtype": "fp32", "model_name": "resnet50",
                              "momentum": 0.9}
    assert (job[-1]["args"]["batchsize"], job[-1]["args"]["rps"], job[-1]["args"]["dtype"],
            job[-1]["args"]["uniform"]) == (4, 80, "bf16", False)
    return job


def _records(filled):
    return [f.get("additional_num_kernels") or f["num_kernels"] for f in filled]


def test_resnet50_bf16_poisson_beside_resnet50_training_bs32(tmp_path, profile_dir):
    """configs[2] with the libraries' DEFAULT solvers: the kernels the bench
    measures (assembly Winograd and implicit-GEMM convolutions, some of which
    accumulate with atomics)."""
    job = _c3_job()
    job[0]["args"]["lr"] = TRAINER_LR
    filled, co, iso_out, co_out, co_dir, alone = _run(str(tmp_path), job, 160_000, profile_dir,
                                                      be_alone=(0,))
    assert co[-1]["iterations"] == REQUESTS + 10 and co[0]["iterations"] > LOSS_ITERATION
    ref = _vision_reference("resnet50", 4)
    err, drift = _rel(co_out, ref, ref), _rel(co_out, iso_out, ref)
    losses = _trainer_losses(co[0], alone[0], bit_exact_first=False)
    _report("c3_default_solvers", hp_vs_cpu_fp32=err, hp_vs_isolated=drift,
            be_iterations=co[0]["iterations"], records=_records(filled),
            be_loss_iteration_alone_colocated=losses)
    assert err <= RESNET_RTOL, err
    assert drift <= DEFAULT_SOLVER_DRIFT, drift
    _check_replay(co_dir)


def test_resnet50_pair_with_deterministic_solvers_is_bit_exact(tmp_path, profile_dir):
    """configs[2] again with solvers that do not accumulate with atomics (im2col +
    GEMM instead of the assembly kernels: more, other records): the inference
    client computes, bit for bit, what it computes alone; so does the trainer in
    its first scheduled iteration, and to TRAINER_LOSS_RTOL eleven iterations on
    (see the module docstring)."""
    job = _c3_job()
    job[0]["args"]["lr"] = TRAINER_LR
    for entry in job:
        entry["args"]["deterministic"] = True
    filled, co, iso_out, co_out, co_dir, alone = _run(str(tmp_path), job, 160_000, profile_dir,
                                                      be_alone=(0,))
    assert co[-1]["iterations"] == REQUESTS + 10 and co[0]["iterations"] > LOSS_ITERATION
    assert torch.equal(iso_out, co_out), float((iso_out - co_out).abs().max())
    losses = _trainer_losses(co[0], alone[0], bit_exact_first=True)
    ref = _vision_reference("resnet50", 4)
    err = _rel(co_out, ref, ref)
    _report("c3_deterministic", hp_vs_cpu_fp32=err, hp_vs_isolated=0.0,
            be_iterations=co[0]["iterations"], records=_records(filled),
            be_loss_iteration_alone_colocated=losses)
    assert err <= RESNET_RTOL, err
    _check_replay(co_dir)


def _c4_job():
    job = bench.c4_job(REQUESTS + 10)
    assert job[0]["arch"] == "bert" and job[0]["args"]["batchsize"] == 8 and job[0]["args"]["train"]
    assert (job[-1]["args"]["batchsize"], job[-1]["args"]["rps"], job[-1]["args"]["dtype"]) == \
        (4, 100, "bf16")
    return job


def test_mobilenet_bf16_poisson_beside_bert_base_training_bs8(tmp_path, profile_dir):
    """configs[3] with default solvers."""
    job = _c4_job()
    filled, co, iso_out, co_out, co_dir, alone = _run(str(tmp_path), job, 100_000, profile_dir,
                                                      be_alone=(0,))
    assert co[-1]["iterations"] == REQUESTS + 10 and co[0]["iterations"] > LOSS_ITERATION
    assert _records(filled)[0] > 500
    ref = _vision_reference("mobilenet_v2", 4)
    err, drift = _rel(co_out, ref, ref), _rel(co_out, iso_out, ref)
    losses = _trainer_losses(co[0], alone[0], bit_exact_first=False)
    _report("c4_default_solvers", hp_vs_cpu_fp32=err, hp_vs_isolated=drift,
            be_iterations=co[0]["iterations"], records=_records(filled),
            be_loss_iteration_alone_colocated=losses)
    assert err <= MOBILENET_RTOL, err
    # depthwise convolutions may take a solver that accumulates with atomics:
    # the two runs agree to bf16 rounding, not necessarily to the bit
    assert drift <= DEFAULT_SOLVER_DRIFT, drift
    _check_replay(co_dir)


def test_mobilenet_pair_with_deterministic_solvers_is_bit_exact(tmp_path, profile_dir):
    """configs[3] with deterministic solvers: the inference client's output and
    the BERT trainer's first loss equal, to the bit, those of their runs alone."""
    job = _c4_job()
    for entry in job:
        entry["args"]["deterministic"] = True
    filled, co, iso_out, co_out, co_dir, alone = _run(str(tmp_path), job, 100_000, profile_dir,
                                                      be_alone=(0,))
    assert co[-1]["iterations"] == REQUESTS + 10 and co[0]["iterations"] > LOSS_ITERATION
    assert torch.equal(iso_out, co_out), float((iso_out - co_out).abs().max())
    losses = _trainer_losses(co[0], alone[0], bit_exact_first=True)
    ref = _vision_reference("mobilenet_v2", 4)
    err = _rel(co_out, ref, ref)
    _report("c4_deterministic", hp_vs_cpu_fp32=err, hp_vs_isolated=0.0,
            be_iterations=co[0]["iterations"], records=_records(filled),
            be_loss_iteration_alone_colocated=losses)
    assert err <= MOBILENET_RTOL, err
    _check_replay(co_dir)


def test_bert_large_closed_loop_beside_three_trainers(tmp_path, profile_dir):
    from transformers import BertForQuestionAnswering
    from orion_amd.benchmark_suite import bert_trainer as bt
    from orion_amd.benchmark_suite import client_common as cc
    job = bench.c5_job(REQUESTS + 50)      # the BERT inference loop drops 50 requests (warm-up)
    assert [j["arch"] for j in job] == ["resnet50", "mobilenet_v2", "bert", "bert"]
    assert [j["args"]["batchsize"] for j in job] == [32, 64, 8, 8]
    assert job[-1]["args"]["rps"] == 0 and not job[-1]["args"]["train"]
    filled, co, iso_out, co_out, co_dir, _ = _run(str(tmp_path), job, 100_000, profile_dir)
    assert co[-1]["iterations"] == REQUESTS + 50
    for k in range(3):
        assert co[k]["iterations"] >= 10, (k, co[k])
    with cc.MODEL_INIT_LOCK:
        cc.seed_everything(42)
        model = BertForQuestionAnswering(bt.bert_config(False)).eval()
    ids, seg, mask, _, _ = bt.DummyDataLoader(8, 42).batch()
    with torch.no_grad():
        out = model(input_ids=ids, token_type_ids=seg, attention_mask=mask)
        ref = torch.stack([out.start_logits, out.end_logits])
    assert co_out.shape == ref.shape == (2, 8, 384)
    err, drift = _rel(co_out, ref, ref), _rel(co_out, iso_out, ref)
    _report("c5", hp_vs_cpu_fp32=err, hp_vs_isolated=drift,
            be_iterations=[co[k]["iterations"] for k in range(3)],
            records=[f.get("additional_num_kernels", f["num_kernels"]) for f in filled])
    assert err <= BERT_LARGE_RTOL, err
    # the inference kernels of this model accumulate without atomics: beside three
    # trainers the client computes, bit for bit, what it computes alone
    assert torch.equal(iso_out, co_out), drift
    _check_replay(co_dir)
