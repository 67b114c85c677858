"""The CPU-only configuration: ResNet-50 inference, batch 4, fp32, random-init
weights, seeded N(0,1) input, on the PyTorch CPU path; and the scheduler policy
replayed on the CPU over that model's kernel trace and profile -- here the
profiles captured on an MI355X for the headline pair (tests/golden/
mi355x_resnet50/, written by tests/golden/make_profile_fixture.py), run under
the deterministic virtual-time model.  The native core must reproduce the
oracle's decision sequence bit for bit."""

import os

import numpy as np
import pytest
import torch

from oracle import obslog, policy_oracle as po, virtual_gpu as vg
from tests import jobs

FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mi355x_resnet50")
HP = os.path.join(FIX, "hp_resnet50_bs4_bf16_inference.csv")
BE = os.path.join(FIX, "be_resnet50_bs32_fp32_training.csv")
BUDGET_NS = 160_000       # the reference's own budget for this pair


def test_resnet50_cpu_forward_is_seeded_and_shaped():
    from orion_amd.benchmark_suite import client_common as cc
    from orion_amd.benchmark_suite.train_imagenet import DummyDataLoader
    from orion_amd.benchmark_suite.vision_models import resnet50
    outs = []
    for _ in range(2):
        with cc.MODEL_INIT_LOCK:
            cc.seed_everything(42)
            model = resnet50().eval()
        data, _ = next(DummyDataLoader(4, 42))
        assert data.shape == (4, 3, 224, 224) and data.dtype == torch.float32
        with torch.no_grad():
            outs.append(model(data))
    assert sum(p.numel() for p in model.parameters()) == 25_557_032
    assert outs[0].shape == (4, 1000) and torch.isfinite(outs[0]).all()
    assert torch.equal(outs[0], outs[1])
    # N(0,1) input: sample moments of 602112 values
    assert abs(float(data.mean())) < 0.01 and abs(float(data.std()) - 1.0) < 0.01


def test_fixture_profiles_have_the_shape_of_the_pair():
    hp, be = po.parse_profile(HP), po.parse_profile(BE)
    assert len(hp) == 371 and len(be) == 713
    assert abs(sum(float(o.duration) for o in hp) / 1e6 - 1.971) < 0.01   # ms of kernels
    assert abs(sum(float(o.duration) for o in be) / 1e6 - 17.27) < 0.05
    assert max(o.sm_used for o in be) == 12544
    assert {o.profile for o in hp} == {-1, 0, 1}
    assert sum(1 for o in be if float(o.duration) > BUDGET_NS) == 4


@pytest.fixture(scope="module")
def replayed():
    hp_iters = 25
    profiles = [po.parse_profile(BE), po.parse_profile(HP)]
    oracle = po.PolicyOracle(profiles, [713, 371], [10_000, hp_iters], [True, False],
                             max_sms=256, sequential_fix=True)
    gaps = (np.random.default_rng(7).exponential(1 / 80.0, 64) * 1e9).astype(np.int64)
    be_trace = [po.MEMCPY] + [po.KERNEL] * 713
    hp_trace = [po.MEMCPY] + [po.KERNEL] * 371 + [po.MEMCPY]
    clients = [vg.VClient(lambda it: be_trace, 10_000, gap_ns=1500),
               vg.VClient(lambda it: hp_trace, hp_iters, gap_ns=2000,
                          arrivals=[int(g) for g in gaps])]
    env = vg.VirtualGpu(clients, lambda c, k: int(oracle.ops[c][k].duration))
    masks = [32, 64, 128, 256]
    rec = obslog.RecordingEnv(env, 2, masks, lambda c, k: oracle.ops[c][k],
                              algo=po.ALGO_ORION, hp_active=lambda: oracle.seen[1] > 0)
    rec.budget = BUDGET_NS
    rec.header(256, [(713, 10_000, True, BE), (371, hp_iters, False, HP)],
               confine_long=True)
    vg.run_job(oracle, env, rec, [(True, 1), (True, 10), (False, 0)], algo=po.ALGO_ORION,
               depth=BUDGET_NS, hp_limit=1, update_start=1, max_polls=30_000_000)
    return oracle, env, rec, hp_iters


def test_policy_replay_over_the_resnet50_trace_is_bit_exact(replayed):
    oracle, env, rec, hp_iters = replayed
    obs, dec = rec.obs_text(), rec.dec.text()
    assert dec.count("\nD ") > 20_000
    assert jobs.native_replay(obs) == dec          # native core, bit for bit
    assert obslog.replay(obs) == dec               # and the log is self-contained


def test_what_the_policy_did_on_that_trace(replayed):
    oracle, env, rec, hp_iters = replayed
    d = [l.split() for l in rec.dec.text().splitlines() if l.startswith("D ")]
    hp = [x for x in d if x[1] == "1"]
    # every high-priority record of every request was dispatched, in order
    assert len(hp) == hp_iters * (371 + 2)
    ks = [int(x[4]) for x in hp if x[3] == po.KERNEL]
    assert ks == list(range(371)) * hp_iters
    # with the confinement option on (header token L1), best-effort kernels that
    # alone outlast the budget never got the whole GPU; short ones did whenever
    # the high-priority client was idle
    be = [x for x in d if x[1] == "0" and x[3] == po.KERNEL]
    long_ops = {k for k, o in enumerate(oracle.ops[0]) if float(o.duration) > BUDGET_NS}
    assert long_ops and all(int(x[6]) < 3 for x in be if int(x[4]) in long_ops)
    assert any(int(x[6]) == 3 for x in be if int(x[4]) not in long_ops)
    # the best-effort trainer made progress beside 25 requests
    assert oracle.cur_iters[0] > 10
