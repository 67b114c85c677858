"""The Transformer-XL client's model and optimiser (CPU, small sizes).

The model is this build's own statement of the architecture the reference's
client instantiates (transformer_trainer.py:63-86).  Pinned here by what the
mathematics fixes: the relative shift against explicit indexing, attention
against the per-pair formula of the paper, the adaptive softmax against a
normalised distribution, and the segment-recurrence identity -- a sequence run
in two segments with memory gives the hidden states of one pass over both.
"""

import math

import numpy as np
import pytest
import torch

from orion_amd.benchmark_suite import transformer_xl as txl

SMALL = dict(n_token=97, n_layer=3, n_head=2, d_model=16, d_head=8, d_inner=32, dropout=0.0,
             dropatt=0.0, dtype=None, tie_weight=True, d_embed=16, div_val=1,
             tie_projs=[False, True, True], pre_lnorm=False, tgt_len=6, ext_len=0, mem_len=6,
             cutoffs=[20, 50], same_length=False, attn_type=0, clamp_len=-1, sample_softmax=-1)


def test_relative_shift_is_the_explicit_reindexing():
    qlen, mlen = 5, 3
    klen = qlen + mlen
    x = torch.arange(2 * qlen * klen, dtype=torch.float32).view(2, qlen, klen)
    y = txl.relative_shift(x)
    for i in range(qlen):
        for j in range(mlen + i + 1):              # visible keys only
            dist = mlen + i - j
            assert torch.equal(y[:, i, j], x[:, i, klen - 1 - dist])


def test_attention_is_the_papers_per_pair_formula():
    torch.manual_seed(0)
    qlen, mlen, bsz, h, dh, d = 4, 3, 2, 2, 8, 16
    klen = qlen + mlen
    att = txl.RelativeAttention(h, d, dh, dropout=0.0).double()
    x, mem = torch.randn(qlen, bsz, d).double(), torch.randn(mlen, bsz, d).double()
    u, v = torch.randn(h, dh).double(), torch.randn(h, dh).double()
    table = txl.sinusoid_table(torch.arange(klen - 1, -1, -1), d, torch.float64)
    mask = torch.full((qlen, klen), float("-inf"), dtype=torch.float64).triu(1 + mlen)
    got = att(x, table, u, v, mask, mem)

    ctx = torch.cat([mem, x])
    qkv = att.qkv(ctx).view(klen, bsz, 3, h, dh)
    out = torch.zeros(qlen, bsz, h * dh, dtype=torch.float64)
    for b in range(bsz):
        for n in range(h):
            for i in range(qlen):
                q = qkv[mlen + i, b, 0, n]
                scores = []
                for j in range(mlen + i + 1):
                    r = att.pos(txl.sinusoid_table(torch.tensor([mlen + i - j]), d,
                                                   torch.float64))[0].view(h, dh)[n]
                    k = qkv[j, b, 1, n]
                    scores.append((q + u[n]) @ k + (q + v[n]) @ r)
                p = torch.softmax(torch.stack(scores) / math.sqrt(dh), dim=0)
                out[i, b, n * dh:(n + 1) * dh] = sum(
                    p[j] * qkv[j, b, 2, n] for j in range(mlen + i + 1))
    want = att.norm(x + att.out(out))
    assert torch.allclose(got, want, atol=1e-10)


def test_adaptive_softmax_is_a_distribution_and_forward_reads_it():
    torch.manual_seed(1)
    crit = txl.AdaptiveLogSoftmax(97, 16, [20, 50])
    for p in crit.parameters():
        torch.nn.init.normal_(p, 0.0, 0.5)
    hidden = torch.randn(40, 16)
    full = crit.full_logprob(hidden)
    assert full.shape == (40, 97)
    assert torch.allclose(full.exp().sum(dim=1), torch.ones(40), atol=1e-5)
    target = torch.randint(0, 97, (40,), generator=torch.Generator().manual_seed(2))
    target[:3] = torch.tensor([0, 20, 96])                      # cluster edges
    nll = crit(hidden, target)
    assert torch.allclose(nll, -full.gather(1, target[:, None]).squeeze(1), atol=1e-5)
    # a batch that never leaves the head (the reference's all-ones input)
    ones = torch.ones(40, dtype=torch.int64)
    assert torch.allclose(crit(hidden, ones), -full[:, 1], atol=1e-5)


def test_two_segments_with_memory_equal_one_pass():
    torch.manual_seed(3)
    model = txl.MemTransformerLM(**SMALL).eval()
    data = torch.randint(0, 97, (12, 2))
    target = torch.randint(0, 97, (12, 2))
    with torch.no_grad():
        whole, _ = model(data, target, None)
        first, mems = model(data[:6], target[:6], None)
        second, mems2 = model(data[6:], target[6:], mems)
    assert mems.shape == (3, 6, 2, 16) and mems2.shape == (3, 6, 2, 16)
    assert torch.allclose(torch.cat([first, second]), whole, atol=1e-5)
    # and the future does not leak: changing a later token leaves earlier losses alone
    data2 = data.clone()
    data2[9] = (data2[9] + 1) % 97
    with torch.no_grad():
        changed, _ = model(data2, target, None)
    assert torch.equal(changed[:9], whole[:9]) and not torch.equal(changed[9:], whole[9:])


def test_memory_keeps_the_last_mem_len_layer_inputs():
    torch.manual_seed(4)
    cfg = dict(SMALL, mem_len=4)
    model = txl.MemTransformerLM(**cfg).eval()
    data = torch.randint(0, 97, (6, 1))
    with torch.no_grad():
        _, mems = model(data, data, None)
        assert mems.shape == (3, 4, 1, 16)
        emb = model.word_emb(data) * math.sqrt(16)
        assert torch.allclose(mems[0], emb[-4:])
        _, mems = model(data, data, mems)
        assert mems.shape == (3, 4, 1, 16)


def test_variants_that_are_not_built_are_refused():
    with pytest.raises(ValueError):
        txl.MemTransformerLM(**dict(SMALL, attn_type=2))
    with pytest.raises(ValueError):
        txl.MemTransformerLM(**dict(SMALL, div_val=4))
    with pytest.raises(ValueError):
        txl.MemTransformerLM(**dict(SMALL, d_embed=8))


def test_lamb_step_by_hand():
    """related/baselines/transformer/lamb.py:108-144, worked with numpy."""
    w = torch.nn.Parameter(torch.tensor([3.0, -4.0, 12.0]))      # norm 13 -> clamped to 10
    z = torch.nn.Parameter(torch.zeros(2))                       # zero weight: ratio 1
    opt = txl.Lamb([w, z], lr=0.1, weight_decay=0.01)
    grads = [np.array([1.0, 2.0, -2.0]), np.array([0.5, -0.5])]
    state = [dict(m=np.zeros(3), v=np.zeros(3), p=np.array([3.0, -4.0, 12.0])),
             dict(m=np.zeros(2), v=np.zeros(2), p=np.zeros(2))]
    for step in range(3):
        for p, g in zip((w, z), grads):
            p.grad = torch.tensor(g * (step + 1), dtype=torch.float32)
        opt.step()
        for s, g in zip(state, grads):
            g = g * (step + 1)
            s["m"] = 0.9 * s["m"] + 0.1 * g
            s["v"] = 0.999 * s["v"] + 0.001 * g * g
            upd = s["m"] / (np.sqrt(s["v"]) + 1e-6) + 0.01 * s["p"]
            wn, un = min(np.linalg.norm(s["p"]), 10.0), np.linalg.norm(upd)
            ratio = 1.0 if wn == 0 or un == 0 else wn / (un + 1e-6)
            s["p"] = s["p"] - 0.1 * ratio * upd
        assert np.allclose(w.detach().numpy(), state[0]["p"], rtol=1e-5)
        assert np.allclose(z.detach().numpy(), state[1]["p"], rtol=1e-5, atol=1e-7)


def test_the_clients_configuration_is_the_references():
    from orion_amd.benchmark_suite import transformer_trainer as tt
    cfg = tt.MODEL_CONFIG
    assert (cfg["n_layer"], cfg["n_head"], cfg["d_model"], cfg["d_head"], cfg["d_inner"]) == \
        (16, 8, 512, 64, 2048)
    assert cfg["n_token"] == 267735 and cfg["cutoffs"] == [19997, 39997, 199997]
    assert cfg["tgt_len"] == cfg["mem_len"] == 192
    loader = tt.DummyDataLoader(4, 42)
    data, target = loader.batch()
    assert data.shape == target.shape == (192, 4) and data.dtype == torch.int64
    assert int(data.max()) < 267735 and int(data.max()) > 199997      # reaches the last cluster
