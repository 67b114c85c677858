"""Transformer-XL language model (Dai et al., 2019) and the LAMB optimiser, as
the reference's ``transformer`` client uses them.

The reference builds ``MemTransformerLM`` and ``lamb.Lamb`` from NVIDIA's
DeepLearningExamples (benchmarking/benchmark_suite/transformer_trainer.py:5-6,
configuration :63-86, optimiser :97).  This module is this build's own
statement of the same architecture for the one variant that configuration
selects: relative multi-head attention with learnable global biases
(``attn_type`` 0), post-layer-norm blocks, one embedding table shared with the
output layer (``div_val`` 1, ``tie_weight``), an adaptive softmax over the
vocabulary clusters given by ``cutoffs`` (Grave et al., 2017), and a memory of
the last ``mem_len`` hidden states per layer.

Shapes follow the reference: token ids and targets are time-major
``[tgt_len, batch]``; ``forward(data, target, mems)`` returns the per-token
negative log-likelihood ``[tgt_len, batch]`` and the new memory.

Attention runs through ``scaled_dot_product_attention``: the content term
(q + u)·k is the fused kernel's own product and the position term (q + v)·r,
shifted to relative offsets, goes in as its additive bias together with the
causal mask.
"""

import math

import torch
import torch.nn as nn
import torch.nn.functional as F


def relative_shift(x):
    """``x[..., i, p]`` holds query i against the p-th entry of a distance table
    ordered from the largest distance (klen - 1) down to 0.  Returns the tensor
    whose ``[..., i, j]`` is query i (absolute position mlen + i) against key j,
    i.e. distance mlen + i - j, for every j <= mlen + i; entries past the
    diagonal are meaningless and must be masked by the caller."""
    *lead, qlen, klen = x.shape
    x = F.pad(x, (1, 0))                                  # one zero column in front
    x = x.reshape(*lead, klen + 1, qlen)[..., 1:, :]      # drop one row: rows slide by one each
    return x.reshape(*lead, qlen, klen)


def sinusoid_table(distances, d_model, dtype):
    inv_freq = 1.0 / (10000 ** (torch.arange(0.0, d_model, 2.0, device=distances.device)
                                / d_model))
    angles = torch.outer(distances.float(), inv_freq)
    return torch.cat([angles.sin(), angles.cos()], dim=-1).to(dtype)


class RelativeAttention(nn.Module):
    def __init__(self, n_head, d_model, d_head, dropout):
        super().__init__()
        self.n_head, self.d_head = n_head, d_head
        self.qkv = nn.Linear(d_model, 3 * n_head * d_head, bias=False)
        self.pos = nn.Linear(d_model, n_head * d_head, bias=False)
        self.out = nn.Linear(n_head * d_head, d_model, bias=False)
        self.drop = nn.Dropout(dropout)
        self.norm = nn.LayerNorm(d_model)

    def forward(self, x, table, u, v, mask, mem):
        """x [qlen, B, d]; table [klen, d] (distances klen-1 .. 0); u, v [H, dh];
        mask [qlen, klen] additive (0 / -inf); mem [mlen, B, d] or None."""
        qlen, bsz, _ = x.shape
        h, dh = self.n_head, self.d_head
        ctx = x if mem is None or mem.size(0) == 0 else torch.cat([mem, x], dim=0)
        klen = ctx.size(0)
        q, k, val = self.qkv(ctx).view(klen, bsz, 3, h, dh).unbind(dim=2)
        q = q[-qlen:].permute(1, 2, 0, 3)                  # [B, H, qlen, dh]
        k = k.permute(1, 2, 0, 3)                          # [B, H, klen, dh]
        val = val.permute(1, 2, 0, 3)
        r = self.pos(table).view(klen, h, dh).permute(1, 0, 2)      # [H, klen, dh]
        scale = 1.0 / math.sqrt(dh)
        bias = relative_shift(torch.matmul(q + v[None, :, None, :], r.transpose(-1, -2)))
        bias = bias * scale + mask
        y = F.scaled_dot_product_attention(q + u[None, :, None, :], k, val,
                                           attn_mask=bias, scale=scale)
        y = y.permute(2, 0, 1, 3).reshape(qlen, bsz, h * dh)
        return self.norm(x + self.drop(self.out(y)))


class FeedForward(nn.Module):
    def __init__(self, d_model, d_inner, dropout):
        super().__init__()
        self.net = nn.Sequential(nn.Linear(d_model, d_inner), nn.ReLU(inplace=True),
                                 nn.Dropout(dropout), nn.Linear(d_inner, d_model),
                                 nn.Dropout(dropout))
        self.norm = nn.LayerNorm(d_model)

    def forward(self, x):
        return self.norm(x + self.net(x))


class AdaptiveLogSoftmax(nn.Module):
    """Negative log-likelihood under a two-level softmax: the head distributes
    over the first ``cutoffs[0]`` tokens plus one entry per tail cluster; a
    tail token's probability is its cluster's head probability times a softmax
    inside the cluster.  All clusters read slices of one ``[n_token, d]`` weight
    (the embedding table when tied) and one bias."""

    def __init__(self, n_token, d_model, cutoffs, weight=None):
        super().__init__()
        self.edges = [0] + list(cutoffs) + [n_token]
        self.n_clusters = len(cutoffs)
        self.weight = weight if weight is not None else nn.Parameter(
            torch.zeros(n_token, d_model))
        self.bias = nn.Parameter(torch.zeros(n_token))
        self.cluster_weight = nn.Parameter(torch.zeros(self.n_clusters, d_model))
        self.cluster_bias = nn.Parameter(torch.zeros(self.n_clusters))

    def head_logprob(self, hidden):
        short = self.edges[1]
        w = torch.cat([self.weight[:short], self.cluster_weight], dim=0)
        b = torch.cat([self.bias[:short], self.cluster_bias], dim=0)
        return F.log_softmax(F.linear(hidden, w, b), dim=-1)

    def forward(self, hidden, target):
        """hidden [n, d], target [n] -> nll [n] (in the order of the rows)."""
        head = self.head_logprob(hidden)
        short = self.edges[1]
        nll = torch.zeros_like(target, dtype=hidden.dtype)
        for c in range(self.n_clusters + 1):
            lo, hi = self.edges[c], self.edges[c + 1]
            rows = ((target >= lo) & (target < hi)).nonzero(as_tuple=False).squeeze(1)
            if rows.numel() == 0:
                continue
            local = target.index_select(0, rows) - lo
            head_rows = head.index_select(0, rows)
            if c == 0:
                logp = head_rows.gather(1, local[:, None]).squeeze(1)
            else:
                tail = F.log_softmax(F.linear(hidden.index_select(0, rows),
                                              self.weight[lo:hi], self.bias[lo:hi]), dim=-1)
                logp = head_rows[:, short + c - 1] + tail.gather(1, local[:, None]).squeeze(1)
            nll.index_copy_(0, rows, -logp)
        return nll

    def full_logprob(self, hidden):
        """Log-probability of every token, [n, n_token] (tests, small sizes)."""
        head = self.head_logprob(hidden)
        short = self.edges[1]
        parts = [head[:, :short]]
        for c in range(1, self.n_clusters + 1):
            lo, hi = self.edges[c], self.edges[c + 1]
            tail = F.log_softmax(F.linear(hidden, self.weight[lo:hi], self.bias[lo:hi]), dim=-1)
            parts.append(head[:, short + c - 1, None] + tail)
        return torch.cat(parts, dim=1)


# keys of the reference's configuration that select other variants of the
# model; only the values below are built
_FIXED = {"div_val": 1, "pre_lnorm": False, "ext_len": 0, "same_length": False,
          "attn_type": 0, "clamp_len": -1, "sample_softmax": -1, "tie_weight": True}


class MemTransformerLM(nn.Module):
    def __init__(self, n_token, n_layer, n_head, d_model, d_head, d_inner, dropout,
                 dropatt=0.0, dtype=None, d_embed=None, tie_projs=None, tgt_len=None,
                 mem_len=None, cutoffs=(), **variant):
        super().__init__()
        for key, value in variant.items():
            if key not in _FIXED or _FIXED[key] != value:
                raise ValueError(f"Transformer-XL variant {key}={value!r} is not built")
        if d_embed not in (None, d_model):
            raise ValueError("d_embed must equal d_model (div_val 1, no projection)")
        if dropatt:
            raise ValueError("attention dropout is not built (the reference uses 0.0)")
        self.n_layer, self.d_model, self.tgt_len, self.mem_len = n_layer, d_model, tgt_len, mem_len
        self.word_emb = nn.Embedding(n_token, d_model)
        self.drop = nn.Dropout(dropout)
        self.u = nn.Parameter(torch.zeros(n_head, d_head))   # content bias (r_w_bias)
        self.v = nn.Parameter(torch.zeros(n_head, d_head))   # position bias (r_r_bias)
        self.attn = nn.ModuleList(RelativeAttention(n_head, d_model, d_head, dropout)
                                  for _ in range(n_layer))
        self.ff = nn.ModuleList(FeedForward(d_model, d_inner, dropout) for _ in range(n_layer))
        self.crit = AdaptiveLogSoftmax(n_token, d_model, list(cutoffs),
                                       weight=self.word_emb.weight)
        self.apply(self._init)
        nn.init.normal_(self.u, 0.0, 0.02)
        nn.init.normal_(self.v, 0.0, 0.02)

    @staticmethod
    def _init(m):
        if isinstance(m, (nn.Linear, nn.Embedding)):
            nn.init.normal_(m.weight, 0.0, 0.02)
            if getattr(m, "bias", None) is not None:
                nn.init.zeros_(m.bias)

    def hidden_states(self, data, mems):
        qlen, _ = data.shape
        mlen = mems[0].size(0) if mems is not None else 0
        klen = qlen + mlen
        x = self.word_emb(data) * math.sqrt(self.d_model)
        table = sinusoid_table(torch.arange(klen - 1, -1, -1, device=data.device),
                               self.d_model, x.dtype)
        # key j is visible to query i when j <= mlen + i
        mask = torch.full((qlen, klen), float("-inf"), device=data.device,
                          dtype=x.dtype).triu(1 + mlen)
        x, table = self.drop(x), self.drop(table)
        inputs = []
        for i in range(self.n_layer):
            inputs.append(x)
            x = self.attn[i](x, table, self.u, self.v, mask,
                             None if mems is None else mems[i])
            x = self.ff[i](x)
        return self.drop(x), self._new_mems(inputs, mems)

    def _new_mems(self, inputs, mems):
        """The last ``mem_len`` inputs of every layer, detached."""
        if not self.mem_len:
            return None
        with torch.no_grad():
            new = torch.stack(inputs)                     # [n_layer, qlen, B, d]
            if mems is not None and mems.size(1) > 0:
                new = torch.cat([mems, new], dim=1)
            return new[:, -self.mem_len:].detach()

    def forward(self, data, target, mems=None):
        hidden, new_mems = self.hidden_states(data, mems)
        tgt_len = target.size(0)
        pred = hidden[-tgt_len:]
        nll = self.crit(pred.reshape(-1, pred.size(-1)), target.reshape(-1))
        return nll.view(tgt_len, -1), new_mems


class Lamb(torch.optim.Optimizer):
    """LAMB (You et al., 2019) as the reference's client uses it
    (related/baselines/transformer/lamb.py:79-146): Adam moments without bias
    correction, the update scaled per tensor by ||w|| (clamped to 10) over
    ||update||, ratio 1 where either norm is zero.  The whole step stays on the
    device (the reference reads both norms back for every tensor)."""

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-6, weight_decay=0.0):
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay))

    @torch.no_grad()
    def step(self):
        for group in self.param_groups:
            params = [p for p in group["params"] if p.grad is not None]
            if not params:
                continue
            grads = [p.grad for p in params]
            for p in params:
                if not self.state[p]:
                    self.state[p]["m"] = torch.zeros_like(p)
                    self.state[p]["v"] = torch.zeros_like(p)
            ms = [self.state[p]["m"] for p in params]
            vs = [self.state[p]["v"] for p in params]
            b1, b2 = group["betas"]
            torch._foreach_mul_(ms, b1)
            torch._foreach_add_(ms, grads, alpha=1 - b1)
            torch._foreach_mul_(vs, b2)
            torch._foreach_addcmul_(vs, grads, grads, value=1 - b2)
            denom = torch._foreach_sqrt(vs)
            torch._foreach_add_(denom, group["eps"])
            update = torch._foreach_div(ms, denom)
            if group["weight_decay"]:
                torch._foreach_add_(update, params, alpha=group["weight_decay"])
            w_norm = torch.stack(torch._foreach_norm(params)).clamp_(0, 10)
            u_norm = torch.stack(torch._foreach_norm(update))
            ratio = torch.where((w_norm == 0) | (u_norm == 0), torch.ones_like(w_norm),
                                w_norm / (u_norm + group["eps"]))
            torch._foreach_mul_(update, list((-group["lr"] * ratio).unbind(0)))
            torch._foreach_add_(params, update)
