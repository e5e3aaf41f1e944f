"""CPU restatement of the reference's vocab-parallel cross entropy for a group of one rank (test
infrastructure; pinned by tests/test_oracle_cross_entropy.py).  Follows
slapo/op/cross_entropy.py:21-124 step by step: maximum, shifted logits, predicted logit of the
target, exp / sum, loss = log(sum) - predicted, softmax kept for the backward, label smoothing
with smoothing = alpha K / (K - 1) over the shard's K classes.  `shard_stats` / `combine` restate
the same loss from per-shard statistics, the form in which a tensor-parallel group exchanges it.
"""
from __future__ import annotations

import torch


def forward(logits, target, label_smoothing=0.0, compute_dtype=torch.float64):
    """(loss, softmax): slapo/op/cross_entropy.py:24-92 with the all-reduces of one rank."""
    x = logits.to(compute_dtype)
    vocab = x.shape[-1]
    x = x - x.max(dim=-1)[0].unsqueeze(-1)                      # :24-27
    x2 = x.reshape(-1, vocab)
    t = target.reshape(-1)
    predicted = x2[torch.arange(x2.shape[0]), t].reshape(target.shape)  # :45-54
    exp_logits = torch.exp(x)                                   # :58-61
    sum_exp = exp_logits.sum(dim=-1)
    loss = torch.log(sum_exp) - predicted                       # :65
    softmax = exp_logits / sum_exp.unsqueeze(-1)                # :68
    if label_smoothing > 0:                                     # :71-86
        smoothing = label_smoothing * vocab / (vocab - 1)
        mean_log_probs = torch.log(softmax).mean(dim=-1)
        loss = (1.0 - smoothing) * loss - smoothing * mean_log_probs
    return loss, softmax


def backward(softmax, target, grad_output, label_smoothing=0.0):
    """grad of the logits: slapo/op/cross_entropy.py:97-124."""
    vocab = softmax.shape[-1]
    grad = softmax.clone().reshape(-1, vocab)
    rows = torch.arange(grad.shape[0])
    t = target.reshape(-1)
    if label_smoothing > 0:
        smoothing = label_smoothing * vocab / (vocab - 1)
        grad[rows, t] -= 1.0 - smoothing
        grad -= smoothing / vocab
    else:
        grad[rows, t] -= 1.0
    return (grad * grad_output.reshape(-1, 1).to(grad.dtype)).reshape(softmax.shape)


def shard_stats(logits, target, vocab_start, compute_dtype=torch.float64):
    """(row_max, sum_exp relative to it, predicted, sum_logits) of one shard."""
    x = logits.to(compute_dtype)
    n = x.shape[-1]
    m = x.max(dim=-1)[0]
    s = torch.exp(x - m.unsqueeze(-1)).sum(dim=-1)
    t = target - vocab_start
    inside = (t >= 0) & (t < n)
    pred = torch.where(inside, x.gather(-1, t.clamp(0, n - 1).unsqueeze(-1)).squeeze(-1),
                       torch.zeros((), dtype=compute_dtype))
    return m, s, pred, x.sum(dim=-1)


def combine(stats):
    """Loss from the statistics of every shard (list of shard_stats tuples)."""
    big = torch.stack([st[0] for st in stats]).max(dim=0)[0]
    total = sum(st[1] * torch.exp(st[0] - big) for st in stats)
    pred = sum(st[2] for st in stats)
    return torch.log(total) + big - pred
