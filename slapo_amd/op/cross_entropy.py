"""Vocab-parallel cross entropy with the reference's names (slapo/op/cross_entropy.py:17-160) on
the HIP kernels of csrc/cross_entropy.hip.

One GPU holds the whole vocabulary here (tensor-parallel world size 1).  The kernels already
produce what a larger group would combine -- per row the shard's maximum, its sum of exponentials
relative to that maximum, the target's logit and the sum of logits -- so a group of p ranks needs
three all-reduces over [tokens] floats (max; sum after rescaling by exp(m_r - M); sum), where the
reference all-reduces the same three quantities (:25, :56, :62) around five passes over the
logits.  That combine is not built: a group of more than one rank raises NotImplementedError.
"""
from __future__ import annotations

import torch
from torch import nn

from . import _kernels as K


def vocab_range_from_per_partition_vocab_size(per_partition_vocab_size, rank, _):
    index_f = rank * per_partition_vocab_size
    index_l = index_f + per_partition_vocab_size
    return index_f, index_l


def _group_rank_and_size(group):
    dist = torch.distributed
    if not (dist.is_available() and dist.is_initialized()):
        return 0, 1
    return dist.get_rank(group=group), dist.get_world_size(group=group)


class _VocabParallelCrossEntropy(torch.autograd.Function):
    # pylint: disable=abstract-method, arguments-differ
    @staticmethod
    def forward(ctx, vocab_parallel_logits, target, label_smoothing=0.0, group=None):
        rank, world = _group_rank_and_size(group)
        if world != 1:
            raise NotImplementedError(
                "vocab-parallel cross entropy over more than one rank: the per-shard statistics "
                "are computed, their all-reduce is not part of this build")
        if not 0.0 <= label_smoothing < 1.0:
            raise ValueError("label_smoothing must be in [0, 1)")
        vocab = vocab_parallel_logits.shape[-1]
        start, _ = vocab_range_from_per_partition_vocab_size(vocab, rank, world)
        m, s, pred, sumx, logits, tgt = K.vocab_ce_fwd(vocab_parallel_logits, target, start)
        # (with p ranks: M = all-reduce-max(m); s *= exp(m - M); all-reduce-sum(s), (pred))
        log_s = torch.log(s)
        loss = log_s + (m - pred)  # m - pred first: exact where the logits sit far from zero
        if label_smoothing > 0:
            if vocab < 2:
                raise ValueError("label smoothing needs at least two classes")
            smoothing = label_smoothing * vocab / (vocab - 1)
            mean_log_probs = (sumx / vocab - m) - log_s
            loss = (1.0 - smoothing) * loss - smoothing * mean_log_probs
        ctx.save_for_backward(logits, tgt, m, 1.0 / s)
        ctx.cfg = (start, float(label_smoothing))
        return loss.view(target.shape)

    @staticmethod
    def backward(ctx, grad_output):
        logits, tgt, m, inv_s = ctx.saved_tensors
        start, label_smoothing = ctx.cfg
        grad = K.vocab_ce_bwd(logits, tgt, m, inv_s, grad_output, start, label_smoothing)
        return grad, None, None, None


def vocab_parallel_cross_entropy(vocab_parallel_logits, target, label_smoothing=0.0, group=None):
    """Per-token loss log(sum exp(logits)) - logits[target], optionally label-smoothed; logits
    [..., vocab/p], target [...] (slapo/op/cross_entropy.py:128-150).  The loss is fp32."""
    return _VocabParallelCrossEntropy.apply(vocab_parallel_logits, target, label_smoothing, group)


class ParallelCrossEntropy(nn.Module):
    def __init__(self, group=None):
        super().__init__()
        self.group = group

    def forward(self, outputs, labels):
        return vocab_parallel_cross_entropy(outputs, labels, group=self.group)
