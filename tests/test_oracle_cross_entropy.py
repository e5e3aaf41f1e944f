"""Pins for oracle/cross_entropy.py (CPU only): the library's cross entropy (with its own label
smoothing, which is the reference's formula at alpha K / (K - 1)), autograd, and the identity
between the whole-vocabulary loss and the loss combined from shard statistics."""
import pytest
import torch
import torch.nn.functional as F

from oracle import cross_entropy as OC


@pytest.mark.parametrize("alpha", [0.0, 0.1, 0.45])
def test_loss_and_gradient_match_the_library(alpha):
    g = torch.Generator().manual_seed(0)
    logits = (torch.randn(5, 7, 23, generator=g, dtype=torch.float64) * 4).requires_grad_(True)
    target = torch.randint(0, 23, (5, 7), generator=g)
    go = torch.randn(5, 7, generator=g, dtype=torch.float64)
    # F.cross_entropy(label_smoothing=a) = (1 - a) nll - a mean(log p): the reference's loss at
    # a = alpha K / (K - 1)
    a = alpha * 23 / 22
    ref = F.cross_entropy(logits.reshape(-1, 23), target.reshape(-1), reduction="none",
                          label_smoothing=a).reshape(5, 7)
    ref.backward(go)
    loss, softmax = OC.forward(logits.detach(), target, alpha)
    torch.testing.assert_close(loss, ref.detach(), atol=1e-12, rtol=0)
    torch.testing.assert_close(softmax, F.softmax(logits.detach(), -1), atol=1e-14, rtol=0)
    torch.testing.assert_close(OC.backward(softmax, target, go, alpha), logits.grad, atol=1e-12,
                               rtol=0)


def test_shard_statistics_combine_to_the_same_loss():
    g = torch.Generator().manual_seed(1)
    logits = torch.randn(9, 40, generator=g, dtype=torch.float64) * 6
    logits[3] = -1e4  # a row far below zero: the shift by the maximum matters
    logits[3, 17] = -9990.0
    target = torch.randint(0, 40, (9,), generator=g)
    whole = OC.forward(logits, target)[0]
    for cuts in ([0, 40], [0, 13, 40], [0, 8, 16, 24, 40]):
        stats = [OC.shard_stats(logits[:, a:b], target, a) for a, b in zip(cuts, cuts[1:])]
        torch.testing.assert_close(OC.combine(stats), whole, atol=1e-11, rtol=0)
        # exactly one shard reports the target's logit
        hits = sum((st[2] != 0).long() for st in stats)
        assert int(hits.max()) <= 1
    m, s, pred, sx = OC.shard_stats(logits, target, 0)
    torch.testing.assert_close(sx, logits.sum(-1))
    torch.testing.assert_close(pred, logits[torch.arange(9), target])
