"""Vocab-parallel cross entropy on the GPU: HIP kernels (through the C ABI) against the CPU oracle
on the same seeded inputs.  Bars: fp32 logits max-abs 1e-5 on the loss and the gradient; fp16 /
bf16 logits: the loss (fp32 math on the rounded inputs) 1e-4 relative, the gradient 2e-2
relative."""
import ctypes

import pytest
import torch

from oracle import cross_entropy as OC
from slapo_amd import _lib, op
from slapo_amd.op import _kernels as K
from tests.conftest import assert_parity, max_abs_err

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]


def _case(shape, vocab, dtype, seed=2013, scale=3.0):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(*shape, vocab, generator=g) * scale).to(dtype)
    target = torch.randint(0, vocab, shape, generator=g)
    go = torch.randn(shape, generator=g)
    return logits, target, go


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape,vocab", [((4, 6), 50257), ((33,), 1000), ((2, 3), 8), ((5,), 1),
                                         ((3, 2), 4099), ((2,), 70000), ((3,), 12289),
                                         ((2, 2), 20001)])
@pytest.mark.parametrize("alpha", [0.0, 0.1])
def test_loss_and_gradient(dtype, shape, vocab, alpha):
    """Unpadded vocabularies (rows start at every element offset: head / body / tail paths),
    tiny and single-class rows, label smoothing; row lengths on both sides of the thresholds at
    which the kernels take larger blocks (8192, 16384, 32768)."""
    if alpha > 0 and vocab < 2:
        pytest.skip("label smoothing needs two classes")
    logits, target, go = _case(shape, vocab, dtype)
    ld = logits.cuda().requires_grad_(True)
    loss = op.vocab_parallel_cross_entropy(ld, target.cuda(), alpha)
    assert loss.dtype == torch.float32 and loss.shape == target.shape
    loss.backward(go.cuda())
    ref, softmax = OC.forward(logits, target, alpha)
    gref = OC.backward(softmax, target, go.double(), alpha)
    if dtype == torch.float32:
        assert max_abs_err(loss, ref) <= 1e-5 * max(1.0, float(ref.abs().max()))
        assert max_abs_err(ld.grad, gref) <= 1e-5
    else:
        assert max_abs_err(loss, ref) <= 1e-4 * max(1.0, float(ref.abs().max()))
        assert_parity(ld.grad, gref, dtype, "grad_logits")


def test_extreme_rows_and_module():
    """Rows far from zero, a row with -inf entries, one dominant class; the module form."""
    logits = torch.randn(6, 300) * 5
    logits[0] += 3e4
    logits[1] -= 3e4
    logits[2, 10:] = float("-inf")
    logits[3, 7] = 80.0
    target = torch.tensor([5, 299, 3, 7, 0, 150])
    ref, softmax = OC.forward(logits, target)
    ld = logits.cuda().requires_grad_(True)
    crit = op.ParallelCrossEntropy()
    loss = crit(ld, target.cuda())
    loss.sum().backward()
    assert max_abs_err(loss, ref) <= 1e-5 * float(ref.abs().max())
    assert max_abs_err(ld.grad, OC.backward(softmax, target, torch.ones(6, dtype=torch.float64))) <= 1e-5
    assert torch.equal(ld.grad[2, 10:].cpu(), torch.zeros(290))  # exp(-inf) = 0, no NaN
    with pytest.raises(ValueError):
        op.vocab_parallel_cross_entropy(ld, target.cuda(), 1.5)


def test_shard_statistics_through_the_c_abi():
    """The forward entry point on column shards of one matrix: the statistics of each shard match
    the oracle's and combine to the whole-vocabulary loss; the backward entry point with the
    combined statistics gives each shard its slice of the whole gradient."""
    lib = _lib.load()
    g = torch.Generator().manual_seed(7)
    rows, vocab = 37, 5003
    logits = torch.randn(rows, vocab, generator=g) * 4
    target = torch.randint(0, vocab, (rows,), generator=g)
    go = torch.randn(rows, generator=g)
    whole, softmax = OC.forward(logits, target)
    gwhole = OC.backward(softmax, target, go.double())
    cuts = [0, 1250, 2501, 5003]
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    tgt = target.cuda()
    stats, shards = [], []
    for a, b in zip(cuts, cuts[1:]):
        shard = logits[:, a:b].contiguous().cuda()
        out = torch.empty(4, rows, device="cuda")
        rc = lib.slapo_amd_vocab_ce_fwd(P(shard), P(tgt), P(out[0]), P(out[1]), P(out[2]),
                                        P(out[3]), rows, b - a, a, _lib.SLAPO_F32, st)
        assert rc == 0
        ref = OC.shard_stats(logits[:, a:b], target, a)
        for got, want in zip(out.cpu(), ref):
            assert max_abs_err(got, want) <= 1e-5 * max(1.0, float(want.abs().max()))
        stats.append(tuple(t.double().cpu() for t in out))
        shards.append(shard)
    assert max_abs_err(OC.combine(stats), whole) <= 1e-5 * float(whole.abs().max())
    big = torch.stack([s[0] for s in stats]).max(0)[0]
    total = sum(s[1] * torch.exp(s[0] - big) for s in stats)
    big_d, inv_d, go_d = big.float().cuda(), (1.0 / total).float().cuda(), go.cuda()
    for (a, b), shard in zip(zip(cuts, cuts[1:]), shards):
        grad = torch.empty_like(shard)
        rc = lib.slapo_amd_vocab_ce_bwd(P(shard), P(tgt), P(big_d), P(inv_d), P(go_d), P(grad),
                                        rows, b - a, a, 0.0, _lib.SLAPO_F32, st)
        assert rc == 0
        assert max_abs_err(grad, gwhole[:, a:b]) <= 1e-5
    # argument checks happen on the host
    assert lib.slapo_amd_vocab_ce_fwd(None, P(tgt), P(out[0]), P(out[1]), P(out[2]), P(out[3]),
                                      rows, 10, 0, _lib.SLAPO_F32, st) == -4
    assert lib.slapo_amd_vocab_ce_bwd(P(shard), P(tgt), P(big_d), P(inv_d), P(go_d), P(grad), rows,
                                      10, 0, 1.0, _lib.SLAPO_F32, st) == -4


@pytest.mark.parametrize("off_x,off_g", [(0, 0), (3, 3), (5, 1), (63, 63), (64, 8)])
def test_rows_that_start_anywhere_relative_to_a_cache_line(off_x, off_g):
    """The kernels align each row's vector body to a cache line and take the elements before
    it one per thread; logits and gradient buffers whose bases differ modulo 16 bytes fall back
    to element-wise accesses.  Buffers offset by a few elements, odd row length."""
    lib = _lib.load()
    g = torch.Generator().manual_seed(11)
    rows, vocab = 19, 1237
    logits = (torch.randn(rows, vocab, generator=g) * 3).to(torch.float16)
    target = torch.randint(0, vocab, (rows,), generator=g)
    go = torch.randn(rows, generator=g)
    buf_x = torch.zeros(rows * vocab + 128, dtype=torch.float16, device="cuda")
    buf_g = torch.full((rows * vocab + 128,), 7.0, dtype=torch.float16, device="cuda")
    x = buf_x[off_x:off_x + rows * vocab].view(rows, vocab)
    x.copy_(logits)
    grad = buf_g[off_g:off_g + rows * vocab].view(rows, vocab)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    out = torch.empty(4, rows, device="cuda")
    tgt = target.cuda()
    assert lib.slapo_amd_vocab_ce_fwd(P(x), P(tgt), P(out[0]), P(out[1]), P(out[2]), P(out[3]),
                                      rows, vocab, 0, _lib.SLAPO_F16, st) == 0
    ref = OC.shard_stats(logits.float(), target, 0)
    for got, want in zip(out.cpu(), ref):
        assert max_abs_err(got, want) <= 1e-4 * max(1.0, float(want.abs().max()))
    inv = (1.0 / out[1]).contiguous()
    assert lib.slapo_amd_vocab_ce_bwd(P(x), P(tgt), P(out[0]), P(inv), P(go.cuda()), P(grad), rows,
                                      vocab, 0, 0.0, _lib.SLAPO_F16, st) == 0
    _, softmax = OC.forward(logits, target)
    assert_parity(grad, OC.backward(softmax, target, go.double()), torch.float16, "grad")
    # nothing outside the gradient's own elements was written
    assert bool((buf_g[:off_g] == 7.0).all()) and bool((buf_g[off_g + rows * vocab:] == 7.0).all())
