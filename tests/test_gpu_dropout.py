"""Dropout RNG parity on the GPU: masks are compared bit for bit with the masks
torch.nn.functional.dropout draws (the reference calls exactly that function:
slapo/op/fused_bias.py:74, slapo/op/attention.py:180) under the same generator seed and offset,
and the generator must move by the same amount."""
import ctypes

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import philox as OP
from slapo_amd import _lib, op
from slapo_amd.op import _kernels as K
from slapo_amd.random import CudaRNGStatesTracker, draw_philox

pytestmark = pytest.mark.gpu


def _gen():
    torch.cuda.init()
    return torch.cuda.default_generators[torch.cuda.current_device()]


def _torch_mask(shape, dtype, p, seed, offset):
    torch.cuda.manual_seed(seed)
    _gen().set_offset(offset)
    y = F.dropout(torch.ones(shape, device="cuda", dtype=dtype), p)
    return (y != 0), _gen().get_offset()


CASES = [
    ((1000,), torch.float32, 0.1, 2013, 0),
    ((4098,), torch.float32, 0.25, 7, 8),
    ((4097,), torch.bfloat16, 0.5, 11, 4),
    ((8192, 1024), torch.bfloat16, 0.1, 2013, 0),        # FusedMLP epilogue shape
    ((4, 1024, 2048), torch.float16, 0.2, 2013, 16),     # reference test_fused_mlp shape
    ((8 * 16, 1024, 1024), torch.float32, 0.1, 2013, 0),  # attention probabilities, GPT-2-medium
    ((3, 77, 130), torch.float32, 0.3, (1 << 40) + 3, 1 << 33),
]


@pytest.mark.parametrize("shape,dtype,p,seed,offset", CASES)
def test_device_mask_is_torch_dropout_mask(shape, dtype, p, seed, offset):
    ref, after = _torch_mask(shape, dtype, p, seed, offset)
    numel = ref.numel()
    esz = torch.empty((), dtype=dtype).element_size()
    plan = K.dropout_plan(numel, esz, "cuda")
    assert after - offset == plan.offset_increment
    mine = K.dropout_mask(numel, esz, p, seed, offset, "cuda")
    assert torch.equal(mine, ref.flatten())


def test_oracle_and_host_mirror_agree_with_torch_on_this_device():
    props = torch.cuda.get_device_properties(0)
    shape, dtype, p, seed, offset = (5, 1000), torch.float16, 0.1, 42, 12
    ref, _ = _torch_mask(shape, dtype, p, seed, offset)
    plan = OP.aten_launch_plan(5000, 2, props.multi_processor_count,
                               props.max_threads_per_multi_processor)
    assert np.array_equal(OP.aten_dropout_mask(plan, p, seed, offset), ref.flatten().cpu().numpy())
    cplan = K.dropout_plan(5000, 2, "cuda")
    host = np.zeros(5000, dtype=np.uint8)
    rc = _lib.load().slapo_amd_dropout_mask_host(host.ctypes.data_as(ctypes.c_void_p),
                                                 ctypes.byref(cplan), p, seed, offset)
    assert rc == 0 and np.array_equal(host.astype(bool), ref.flatten().cpu().numpy())


def test_draw_advances_generator_like_torch():
    torch.cuda.manual_seed(77)
    seed, off = draw_philox(16)
    assert (seed, off) == (77, 0) and _gen().get_offset() == 16
    with pytest.raises(ValueError):
        draw_philox(3)


def test_bias_dropout_consumes_the_stream_exactly_like_torch():
    """Same seed => same mask AND the following random op sees the same state."""
    x = torch.randn(64, 512, device="cuda", dtype=torch.bfloat16)
    b = torch.randn(512, device="cuda", dtype=torch.bfloat16)
    torch.cuda.manual_seed(123)
    ref = F.dropout(x + b, 0.2)
    ref_next = torch.rand(4, device="cuda")
    torch.cuda.manual_seed(123)
    out = op.bias_dropout(x, b, 0.2, True)
    next_ = torch.rand(4, device="cuda")
    assert torch.equal(out == 0, ref == 0)
    assert torch.equal(next_, ref_next)
    # eval mode and p == 0 draw nothing
    torch.cuda.manual_seed(123)
    op.bias_dropout(x, b, 0.2, False)
    op.bias_dropout(x, b, 0.0, True)
    assert _gen().get_offset() == 0


def test_fork_changes_the_mask_and_restores_the_stream():
    """Restates tests/test_fork_rng.py:56-67 and tests/test_random.py:49-63 for the HIP op."""
    x = torch.ones(32, 256, device="cuda", dtype=torch.float16)
    b = torch.zeros(256, device="cuda", dtype=torch.float16)
    tracker = CudaRNGStatesTracker()
    torch.cuda.manual_seed(2013)
    tracker.add("model-parallel-rng", 2013 + 2718)
    plain = op.bias_dropout(x, b, 0.5, True)
    torch.cuda.manual_seed(2013)
    with tracker.fork():
        assert torch.cuda.initial_seed() == 2013 + 2718
        forked = op.bias_dropout(x, b, 0.5, True)
    assert torch.cuda.initial_seed() == 2013 and _gen().get_offset() == 0
    assert not torch.equal(plain == 0, forked == 0)
    after_fork = op.bias_dropout(x, b, 0.5, True)
    assert torch.equal(after_fork == 0, plain == 0)
    with tracker.fork():
        forked2 = op.bias_dropout(x, b, 0.5, True)
    assert not torch.equal(forked2 == 0, forked == 0)  # the forked stream moved on


def test_recompute_under_restored_state_reproduces_mask():
    """Activation checkpointing restores the generator state and reruns forward
    (slapo/checkpoint.py:79-92, tests/test_checkpoint.py:190-198)."""
    q, k, v = (torch.randn(2, 128, 2, 64, device="cuda", dtype=torch.float16) for _ in range(3))
    torch.cuda.manual_seed(5)
    state = torch.cuda.get_rng_state()
    a = op.hip_attention(q, k, v, None, causal=True, p=0.3)
    moved = _gen().get_offset()
    assert moved > 0
    torch.cuda.set_rng_state(state)
    b = op.hip_attention(q, k, v, None, causal=True, p=0.3)
    assert torch.equal(a, b) and _gen().get_offset() == moved
    c = op.hip_attention(q, k, v, None, causal=True, p=0.3)
    assert not torch.equal(a, c)


def test_checkpointed_block_of_hip_ops_matches_the_plain_run():
    """Activation checkpointing with tracked streams around the HIP ops (reference
    slapo/checkpoint.py:15-124, tests/test_checkpoint.py:138-198): attention dropout under the
    forked stream, the fused epilogues under the outer one.  Output and every gradient of the
    checkpointed run equal the plain run bit for bit, and the recompute leaves both streams
    where the forward left them."""
    import slapo_amd
    from slapo_amd.checkpoint import checkpoint
    from slapo_amd.random import get_cuda_rng_tracker

    B, S, H, D = 2, 256, 4, 64
    hid = H * D
    dt = torch.float16
    g = torch.Generator(device="cuda").manual_seed(1)
    qkv_w = (torch.randn(hid, 3 * hid, device="cuda", dtype=dt, generator=g) * 0.05).requires_grad_()
    out_b = torch.randn(hid, device="cuda", dtype=dt, generator=g).requires_grad_()
    ln = op.HipBiasDropoutResidualLayerNorm(hid, p=0.2, device="cuda", dtype=dt)
    up_b = torch.randn(hid, device="cuda", dtype=dt, generator=g).requires_grad_()
    x0 = torch.randn(B, S, hid, device="cuda", dtype=dt, generator=g)
    params = [qkv_w, out_b, up_b, ln.weight, ln.bias]

    def block(x, p_attn):
        qkv = (x @ qkv_w).view(B, S, H, 3 * D)
        q, k, v = qkv.split(D, dim=-1)             # strided views, read in place
        with get_cuda_rng_tracker().fork():
            a = op.hip_attention(q, k, v, None, causal=True, p=p_attn)
        h = ln(a.reshape(B, S, hid), out_b, x)
        h = op.bias_gelu(h, up_b)
        return op.bias_dropout_residual(h, out_b, x, 0.1, True)

    def run(use_checkpoint):
        slapo_amd.set_random_seed(123, None, None, 0)
        x = x0.clone().requires_grad_()
        out = checkpoint(block, x, 0.3) if use_checkpoint else block(x, 0.3)
        offset = _gen().get_offset()
        forked = get_cuda_rng_tracker().get_states()["model-parallel-rng"].clone()
        assert offset > 0
        out.float().square().mean().backward()
        assert _gen().get_offset() == offset
        assert torch.equal(get_cuda_rng_tracker().get_states()["model-parallel-rng"], forked)
        grads = [t.grad.clone() for t in [x] + params]
        for t in params:
            t.grad = None
        return [out.detach()] + grads

    ref = run(False)
    got = run(True)
    for a, b in zip(ref, got):
        assert torch.equal(a, b)
    assert ref[0].isfinite().all() and (ref[1] != 0).any()
    get_cuda_rng_tracker().reset()
