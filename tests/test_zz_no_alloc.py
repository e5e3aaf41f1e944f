"""The backward entry point that allocates nothing (its delta workspace is an array inside the
library) against slapo_amd_attn_bwd on the same inputs, through the raw C ABI: bitwise equal
gradients on two calls in a row, the second with a smaller input, and a clear error beyond the
array's size."""
import ctypes

import pytest
import torch

from slapo_amd import _lib
from slapo_amd.op import _kernels as K

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _both_backwards(dtype, b, s, h, d, causal, p, seed):
    lib = _lib.load()
    g = torch.Generator().manual_seed(seed)
    q, k, v, do = (torch.randn(b, s, h, d, generator=g).to(dtype).cuda() for _ in range(4))
    plan = K.dropout_plan(b * h * s * s, 4, q.device) if p > 0 else None
    o, lse, _, km = K.attn_fwd(q, k, v, None, causal, 0, d ** -0.5, p, 11, 0, plan,
                               save_mask=True)
    prm = K.make_attn_params(q, k, v, o, None, causal, 0, d ** -0.5, p, 11, 0, plan, km)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    outs = []
    for which in ("workspace", "static"):
        dq, dk, dv = torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v)
        strides = [K._bshd_strides(t) for t in (dq, dk, dv)]
        args = [ctypes.byref(prm), _ptr(q), _ptr(k), _ptr(v), None, _ptr(o), _ptr(do), _ptr(lse),
                _ptr(dq), _ptr(dk), _ptr(dv), *strides]
        if which == "workspace":
            nb = lib.slapo_amd_attn_bwd_workspace_bytes(ctypes.byref(prm))
            ws = torch.empty(nb // 4, dtype=torch.float32, device=q.device)
            rc = lib.slapo_amd_attn_bwd(*args, _ptr(ws), nb, st)
        else:
            rc = lib.slapo_amd_attn_bwd_static_scratch(*args, st)
        assert rc == 0, f"{which}: status {rc}"
        torch.cuda.synchronize()
        outs.append((dq, dk, dv))
    return outs


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_static_scratch_backward_equals_workspace_backward(dtype):
    # two calls in a row on the same device; the second is smaller, so part of the array still
    # holds the first call's delta
    for (b, s, h, d, causal, p, seed) in ((2, 384, 4, 64, True, 0.0, 1), (1, 130, 2, 64, True, 0.1, 2)):
        if dtype == torch.float32:
            p = 0.0
        (dq0, dk0, dv0), (dq1, dk1, dv1) = _both_backwards(dtype, b, s, h, d, causal, p, seed)
        assert torch.isfinite(dq0).all() and dq0.abs().max() > 0
        assert torch.equal(dq0, dq1) and torch.equal(dk0, dk1) and torch.equal(dv0, dv1)


def test_static_scratch_rejects_sizes_beyond_the_array():
    lib = _lib.load()
    prm = _lib.AttnParams()
    prm.dtype = _lib.SLAPO_F16
    prm.batch, prm.heads, prm.seqlen_q, prm.seqlen_k, prm.head_dim = 8, 32, 4097, 64, 64
    prm.scale = 0.125
    rc = lib.slapo_amd_attn_bwd_static_scratch(ctypes.byref(prm), None, None, None, None, None,
                                               None, None, None, None, None, None, None, None,
                                               None)
    assert rc == -7  # SLAPO_ERR_WORKSPACE
    assert b"workspace" in lib.slapo_amd_status_string(rc)


def _static_call(dtype=torch.float16, b=2, s=256, h=4, d=64, seed=5):
    lib = _lib.load()
    g = torch.Generator().manual_seed(seed)
    q, k, v, do = (torch.randn(b, s, h, d, generator=g).to(dtype).cuda() for _ in range(4))
    o, lse, _ = K.attn_fwd(q, k, v, None, True, 0, d ** -0.5, 0.0, 0, 0, None)
    prm = K.make_attn_params(q, k, v, o, None, True, 0, d ** -0.5, 0.0, 0, 0, None)
    dq, dk, dv = torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v)
    strides = [K._bshd_strides(t) for t in (dq, dk, dv)]
    keep = (q, k, v, do, o, lse, prm, strides)  # alive for as long as the closure is

    def call():
        rc = lib.slapo_amd_attn_bwd_static_scratch(
            ctypes.byref(prm), _ptr(q), _ptr(k), _ptr(v), None, _ptr(o), _ptr(do), _ptr(lse),
            _ptr(dq), _ptr(dk), _ptr(dv), *strides,
            ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, rc

    return call, (dq, dk, dv), keep


def test_static_scratch_call_leaves_device_memory_and_the_allocator_alone():
    """The property the entry point exists for: between two points with no other work, neither
    the device's free memory nor torch's allocator moves (no hipMalloc, no hipFree, no torch
    allocation inside the call)."""
    call, _, _keep = _static_call()
    call()  # first call on the device: resolves the array's address, sets kernel attributes
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    alloc0, reserved0 = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    n_alloc0 = torch.cuda.memory_stats()["allocation.all.allocated"]
    for _ in range(3):
        call()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0
    assert torch.cuda.memory_allocated() == alloc0 and torch.cuda.memory_reserved() == reserved0
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == n_alloc0


def test_static_scratch_backward_under_graph_capture():
    """After one call outside a capture (which resolves the array's address), the entry point can
    be recorded into a HIP graph and replayed; every replay equals the eager result."""
    call, grads, _keep = _static_call(torch.bfloat16, 1, 320, 2, 128, seed=6)
    call()
    torch.cuda.synchronize()
    eager = [t.clone() for t in grads]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()  # launches on the capturing stream
    for round_ in range(3):
        for t in grads:
            t.zero_()  # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(grads, eager):
            assert torch.equal(got, want), f"replay {round_}"
