"""The C ABI under HIP graph capture: the entry points neither allocate nor synchronise, so a
forward + backward of the attention op and the epilogues can be recorded once and replayed.  Every
replay is checked against the eager result, with eager work and synchronisations in between."""
import pytest
import torch

from slapo_amd.op import _kernels as K

pytestmark = pytest.mark.gpu


def _attention(q, k, v, do, causal, p, plan):
    o, lse, _, bits = K.attn_fwd(q, k, v, None, causal, 0, q.shape[-1] ** -0.5, p, 11, 0, plan,
                                 save_mask=True)
    dq, dk, dv = K.attn_bwd(do, q, k, v, None, o, lse, causal, 0, q.shape[-1] ** -0.5, p, 11, 0,
                            plan, bits)
    return o, dq, dk, dv


@pytest.mark.parametrize("shape,p", [((2, 384, 4, 64), 0.0), ((1, 320, 2, 128), 0.1)])
def test_attention_forward_backward_replays(shape, p):
    g = torch.Generator().manual_seed(3)
    mk = lambda: torch.randn(*shape, generator=g).to(torch.bfloat16).cuda()
    q, k, v, do = mk(), mk(), mk(), mk()
    b, s, h, _ = shape
    plan = K.dropout_plan(b * h * s * s, 4, q.device) if p > 0 else None
    eager = _attention(q, k, v, do, True, p, plan)  # also the warm-up: first launches set the
    torch.cuda.synchronize()                        # dynamic shared memory limit of a kernel
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = _attention(q, k, v, do, True, p, plan)
    for round_ in range(3):
        for t in captured:
            t.zero_()  # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(captured, eager):
            assert torch.equal(got, want), f"replay {round_}"
    # new inputs in the same buffers are picked up by the next replay
    q.copy_(mk())
    want = _attention(q, k, v, do, True, p, plan)
    graph.replay()
    torch.cuda.synchronize()
    for got, ref in zip(captured, want):
        assert torch.equal(got, ref)


def test_epilogues_replay():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(256, 1024, generator=g).to(torch.bfloat16).cuda()
    r = torch.randn(256, 1024, generator=g).to(torch.bfloat16).cuda()
    b = torch.randn(1024, generator=g).to(torch.bfloat16).cuda()
    w = torch.ones(1024, dtype=torch.bfloat16, device="cuda")
    plan = K.dropout_plan(x.numel(), 2, x.device)

    def run():
        y = K.bias_gelu_fwd(x, b)
        dx, db = K.bias_gelu_bwd(r, x, b)
        out, z, mean, rstd = K.bias_dropout_residual_ln_fwd(x, b, r, w, b, 1e-5, 0.1, 5, 0, plan)
        grads = K.bias_dropout_residual_ln_bwd(r, z, mean, rstd, w, 0.1, 5, 0, plan)
        return (y, dx, db, out) + tuple(grads)

    eager = run()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = run()
    for _ in range(3):
        for t in captured:
            t.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(captured, eager):
            assert torch.equal(got, want)
