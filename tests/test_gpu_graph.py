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


# ---- dropout whose (seed, offset) pair lives in device memory ---------------------------------
def _state(seed, offset):
    return torch.tensor([seed, offset], dtype=torch.int64, device="cuda")


@pytest.mark.parametrize("shape,window,save_mask", [((2, 200, 2, 64), 0, True),
                                                    ((1, 320, 2, 128), 0, False),
                                                    ((1, 300, 2, 128), 100, True),
                                                    ((1, 131, 2, 80), 0, False)])
def test_attention_reads_seed_and_offset_from_device_memory(shape, window, save_mask):
    """plan.rng_state pointing at {seed, offset} gives bitwise what the same pair gives by value,
    in the forward (in-kernel draws, and the kernel that draws the keep bits of a window ahead of
    it) and in a backward that regenerates the mask or reads the stored bits; the by-value fields
    are ignored then."""
    g = torch.Generator().manual_seed(5)
    mk = lambda: torch.randn(*shape, generator=g).to(torch.bfloat16).cuda()
    q, k, v, do = mk(), mk(), mk(), mk()
    b, s, h, d = shape
    plan = K.dropout_plan(b * h * s * s, 4, q.device)
    seed, offset, p, scale = 1234567890123, 40, 0.2, d ** -0.5

    def run(seed_arg, offset_arg, state):
        o, lse, _, bits = K.attn_fwd(q, k, v, None, True, window, scale, p, seed_arg, offset_arg,
                                     plan, save_mask=save_mask, rng_state=state)
        grads = K.attn_bwd(do, q, k, v, None, o, lse, True, window, scale, p, seed_arg,
                           offset_arg, plan, bits, rng_state=state)
        return (o,) + tuple(grads)

    want = run(seed, offset, None)
    got = run(999, 4, _state(seed, offset))
    for a, b_ in zip(got, want):
        assert torch.equal(a, b_)
    other = run(seed, offset + 4, None)
    assert not torch.equal(other[0], want[0])


def test_epilogues_read_seed_and_offset_from_device_memory():
    g = torch.Generator().manual_seed(6)
    x = torch.randn(300, 1024, generator=g).to(torch.bfloat16).cuda()
    r = torch.randn(300, 1024, generator=g).to(torch.bfloat16).cuda()
    b = torch.randn(1024, generator=g).to(torch.bfloat16).cuda()
    w = torch.randn(1024, generator=g).to(torch.bfloat16).cuda()
    plan = K.dropout_plan(x.numel(), 2, x.device)
    seed, offset, p = 77, 1 << 33, 0.3

    def run(seed_arg, offset_arg, state):
        out = K.bias_dropout_residual_fwd(x, b, r, p, seed_arg, offset_arg, plan, rng_state=state)
        dx, db = K.bias_dropout_residual_bwd(r, b, p, seed_arg, offset_arg, plan, rng_state=state)
        y, z, mean, rstd = K.bias_dropout_residual_ln_fwd(x, b, r, w, b, 1e-5, p, seed_arg,
                                                          offset_arg, plan, rng_state=state)
        grads = K.bias_dropout_residual_ln_bwd(r, z, mean, rstd, w, p, seed_arg, offset_arg,
                                               plan, rng_state=state)
        mask = K.dropout_mask(x.numel(), 2, p, seed_arg, offset_arg, x.device, rng_state=state)
        return (out, dx, db, y, z, mask) + tuple(grads)

    want = run(seed, offset, None)
    got = run(1, 0, _state(seed, offset))
    for a, b_ in zip(got, want):
        assert torch.equal(a, b_)
    with pytest.raises(ValueError):
        K.bias_dropout_residual_fwd(x, b, r, p, 0, 0, plan, rng_state=torch.zeros(2, device="cuda"))


def test_ops_with_dropout_capture_and_draw_a_fresh_mask_per_replay(monkeypatch):
    """The attention op and the LayerNorm epilogue with p > 0, forward and backward, recorded
    into one graph.  Under capture their (seed, offset) pair is a device tensor written by a
    captured torch random kernel: every replay must equal an eager run of the C ABI with the pair
    that replay found there (read back after it), forward and backward; successive replays draw
    different masks; re-seeding the generator repeats the sequence."""
    from slapo_amd import op
    from slapo_amd.op import attention as A
    from slapo_amd.op import fused_bias as FB
    from slapo_amd import random as R

    states = []

    def recording(increment, device=None):
        seed, offset, state = R.draw_philox_state(increment, device)
        states.append(state)
        return seed, offset, state

    monkeypatch.setattr(A, "draw_philox_state", recording)
    monkeypatch.setattr(FB, "draw_philox_state", recording)
    g = torch.Generator().manual_seed(8)
    shape, p = (1, 256, 4, 64), 0.25
    mk = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).cuda()
    q, k, v, do = (mk(*shape).requires_grad_(True) for _ in range(4))
    x, res, gy = mk(256, 256).requires_grad_(True), mk(256, 256), mk(256, 256)
    bias, w, lb = mk(256).requires_grad_(True), mk(256).requires_grad_(True), mk(256)

    def step():
        out = op.hip_attention(q, k, v, None, causal=True, p=p)
        y = op.bias_dropout_residual_layer_norm(x, bias, res, w, lb, p, 1e-5, True)
        grads = torch.autograd.grad((out, y), (q, k, v, x, bias, w), (do.detach(), gy))
        return (out, y) + tuple(grads)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()  # warm-up: plans, dynamic shared memory limits, autograd buffers
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    assert all(s is None for s in states)  # eager calls take the pair by value
    states.clear()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    assert len(states) == 2 and all(s is not None and s.numel() == 2 for s in states)

    b_, s_, h_, d_ = shape
    plan_a = K.dropout_plan(b_ * h_ * s_ * s_, 4, q.device)
    plan_e = K.dropout_plan(x.numel(), 2, x.device)

    def eager_with(pair_a, pair_e):
        qd, kd, vd = q.detach(), k.detach(), v.detach()
        o, lse, _, bits = K.attn_fwd(qd, kd, vd, None, True, 0, d_ ** -0.5, p, pair_a[0],
                                     pair_a[1], plan_a, save_mask=True)
        dq, dk, dv = K.attn_bwd(do.detach(), qd, kd, vd, None, o, lse, True, 0, d_ ** -0.5, p,
                                pair_a[0], pair_a[1], plan_a, bits)
        y, z, mean, rstd = K.bias_dropout_residual_ln_fwd(
            x.detach(), bias.detach(), res, w.detach(), lb, 1e-5, p, pair_e[0], pair_e[1], plan_e)
        dx, _, dw, _, db = K.bias_dropout_residual_ln_bwd(gy, z, mean, rstd, w.detach(), p,
                                                          pair_e[0], pair_e[1], plan_e)
        return (o, y, dq, dk, dv, dx, db, dw)

    def replay():
        for t in captured:
            t.zero_()  # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        pairs = [tuple(int(e) for e in s.tolist()) for s in states]
        return [t.clone() for t in captured], pairs

    torch.cuda.manual_seed(31)
    seen = []
    for round_ in range(3):
        got, pairs = replay()
        want = eager_with(*pairs)
        for a, b2 in zip(got, want):
            assert torch.equal(a, b2), f"replay {round_}"
        seen.append((got, pairs))
    assert seen[0][1] != seen[1][1] != seen[2][1]
    assert not torch.equal(seen[0][0][0], seen[1][0][0])  # another mask, another output
    torch.cuda.manual_seed(31)
    for round_ in range(3):
        got, pairs = replay()
        assert pairs == seen[round_][1]
        for a, b2 in zip(got, seen[round_][0]):
            assert torch.equal(a, b2)
