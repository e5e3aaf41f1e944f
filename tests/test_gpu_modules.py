"""Module-level parity on the GPU: FlashAttention / FlashAttentionOp as schedules install them,
against an oracle composite built from the same weights (restates tests/test_op.py::test_attention,
whose bar is atol = rtol = 5e-2 in fp16)."""
import pytest
import torch

from oracle import attention as OA
from slapo_amd import op
from tests.conftest import assert_parity

pytestmark = pytest.mark.gpu


def _oracle_block(m, x, mask):
    """QKV GEMM with the head-interleaved [H, 3, D] packing, oracle attention, out_proj."""
    w = {n: p.detach().cpu().double() for n, p in m.named_parameters()}
    b, s, _ = x.shape
    h, d = m.num_attention_heads, m.attention_head_size
    if m.fused_qkv:
        packed = (x @ w["qkv.weight"].t() + w["qkv.bias"]).view(b, s, h, 3 * d)
        q, k, v = packed.split(d, dim=-1)
    else:
        q, k, v = ((x @ w[f"{n}.weight"].t() + w[f"{n}.bias"]).view(b, s, h, d)
                   for n in ("query", "key", "value"))
    ctx = OA.xformers_ref(q, k, v, mask, m.output_proj, compute_dtype=torch.float64)
    ctx = ctx.reshape(b, s, h * d)
    if m.output_proj:
        ctx = ctx @ w["out_proj.weight"].t() + w["out_proj.bias"]
    return ctx


@pytest.mark.parametrize("fused_qkv,output_proj", [(True, True), (False, True), (False, False)])
def test_flash_attention_module_fwd_bwd(fused_qkv, output_proj):
    torch.manual_seed(0)
    b, s, hidden, heads = 2, 256, 512, 8
    m = op.FlashAttention(hidden_size=hidden, num_attention_heads=heads, output_proj=output_proj,
                          attn_pdrop=0.0, resid_pdrop=0.0, attn_op_name="hip_cdna4",
                          fused_qkv=fused_qkv).half().cuda()
    x = torch.randn(b, s, hidden, dtype=torch.float16, device="cuda", requires_grad=True)
    mask = torch.randn(b, 1, 1, s, dtype=torch.float16, device="cuda", requires_grad=True)
    out, present = m(x, mask, None)
    assert present is None and out.shape == (b, s, hidden)
    out.backward(torch.ones_like(out))
    xr = x.detach().cpu().double().requires_grad_(True)
    ref = _oracle_block(m, xr, mask.detach().cpu().double())
    ref.backward(torch.ones_like(ref))
    torch.testing.assert_close(out.detach().cpu().double(), ref.detach(), atol=5e-2, rtol=5e-2)
    torch.testing.assert_close(x.grad.cpu().double(), xr.grad, atol=5e-2, rtol=5e-2)
    assert mask.grad is None  # bias gradient is not produced (as in the reference)
    out2, present = m(x, mask, None, use_cache=True)
    assert present[0].shape == (b, s, heads, hidden // heads)


def test_flash_attention_op_replacement_call():
    """The tutorial's subgraph replacement calls the op with concrete_args attention_mask=None,
    p=0.1 (docs/source/scripts/attention-single-gpu.py:279-282)."""
    core = op.FlashAttentionOp("hip_cdna4", apply_causal_mask=False)
    q, k, v = (torch.randn(2, 64, 4, 64, device="cuda", dtype=torch.bfloat16) for _ in range(3))
    out = core(q, k, v, None, 0.0)
    ref = OA.xformers_ref(q.cpu(), k.cpu(), v.cpu(), None, False, compute_dtype=torch.float64)
    assert_parity(out, ref, torch.bfloat16, "op forward")
    assert core(q, k, v, None, 0.1).shape == q.shape


def test_window_kwarg_local_attention_module():
    m = op.FlashAttention(128, 2, attn_op_name="hip_cdna4", fused_qkv=True, window=16).half().cuda()
    x = torch.randn(1, 96, 128, dtype=torch.float16, device="cuda")
    out, _ = m(x)
    mg = op.FlashAttention(128, 2, attn_op_name="hip_cdna4", fused_qkv=True).half().cuda()
    mg.load_state_dict(m.state_dict())
    out_g, _ = mg(x)
    # the first `window` positions see the same keys under both masks, later ones do not
    assert torch.equal(out[:, :16], out_g[:, :16]) and not torch.equal(out[:, 16:], out_g[:, 16:])


def _attention_with_dropout_tail():
    torch.manual_seed(3)
    m = op.FlashAttention(hidden_size=256, num_attention_heads=4, output_proj=True,
                          attn_pdrop=0.0, resid_pdrop=0.1, attn_op_name="hip_cdna4",
                          fused_qkv=True).half().cuda()
    x = torch.randn(2, 128, 256, dtype=torch.float16, device="cuda")
    return m, x


def _same_mask_close_values(a, b):
    assert ((a == 0) != (b == 0)).float().mean().item() < 5e-4  # exact zeros of the GEMM aside
    assert 0.08 < (a == 0).float().mean().item() < 0.12
    torch.testing.assert_close(a.float(), b.float(), atol=1e-2, rtol=1e-2)


def test_hooks_on_out_proj_fire_and_their_result_is_used():
    """Schedules hang the tensor-parallel all-reduce on `out_proj` as a forward hook
    (`.sync(mode="fwd_post")`: slapo/sharding/shard_ops.py:436-440, model_schedule/gpt2.py:482-485)
    and `.replace` carries hooks over (primitives/replace.py:254).  With a hook on either child the
    block calls the children as the reference does (attention.py:514-516): the hook runs once per
    forward and what it returns is what `resid_dropout` sees.  Without hooks the fused pass runs
    and draws the same mask as `nn.Dropout`."""
    m, x = _attention_with_dropout_tail()
    torch.cuda.manual_seed(77)
    plain, _ = m(x)

    calls = []

    def post(mod, inp, out):
        calls.append(tuple(out.shape))
        return out * 2

    h = m.out_proj.register_forward_hook(post)
    torch.cuda.manual_seed(77)
    hooked, _ = m(x)
    assert calls == [(2, 128, 256)]
    # the same draw masks both paths; values differ by the roundings of GEMM-with-bias then
    # dropout against GEMM then bias + dropout in one pass
    _same_mask_close_values(hooked, plain * 2)
    h.remove()

    pre_calls = []
    h = m.out_proj.register_forward_pre_hook(lambda mod, inp: pre_calls.append(1))
    torch.cuda.manual_seed(77)
    again, _ = m(x)
    assert pre_calls == [1]
    _same_mask_close_values(again, plain)
    h.remove()

    grads = []
    h = m.out_proj.register_full_backward_hook(lambda mod, gi, go: grads.append(go[0].shape))
    xg = x.clone().requires_grad_(True)
    m(xg)[0].sum().backward()
    assert len(grads) == 1
    h.remove()


def test_replaced_children_of_the_tail_are_called_as_modules():
    """A `resid_dropout` replaced by Identity (no `.p`) or an `out_proj` wrapped in another module
    type must keep working: the block then calls them as the reference does."""
    m, x = _attention_with_dropout_tail()
    torch.cuda.manual_seed(5)
    fused, _ = m(x)
    m.resid_dropout = torch.nn.Identity()
    no_drop, _ = m(x)
    kept = fused != 0
    assert torch.allclose(fused[kept].float(), no_drop[kept].float() / 0.9, atol=2e-3, rtol=2e-3)

    class Wrapped(torch.nn.Module):
        def __init__(self, inner):
            super().__init__()
            self.inner = inner

        def forward(self, t):
            return self.inner(t) + 1

    m.out_proj = Wrapped(m.out_proj)
    assert torch.equal(m(x)[0], no_drop + 1)


def test_ops_on_side_streams_from_two_threads():
    """The entry points take the caller's stream and keep no state between calls: two host
    threads, each on a stream of its own (default priority), run attention forward + backward and
    the LayerNorm epilogue at the same time and get what a single-threaded run on the default
    stream gets, bit for bit."""
    import threading

    from slapo_amd import op

    g = torch.Generator().manual_seed(21)
    mk = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).cuda()
    cases = []
    for d in (64, 128):
        q, k, v, do = (mk(2, 384, 4, d) for _ in range(4))
        x, res, gy, w, b = mk(384, 512), mk(384, 512), mk(384, 512), mk(512), mk(512)
        cases.append((q, k, v, do, x, res, gy, w, b))

    def run(case):
        q, k, v, do, x, res, gy, w, b = case
        ql, kl, vl, xl = (t.clone().requires_grad_(True) for t in (q, k, v, x))
        out = op.hip_attention(ql, kl, vl, None, causal=True)
        y = op.bias_dropout_residual_layer_norm(xl, b, res, w, b, 0.0, 1e-5, True)
        grads = torch.autograd.grad((out, y), (ql, kl, vl, xl), (do, gy))
        return (out, y) + tuple(grads)

    want = [run(c) for c in cases]
    torch.cuda.synchronize()
    got, errors = [None, None], []

    def worker(i):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(5):
                    res_ = run(cases[i])
                stream.synchronize()
            got[i] = res_
        except Exception as exc:  # pylint: disable=broad-except
            errors.append(exc)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(60)
    assert not errors, errors
    for i in range(2):
        for a, b_ in zip(got[i], want[i]):
            assert torch.equal(a, b_)
