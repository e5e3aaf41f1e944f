"""The kernels as schedules install them: a block is traced, a functional subgraph is matched
and replaced by a HIP payload under the reference's arity rule (slapo/primitives/replace.py:48-88),
a whole attention module is replaced by FlashAttention with the keyword arguments of
slapo/model_schedule/gpt2.py:212-220, and fork_rng wraps a forward as
slapo/primitives/tensor_parallel.py:183-194 does.  Each test compares the scheduled block with the
unscheduled one under the same seeds, restating tests/test_fusion.py:118-204 and
tests/test_fork_rng.py:56-67 of the reference (its bars: torch.testing.assert_close defaults)."""
import copy
import operator

import pytest
import torch
import torch.nn.functional as F
from torch import nn

import slapo_amd
from slapo_amd import op
from tests import sched_shim as S

pytestmark = pytest.mark.gpu


def _seed(s=9999):
    torch.manual_seed(s)
    torch.cuda.manual_seed(s)


class _GeluBlock(nn.Module):
    def __init__(self):
        super().__init__()
        self.linear = nn.Linear(1024, 1024)

    def forward(self, x):
        # the reference's fused kernel is the tanh form (slapo/op/fused_bias.py:18-21)
        return F.gelu(self.linear(x), approximate="tanh")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_fuse_bias_gelu_subgraph(dtype):
    _seed()
    mod = _GeluBlock().to(dtype).cuda()
    sch = copy.deepcopy(mod)
    S.decompose(sch, "linear")
    gm = S.trace(sch)

    def pattern(x, bias):
        return F.gelu(x + bias, approximate="tanh")

    found = S.find(gm, pattern)
    assert len(found) == 1 and len(found[0]) == 2
    assert found[0][0].target == operator.add and found[0][1].target == F.gelu
    name = S.replace_subgraph(gm, found[0], op.HipBiasGeLU(), "BiasGeLU")
    assert name == "BiasGeLU_0" and gm.BiasGeLU_0.__class__.__name__ == "HipBiasGeLU"
    assert not [n for n in gm.graph.nodes if n.target in (F.gelu, operator.add)]

    x = torch.randn(1, 16, 256, 1024, dtype=dtype, device="cuda", requires_grad=True)
    xr = x.detach().clone().requires_grad_(True)
    out, ref = gm(x), mod(xr)
    # fp16: the unfused block rounds GEMM + bias once and the activation once more, the fused one
    # rounds the GEMM, adds the bias in fp32 and rounds the activation: one fp16 ulp apart
    tol = dict(rtol=5e-3, atol=5e-3) if dtype == torch.float16 else dict(rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(out, ref, **tol)
    out.sum().backward()
    ref.sum().backward()
    torch.testing.assert_close(x.grad, xr.grad, **tol)
    torch.testing.assert_close(gm.linear.bias.grad, mod.linear.bias.grad, rtol=2e-3, atol=2e-2)


class _Projection(nn.Module):
    def __init__(self, p):
        super().__init__()
        self.linear = nn.Linear(1024, 1024)
        self.ln = nn.LayerNorm(1024)
        self.p = p

    def forward(self, x, residual):
        x = F.dropout(self.linear(x), 0.2)
        return self.ln(x + residual)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_fuse_bias_dropout_residual_layer_norm_subgraph(dtype):
    _seed()
    p = 0.2
    mod = _Projection(p).to(dtype).cuda()
    sch = copy.deepcopy(mod)
    S.decompose(sch, "linear")
    gm = S.trace(sch)

    def pattern(x, bias, residual):
        return F.dropout(x + bias, 0.2) + residual

    found = S.find(gm, pattern)
    assert len(found) == 1 and len(found[0]) == 3
    ops = found[0]
    (ln_node,) = list(ops[-1].users)  # the LayerNorm module that consumes the sum, as in
    ops = ops + [ln_node]             # tests/test_fusion.py:187-191 of the reference
    assert [n.target for n in ops] == [operator.add, F.dropout, operator.add, "ln"]
    with pytest.raises(ValueError, match="does not match"):
        S.required_args(op.HipBiasGeLU(), ops)  # two required arguments against three inputs
    payload = op.HipBiasDropoutResidualLayerNorm.from_layer_norm(gm.ln, p)
    assert S.replace_subgraph(gm, ops, payload, "FusedLN") == "FusedLN_0"
    assert [n.target for n in gm.graph.nodes if n.op == "call_module"] == ["FusedLN_0"]

    x = torch.randn(1, 16, 256, 1024, dtype=dtype, device="cuda", requires_grad=True)
    res = torch.randn(1, 16, 256, 1024, dtype=dtype, device="cuda", requires_grad=True)
    xr, rr = x.detach().clone().requires_grad_(True), res.detach().clone().requires_grad_(True)
    _seed(5)
    out = gm(x, res)
    _seed(5)
    ref = mod(xr, rr)  # same seed: F.dropout and the fused kernel draw the same mask
    tol = dict(rtol=1.6e-2, atol=3e-2) if dtype == torch.bfloat16 else dict(rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(out, ref, **tol)
    g = torch.randn_like(out)
    out.backward(g)
    ref.backward(g)
    torch.testing.assert_close(x.grad, xr.grad, **tol)
    torch.testing.assert_close(res.grad, rr.grad, **tol)
    torch.testing.assert_close(gm.FusedLN_0.weight.grad, mod.ln.weight.grad, rtol=2e-2, atol=0.5)


class _TinyGPT2Attention(nn.Module):
    """The unscheduled block: GPT-2 style causal self-attention written with plain torch ops on
    the parameter layout of FlashAttention(fused_qkv=True)."""

    def __init__(self, hidden, heads, resid_pdrop):
        super().__init__()
        self.heads, self.head_size = heads, hidden // heads
        self.qkv = nn.Linear(hidden, 3 * hidden)
        self.out_proj = nn.Linear(hidden, hidden)
        self.resid_dropout = nn.Dropout(resid_pdrop)

    def forward(self, hidden_states, attention_mask=None):
        b, s, _ = hidden_states.shape
        packed = self.qkv(hidden_states).view(b, s, self.heads, 3 * self.head_size)
        q, k, v = (t.transpose(1, 2).float() for t in packed.split(self.head_size, dim=-1))
        scores = q @ k.transpose(-1, -2) * self.head_size ** -0.5
        if attention_mask is not None:
            scores = scores + attention_mask.float()
        causal = torch.ones(s, s, dtype=torch.bool, device=scores.device).tril()
        scores = scores.masked_fill(~causal, float("-inf"))
        ctx = (scores.softmax(-1) @ v).transpose(1, 2).reshape(b, s, -1).to(hidden_states.dtype)
        return (self.resid_dropout(self.out_proj(ctx)), None)


class _Layer(nn.Module):
    def __init__(self, hidden, heads, resid_pdrop):
        super().__init__()
        self.ln_1 = nn.LayerNorm(hidden)
        self.attn = _TinyGPT2Attention(hidden, heads, resid_pdrop)

    def forward(self, x, attention_mask=None):
        return x + self.attn(self.ln_1(x), attention_mask)[0]


@pytest.mark.parametrize("resid_pdrop", [0.0, 0.1])
def test_replace_attention_module_with_flash_attention(resid_pdrop):
    _seed()
    hidden, heads = 512, 8
    mod = _Layer(hidden, heads, resid_pdrop).half().cuda()
    sch = copy.deepcopy(mod)
    init_config = dict(hidden_size=hidden, num_attention_heads=heads, output_proj=True,
                       attn_pdrop=0.0, resid_pdrop=resid_pdrop, attn_op_name="hip_cdna4",
                       fused_qkv=True)  # model_schedule/gpt2.py:212-220
    new = op.FlashAttention(**init_config).half().cuda()
    new.load_state_dict(sch.attn.state_dict())  # same child names: qkv, out_proj
    S.replace_module(sch, "attn", new)
    assert isinstance(sch.attn, op.FlashAttention) and sch.attn.resid_dropout.p == resid_pdrop

    x = torch.randn(2, 256, hidden, dtype=torch.float16, device="cuda", requires_grad=True)
    xr = x.detach().clone().requires_grad_(True)
    mask = torch.zeros(2, 1, 1, 256, dtype=torch.float16, device="cuda")
    mask[1, ..., 200:] = torch.finfo(torch.float16).min
    _seed(3)
    out = sch(x, mask)
    _seed(3)
    ref = mod(xr, mask)  # resid_dropout draws the same mask on both sides
    torch.testing.assert_close(out, ref, rtol=5e-2, atol=5e-2)  # tests/test_op.py:130 bar
    if resid_pdrop > 0:  # the dropped positions coincide exactly
        with torch.no_grad():
            h = mod.ln_1(x)
            _seed(4)
            a = sch.attn(h, mask)[0]
            _seed(4)
            r = mod.attn(h, mask)[0]
        # the same positions are dropped on both sides (two independent masks would disagree on
        # 18 % of them); the few zeros that are not shared are sums GEMM + bias that cancel
        # exactly in one rounding order and not in the other
        assert 0.05 < (a == 0).float().mean() < 0.2
        assert ((a == 0) != (r == 0)).float().mean() < 5e-4
    g = torch.randn_like(out)
    out.backward(g)
    ref.backward(g)
    torch.testing.assert_close(x.grad, xr.grad, rtol=5e-2, atol=5e-2)


class _DropoutModel(nn.Module):
    def __init__(self):
        super().__init__()
        self.proj = op.LinearWithDropout(64, 64, p=0.5)

    def forward(self, x):
        return self.proj(x)


def test_fork_rng_wraps_forward_and_decorrelates_ranks():
    """tests/test_fork_rng.py:56-67 on one device: the tensor-parallel ranks are played one after
    the other through their seeds.  Without fork_rng every rank draws the same mask; with it the
    masks differ, and the default stream is where it would be without the fork."""
    model = _DropoutModel().cuda()
    data = torch.randn(10, 64, device="cuda")

    def run(m, tp_rank):
        slapo_amd.set_random_seed(123, None, None, tp_rank)
        out = m(data)
        return out, torch.cuda.default_generators[0].get_offset()

    plain = [run(model, r)[0] for r in (0, 1)]
    torch.testing.assert_close(plain[0], plain[1])

    forked = S.fork_rng(copy.deepcopy(model))
    assert forked.traceable is False
    gm = S.trace(nn.Sequential(forked))  # a non-traceable module stays one call_module node
    assert [n.op for n in gm.graph.nodes] == ["placeholder", "call_module", "output"]
    outs = [run(forked, r) for r in (0, 1)]
    with pytest.raises(AssertionError):
        torch.testing.assert_close(outs[0][0], outs[1][0])
    # the fork leaves the default stream untouched (the draw came from the forked state)
    slapo_amd.set_random_seed(123, None, None, 0)
    assert outs[0][1] == torch.cuda.default_generators[0].get_offset()


# ---- the attention wrappers of the other model schedules ---------------------------------------
from oracle import attention as OA  # noqa: E402
from tests import adapters as AD  # noqa: E402


def _hf_padding_mask(b, s, valid, dtype):
    """HF extended attention mask: 0 on valid keys, finfo.min on padded ones, [B,1,1,S]."""
    m = torch.zeros(b, 1, 1, s, dtype=dtype, device="cuda")
    for i, n in enumerate(valid):
        m[i, :, :, n:] = torch.finfo(dtype).min
    return m


def _oracle_of(m, x, mask):
    """What the wrapped FlashAttention computes, from its own weights, on the CPU in fp64."""
    w = {n: p.detach().cpu().double() for n, p in m.named_parameters()}
    b, s, _ = x.shape
    h, d = m.num_attention_heads, m.attention_head_size
    packed = x.cpu().double() @ w["qkv.weight"].t()
    if "qkv.bias" in w:
        packed = packed + w["qkv.bias"]
    q, k, v = packed.view(b, s, h, 3 * d).split(d, dim=-1)
    ctx = OA.xformers_ref(q, k, v, None if mask is None else mask.cpu().double(), m.output_proj,
                          compute_dtype=torch.float64).reshape(b, s, h * d)
    if m.output_proj:
        ctx = ctx @ w["out_proj.weight"].t()
        if "out_proj.bias" in w:
            ctx = ctx + w["out_proj.bias"]
    return ctx


@pytest.mark.parametrize("family", ["gpt2", "gpt_neo", "opt", "bert", "albert"])
def test_model_schedule_wrappers_call_and_trim_as_the_reference_does(family):
    """Each wrapper is called the way its HF parent layer calls the original attention, and must
    hand back what that layer unpacks: gpt2.py:241-264 and gpt_neo.py:193-215 (`outputs[:1]`),
    opt.py:169-201 (`(out, None, None)`), bert.py:196-208 (`outputs[:1]`), albert.py:196-205
    (`(context, None)`).  Values against the oracle at the bar of the reference's module test
    (tests/test_op.py: atol = rtol = 5e-2 in fp16)."""
    _seed(4)
    dtype = torch.float16
    cfg = AD.model_config()
    wrapper = AD.make_adapter(family, op.FlashAttention, cfg, "cuda").to(dtype).cuda()
    b, s = 2, 192
    x = torch.randn(b, s, cfg.hidden_size, dtype=dtype, device="cuda")
    mask = _hf_padding_mask(b, s, [s, 150], dtype)
    if family == "gpt2":  # GPT2Block: attn(hidden, layer_past=, attention_mask=, head_mask=, ...)
        out = wrapper(x, layer_past=None, attention_mask=mask, head_mask=None, use_cache=False,
                      output_attentions=False)
        assert isinstance(out, tuple) and len(out) == 1
    elif family == "gpt_neo":  # GPTNeoBlock: same keywords without the encoder pair
        out = wrapper(x, layer_past=None, attention_mask=mask, head_mask=None, use_cache=False,
                      output_attentions=False)
        assert isinstance(out, tuple) and len(out) == 1
    elif family == "opt":  # OPTDecoderLayer unpacks three values
        out = wrapper(hidden_states=x, past_key_value=None, attention_mask=mask,
                      layer_head_mask=None, output_attentions=False)
        assert len(out) == 3 and out[1] is None and out[2] is None
    elif family == "bert":  # BertAttention: self(hidden, attention_mask, head_mask, ...)
        out = wrapper(x, mask, None, None, None, None, False)
        assert isinstance(out, tuple) and len(out) == 1
    else:  # AlbertLayer: attention(hidden, attention_mask, head_mask, output_attentions)
        out = wrapper(x, mask, None, False)
        assert len(out) == 2 and out[1] is None
    ref = _oracle_of(AD.inner(wrapper), x, mask)
    torch.testing.assert_close(out[0].cpu().double(), ref, atol=5e-2, rtol=5e-2)


def test_gpt_neo_wrapper_has_no_projection_biases_and_trains():
    """bias=False (gpt_neo.py:171) removes the biases of qkv and out_proj; the block's tail then
    runs as the two child calls (there is no bias for the fused pass to add)."""
    _seed(5)
    wrapper = AD.make_adapter("gpt_neo", op.FlashAttention,
                              AD.model_config(resid_dropout=0.1, attention_dropout=0.1),
                              "triton").half().cuda()
    m = AD.inner(wrapper)
    assert m.qkv.bias is None and m.out_proj.bias is None
    x = torch.randn(2, 128, 256, dtype=torch.float16, device="cuda", requires_grad=True)
    (out,) = wrapper(x, attention_mask=None)
    out.float().sum().backward()
    assert torch.isfinite(x.grad.float()).all() and m.qkv.weight.grad is not None
    assert 0.05 < (out == 0).float().mean().item() < 0.15  # resid_dropout ran
