"""FusedMLP epilogue parity on the GPU: HIP kernels (through the C ABI) against the CPU oracle
on the same seeded inputs.  Bars: fp32 max-abs 1e-5, bf16/fp16 relative 2e-2; masks bit-exact."""
import pytest
import torch
import torch.nn.functional as F

from oracle import epilogue as OE
from slapo_amd import op
from slapo_amd.op import _kernels as K
from tests.conftest import assert_parity, max_abs_err

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]


def _data(shape, dtype, seed=2013, n=3):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(shape, generator=g).to(dtype) for _ in range(n)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(512, 4096), (4, 33, 1024), (7, 10), (1, 8), (3, 5, 1000)])
def test_bias_gelu_fwd_bwd(dtype, shape):
    y, go = _data(shape, dtype, n=2)
    b = _data((shape[-1],), dtype, seed=1, n=1)[0]
    yd, bd = y.cuda().requires_grad_(True), b.cuda().requires_grad_(True)
    out = op.bias_gelu(yd, bd)
    out.backward(go.cuda())
    ref = OE.bias_gelu(b, y, torch.float64)
    dx, dbias = OE.bias_gelu_bwd(go, b, y, torch.float64)
    assert out.dtype == dtype and out.shape == y.shape
    assert_parity(out, ref, dtype, "bias_gelu fwd")
    assert_parity(yd.grad, dx, dtype, "bias_gelu dx")
    if dtype == torch.float32:
        # a sum over rows: bar scales with the number of addends
        assert max_abs_err(bd.grad, dbias) <= 1e-5 * max(1.0, y.numel() / shape[-1] / 16)
    else:
        assert_parity(bd.grad, dbias, dtype, "bias_gelu dbias")


def test_bias_new_gelu_is_the_same_function():
    y, = _data((64, 256), torch.float32, n=1)
    b, = _data((256,), torch.float32, seed=1, n=1)
    out = op.bias_new_gelu(y.cuda(), b.cuda())
    assert_parity(out, OE.bias_new_gelu(y, b, torch.float64), torch.float32, "gelu_new")
    # and it is the library tanh-GeLU
    assert max_abs_err(out, F.gelu((y + b).double(), approximate="tanh")) <= 1e-5


@pytest.mark.parametrize("dtype", DTYPES)
def test_new_gelu_without_a_bias(dtype):
    """`new_gelu(inp)` of fused_bias.py:49-60 and its autograd-derived gradient."""
    y, go = _data((3, 50, 136), dtype, n=2)
    yd = y.cuda().requires_grad_(True)
    out = op.new_gelu(yd)
    out.backward(go.cuda())
    y64 = y.double().requires_grad_(True)
    ref = OE.new_gelu(y64)
    ref.backward(go.double())
    assert out.dtype == dtype and out.shape == y.shape
    assert_parity(out, ref.detach(), dtype, "new_gelu fwd")
    assert_parity(yd.grad, y64.grad, dtype, "new_gelu dx")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(256, 1024), (4, 33, 1024), (7, 10)])
@pytest.mark.parametrize("residual", [False, True])
def test_bias_dropout_residual_p0(dtype, shape, residual):
    x, r, go = _data(shape, dtype)
    b = _data((shape[-1],), dtype, seed=1, n=1)[0]
    xd, bd, rd = (t.cuda().requires_grad_(True) for t in (x, b, r))
    if residual:
        out = op.bias_dropout_residual(xd, bd, rd, 0.0, True)
    else:
        out = op.bias_dropout(xd, bd, 0.0, True)
    out.backward(go.cuda())
    ref = OE.bias_dropout_residual(x, b, r if residual else None, 0.0, None, torch.float64)
    dx, dbias, dres = OE.bias_dropout_residual_bwd(go, 0.0, None, torch.float64)
    assert_parity(out, ref, dtype, "fwd")
    assert_parity(xd.grad, dx, dtype, "dx")
    if dtype == torch.float32:
        assert max_abs_err(bd.grad, dbias) <= 1e-5 * max(1.0, x.numel() / shape[-1] / 16)
    else:
        assert_parity(bd.grad, dbias, dtype, "dbias")
    if residual:
        assert torch.equal(rd.grad.cpu(), go)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(8192, 1024), (4, 33, 1000), (7, 10)])
def test_bias_dropout_residual_with_dropout(dtype, shape):
    """p = 0.1: the mask must be torch's own mask for the same seed/offset (bit exact) and the
    values must follow the oracle evaluated with that mask."""
    p, seed = 0.1, 2013
    x, r, go = _data(shape, dtype)
    b = _data((shape[-1],), dtype, seed=1, n=1)[0]
    torch.cuda.manual_seed(seed)
    keep = (F.dropout(torch.ones(shape, device="cuda", dtype=dtype), p) != 0).cpu()
    xd, bd, rd = (t.cuda().requires_grad_(True) for t in (x, b, r))
    torch.cuda.manual_seed(seed)
    out = op.bias_dropout_residual(xd, bd, rd, p, True)
    out.backward(go.cuda())
    # mask bits, read off the output: out - residual is zero exactly where dropped
    torch.cuda.manual_seed(seed)
    probe = op.bias_dropout(torch.ones(shape, device="cuda", dtype=dtype),
                            torch.zeros(shape[-1], device="cuda", dtype=dtype), p, True)
    assert torch.equal((probe != 0).cpu(), keep)
    ref = OE.bias_dropout_residual(x, b, r, p, keep, torch.float64)
    dx, dbias, dres = OE.bias_dropout_residual_bwd(go, p, keep, torch.float64)
    assert_parity(out, ref, dtype, "fwd")
    assert_parity(xd.grad, dx, dtype, "dx")
    assert torch.equal((xd.grad != 0).cpu() | (go == 0), keep | (go == 0))
    if dtype == torch.float32:
        assert max_abs_err(bd.grad, dbias) <= 1e-5 * max(1.0, x.numel() / shape[-1] / 16)
    else:
        assert_parity(bd.grad, dbias, dtype, "dbias")
    assert torch.equal(rd.grad.cpu(), go)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape,p", [((1024, 1024), 0.2), ((4, 33, 1024), 0.0), ((37, 2560), 0.1),
                                     ((5, 7, 4096), 0.3), ((19, 8192), 0.1), ((3, 8), 0.5),
                                     ((130, 1000), 0.1), ((17, 264), 0.0)])
def test_bias_dropout_residual_layer_norm(dtype, shape, p):
    """layer_norm(dropout(x + bias) + residual), forward and all five gradients, against the
    oracle evaluated with torch's own mask (wavefront-per-row and block-per-row kernels, both
    mask geometries, ragged row counts)."""
    seed, eps = 2013, 1e-5
    cols = shape[-1]
    if dtype == torch.float32 and cols > 4096:
        pytest.skip("fp32 rows are limited to 4096 columns")
    x, r, go = _data(shape, dtype)
    b, w, lb = _data((cols,), dtype, seed=1, n=3)
    w = (1 + 0.1 * w.float()).to(dtype)
    keep = None
    if p > 0:
        torch.cuda.manual_seed(seed)
        keep = (F.dropout(torch.ones(shape, device="cuda", dtype=dtype), p) != 0).cpu()
    xd, bd, rd, wd, lbd = (t.cuda().requires_grad_(True) for t in (x, b, r, w, lb))
    torch.cuda.manual_seed(seed)
    out = op.bias_dropout_residual_layer_norm(xd, bd, rd, wd, lbd, p, eps, True)
    out.backward(go.cuda())
    # the kernel takes the statistics from z rounded to the tensor type, like the unfused modules
    y, z, mean, rstd = OE.bias_dropout_residual_layer_norm(x, b, r, w, lb, eps, p, keep,
                                                           torch.float64, dtype)
    dx, dbias, dres, dw, dlb = OE.bias_dropout_residual_layer_norm_bwd(go, z, mean, rstd, w, p,
                                                                       keep, torch.float64)
    rows = x.numel() // cols
    assert_parity(out, y, dtype, "y")
    assert_parity(xd.grad, dx, dtype, "dx")
    assert_parity(rd.grad, dres, dtype, "dresidual")
    if p > 0:  # dropped positions carry no gradient, kept ones do (unless dz rounds to zero)
        assert torch.equal((xd.grad != 0).cpu() & ~keep, torch.zeros_like(keep))
    for name, got, want in (("dbias", bd.grad, dbias), ("dweight", wd.grad, dw),
                            ("dln_bias", lbd.grad, dlb)):
        if dtype == torch.float32:
            assert max_abs_err(got, want) <= 1e-5 * max(1.0, rows / 16), name
        else:
            assert_parity(got, want, dtype, name)


def test_layer_norm_fusion_module_and_optional_operands():
    """The module against nn.LayerNorm on the same parameters; bias / residual left out; no
    gradient requested (nothing saved); argument errors."""
    torch.manual_seed(0)
    ln = torch.nn.LayerNorm(512).cuda()
    ln.weight.data.normal_(1, 0.1), ln.bias.data.normal_()
    fused = op.HipBiasDropoutResidualLayerNorm.from_layer_norm(ln, p=0.0)
    assert fused.weight is ln.weight and fused.bias is ln.bias
    x, b, r = torch.randn(6, 50, 512, device="cuda"), torch.randn(512, device="cuda"), \
        torch.randn(6, 50, 512, device="cuda")
    assert max_abs_err(fused(x, b, r), ln(x + b + r).double()) <= 1e-5
    assert max_abs_err(fused(x, None, None), ln(x).double()) <= 1e-5
    assert max_abs_err(fused(x, None, r), ln(x + r).double()) <= 1e-5
    fused.p = 0.5
    fused.eval()
    assert max_abs_err(fused(x, b, r), ln(x + b + r).double()) <= 1e-5
    fused.train()
    torch.cuda.manual_seed(3)
    got = fused(x, b, r)
    torch.cuda.manual_seed(3)
    want = ln(F.dropout(x + b, 0.5) + r)
    assert max_abs_err(got, want.double()) <= 1e-5  # same generator traffic as F.dropout
    with pytest.raises(ValueError):
        op.bias_dropout_residual_layer_norm(x, b, r, ln.weight, ln.bias, 1.5)
    with pytest.raises(ValueError):  # 20000 columns: beyond what a block keeps in registers
        big = torch.randn(2, 20000, device="cuda")
        op.bias_dropout_residual_layer_norm(big, None, None, torch.ones(20000, device="cuda"),
                                            torch.zeros(20000, device="cuda"), 0.0)
    with pytest.raises(ValueError):  # 1002 columns: not a multiple of the 16-byte vector
        odd = torch.randn(2, 1002, device="cuda")
        op.bias_dropout_residual_layer_norm(odd, None, None, torch.ones(1002, device="cuda"),
                                            torch.zeros(1002, device="cuda"), 0.0)


def test_p_one_and_eval_mode():
    x = torch.randn(16, 64, device="cuda")
    b = torch.randn(64, device="cuda")
    r = torch.randn(16, 64, device="cuda")
    assert torch.equal(op.bias_dropout_residual(x, b, r, 1.0, True), r)
    assert max_abs_err(op.bias_dropout(x, b, 0.7, False), (x + b).double()) <= 1e-6
    with pytest.raises(ValueError):
        op.bias_dropout(x, b, 1.5, True)


def test_baseline_epilogue_config_full_size_properties():
    """bf16, tokens 8192, 1024 -> 4096 -> 1024 at full size, through properties that need no
    oracle pass: row-permutation equivariance, bias linearity of the residual epilogue, column
    sums of the backward, and a sampled comparison with the oracle."""
    T, I, Hd = 8192, 4096, 1024
    g = torch.Generator().manual_seed(2013)
    y = torch.randn(T, I, generator=g).bfloat16().cuda()
    b = torch.randn(I, generator=g).bfloat16().cuda()
    out = K.bias_gelu_fwd(y, b)
    perm = torch.randperm(T, device="cuda")
    assert torch.equal(K.bias_gelu_fwd(y[perm], b), out[perm])
    rows = torch.arange(0, T, 257)
    ref = OE.bias_gelu(b.cpu(), y[rows.cuda()].cpu(), torch.float64)
    assert_parity(out[rows.cuda()], ref, torch.bfloat16, "sampled rows")
    go = torch.randn(T, I, generator=g).bfloat16().cuda()
    dx, dbias = K.bias_gelu_bwd(go, y, b)
    colsum = dx.double().sum(0)
    assert ((dbias.double() - colsum).abs().max() / colsum.abs().max()).item() < 1e-2
    x = torch.randn(T, Hd, generator=g).bfloat16().cuda()
    r = torch.randn(T, Hd, generator=g).bfloat16().cuda()
    b2 = torch.randn(Hd, generator=g).bfloat16().cuda()
    plan = K.dropout_plan(T * Hd, 2, "cuda")
    o1 = K.bias_dropout_residual_fwd(x, b2, r, 0.1, 2013, 0, plan)
    o2 = K.bias_dropout_residual_fwd(x, b2, r, 0.1, 2013, 0, plan)
    assert torch.equal(o1, o2)  # a pure function of (seed, offset)
    dropped = (o1 == r)
    frac = dropped.float().mean().item()
    assert abs(frac - 0.1) < 2e-3
    keep = ~dropped
    ref = OE.bias_dropout_residual(x[rows.cuda()].cpu(), b2.cpu(), r[rows.cuda()].cpu(), 0.1,
                                   keep[rows.cuda()].cpu(), torch.float64)
    assert_parity(o1[rows.cuda()], ref, torch.bfloat16, "sampled rows, dropout")


@pytest.mark.parametrize("act", ["gelu", "gelu_new"])
def test_fused_mlp_against_oracle_composite(act):
    """Restates tests/test_op.py::test_fused_mlp: FusedMLP vs the unfused MLP (linear, tanh GeLU,
    linear, dropout) with the same seed => same dropout mask; fp16, p = 0.2; fwd + bwd."""
    torch.manual_seed(0)
    hidden, inter, p = 256, 1024, 0.2
    mlp = op.FusedMLP(hidden, inter, act, p).half().cuda()
    x = torch.randn(4, 128, hidden, dtype=torch.float16, device="cuda", requires_grad=True)
    torch.cuda.manual_seed(2013)
    out = mlp(x)
    out.backward(torch.ones_like(out))
    torch.cuda.manual_seed(2013)
    keep = (F.dropout(torch.ones_like(out), p) != 0).cpu()
    w1, b1 = mlp.fc_in.weight.detach().cpu().double(), mlp.fc_in.bias.detach().cpu().double()
    w2, b2 = mlp.fc_out.weight.detach().cpu().double(), mlp.fc_out.bias.detach().cpu().double()
    xr = x.detach().cpu().double().requires_grad_(True)
    hmid = OE.bias_gelu(b1, xr @ w1.t(), torch.float64)
    ref = OE.bias_dropout_residual(hmid @ w2.t(), b2, None, p, keep, torch.float64)
    ref.backward(torch.ones_like(ref))
    # the reference's own bar for this test is atol = rtol = 5e-2 (tests/test_op.py:207-208)
    torch.testing.assert_close(out.detach().cpu().double(), ref.detach(), atol=5e-2, rtol=5e-2)
    torch.testing.assert_close(x.grad.cpu().double(), xr.grad, atol=5e-2, rtol=5e-2)
    # dropped positions are exact zeros; kept ones are not (up to fp16 underflow)
    assert bool((out.detach().cpu()[~keep] == 0).all())
    assert (out.detach().cpu()[keep] != 0).float().mean().item() > 0.999
