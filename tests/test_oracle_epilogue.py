"""Pins for oracle/epilogue.py (CPU only)."""
import torch
import torch.nn.functional as F

from oracle import epilogue as OE


def test_bias_gelu_matches_library_tanh_gelu():
    g = torch.Generator().manual_seed(0)
    y = torch.randn(37, 24, generator=g, dtype=torch.float64) * 3
    b = torch.randn(24, generator=g, dtype=torch.float64)
    ref = F.gelu(y + b, approximate="tanh")
    # the reference rounds sqrt(2/pi) to 0.79788456: agreement to ~1e-8, far from any wrong term
    torch.testing.assert_close(OE.bias_gelu(b, y, torch.float64), ref, atol=5e-8, rtol=0)
    torch.testing.assert_close(OE.bias_new_gelu(y, b, torch.float64), ref, atol=1e-12, rtol=0)


def test_bias_gelu_back_is_the_derivative_of_bias_gelu():
    g = torch.Generator().manual_seed(1)
    y = (torch.randn(19, 8, generator=g, dtype=torch.float64) * 2).requires_grad_(True)
    b = torch.randn(8, generator=g, dtype=torch.float64).requires_grad_(True)
    go = torch.randn(19, 8, generator=g, dtype=torch.float64)
    OE.bias_gelu(b, y, torch.float64).backward(go)
    dx, dbias = OE.bias_gelu_bwd(go, b.detach(), y.detach(), torch.float64)
    # 0.1070322243 = 3 * 0.044715 * 0.79788456 to 10 digits
    torch.testing.assert_close(dx, y.grad, atol=1e-9, rtol=0)
    torch.testing.assert_close(dbias, b.grad, atol=1e-8, rtol=0)


def test_bias_dropout_residual_semantics():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(5, 7, 6, generator=g, dtype=torch.float64)
    b = torch.randn(6, generator=g, dtype=torch.float64)
    r = torch.randn(5, 7, 6, generator=g, dtype=torch.float64)
    torch.testing.assert_close(OE.bias_dropout_residual(x, b, None, 0.0, None, torch.float64), x + b)
    torch.testing.assert_close(OE.bias_dropout_residual(x, b, r, 0.0, None, torch.float64), x + b + r)
    keep = torch.rand(5, 7, 6, generator=g) > 0.4
    out = OE.bias_dropout_residual(x, b, r, 0.4, keep, torch.float64)
    torch.testing.assert_close(out[keep], ((x + b) / 0.6 + r)[keep])
    torch.testing.assert_close(out[~keep], r[~keep])
    # matches F.dropout's convention when fed F.dropout's own mask
    torch.manual_seed(3)
    d = F.dropout(torch.ones(5, 7, 6, dtype=torch.float64), 0.4)
    torch.manual_seed(3)
    ref = F.dropout(x + b, 0.4) + r
    torch.testing.assert_close(OE.bias_dropout_residual(x, b, r, 0.4, d != 0, torch.float64), ref)


def test_bias_dropout_residual_bwd_is_autograd():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(9, 6, generator=g, dtype=torch.float64, requires_grad=True)
    b = torch.randn(6, generator=g, dtype=torch.float64, requires_grad=True)
    r = torch.randn(9, 6, generator=g, dtype=torch.float64, requires_grad=True)
    keep = torch.rand(9, 6, generator=g) > 0.2
    go = torch.randn(9, 6, generator=g, dtype=torch.float64)
    OE.bias_dropout_residual(x, b, r, 0.2, keep, torch.float64).backward(go)
    dx, dbias, dres = OE.bias_dropout_residual_bwd(go, 0.2, keep, torch.float64)
    torch.testing.assert_close(dx, x.grad)
    torch.testing.assert_close(dbias, b.grad)
    torch.testing.assert_close(dres, r.grad)


def test_layer_norm_fusion_matches_library_layer_norm_and_autograd():
    """The written-out LayerNorm against F.layer_norm (library routine) and the closed-form
    backward against autograd through the library routine; a biased / unbiased variance mix-up,
    a missing eps or a dropped mean term in dz each fail here."""
    g = torch.Generator().manual_seed(5)
    f64 = torch.float64
    x = torch.randn(4, 9, 12, generator=g, dtype=f64, requires_grad=True)
    b = torch.randn(12, generator=g, dtype=f64, requires_grad=True)
    r = torch.randn(4, 9, 12, generator=g, dtype=f64, requires_grad=True)
    w = torch.randn(12, generator=g, dtype=f64, requires_grad=True)
    lb = torch.randn(12, generator=g, dtype=f64, requires_grad=True)
    keep = torch.rand(4, 9, 12, generator=g) > 0.3
    go = torch.randn(4, 9, 12, generator=g, dtype=f64)
    eps = 1e-2  # large enough that leaving it out is visible
    zz = ((x + b) * keep / 0.7 + r)
    ref = F.layer_norm(zz, (12,), w, lb, eps)
    ref.backward(go)
    y, z, mean, rstd = OE.bias_dropout_residual_layer_norm(
        x.detach(), b.detach(), r.detach(), w.detach(), lb.detach(), eps, 0.3, keep, f64)
    torch.testing.assert_close(y, ref.detach(), atol=1e-12, rtol=0)
    torch.testing.assert_close(z, zz.detach())
    torch.testing.assert_close(mean, zz.detach().mean(-1))
    torch.testing.assert_close(rstd, 1 / torch.sqrt(zz.detach().var(-1, unbiased=False) + eps))
    dx, dbias, dres, dw, dlb = OE.bias_dropout_residual_layer_norm_bwd(
        go, z, mean, rstd, w.detach(), 0.3, keep, f64)
    for got, want in ((dx, x.grad), (dbias, b.grad), (dres, r.grad), (dw, w.grad), (dlb, lb.grad)):
        torch.testing.assert_close(got, want, atol=1e-11, rtol=0)
    # rows that are constant normalise to ln_bias exactly (var = 0, rstd = eps^-1/2)
    y0 = OE.bias_dropout_residual_layer_norm(torch.full((2, 12), 3.0, dtype=f64), None, None,
                                             w.detach(), lb.detach(), eps, 0.0, None, f64)[0]
    torch.testing.assert_close(y0, lb.detach().expand(2, 12))
    # rounding z first changes the statistics the way a bf16 module's stored sum does
    yb = OE.bias_dropout_residual_layer_norm(x.detach(), b.detach(), r.detach(), w.detach(),
                                             lb.detach(), eps, 0.0, None, f64, torch.bfloat16)
    zb = (x + b + r).detach().to(torch.bfloat16).to(f64)
    torch.testing.assert_close(yb[0], F.layer_norm(zb, (12,), w.detach(), lb.detach(), eps))
