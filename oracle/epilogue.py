"""CPU restatement of the reference's fused-bias epilogues (test infrastructure; see
oracle/__init__.py for what pins it).  Follows slapo/op/fused_bias.py line by line in meaning:
`bias_gelu` (:18-21), `bias_gelu_back` (:26-34), `new_gelu` (:49-60), `bias_new_gelu` (:63-64),
`bias_dropout` (:67-74), the residual fusion pattern of tests/test_fusion.py:179-180 and the
LayerNorm fusion pattern of tests/test_fusion.py:184-185 (`F.layer_norm(F.dropout(x + bias) +
residual, n)`, written out as mean / biased variance / affine, with the backward in closed form).
Dropout takes an explicit boolean keep-mask so that any mask source can be checked.
"""
from __future__ import annotations

import math

import torch


def bias_gelu(bias, y, compute_dtype=torch.float32):
    x = bias.to(compute_dtype) + y.to(compute_dtype)
    return x * 0.5 * (1.0 + torch.tanh(0.79788456 * x * (1 + 0.044715 * x * x)))


def bias_gelu_back(g, bias, y, compute_dtype=torch.float32):
    x = bias.to(compute_dtype) + y.to(compute_dtype)
    tanh_out = torch.tanh(0.79788456 * x * (1 + 0.044715 * x * x))
    ff = 0.5 * x * ((1 - tanh_out * tanh_out) * (0.79788456 + 0.1070322243 * x * x)) + 0.5 * (
        1 + tanh_out
    )
    return ff * g.to(compute_dtype)


def bias_gelu_bwd(g, bias, y, compute_dtype=torch.float32):
    """(dx, dbias): the reference returns the same tensor for both inputs (fused_bias.py:42-46)
    and autograd reduces the bias copy over the broadcast (leading) dimensions."""
    dx = bias_gelu_back(g, bias, y, compute_dtype)
    return dx, dx.reshape(-1, dx.shape[-1]).sum(0)


def new_gelu(inp):
    return 0.5 * inp * (
        1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (inp + 0.044715 * torch.pow(inp, 3.0)))
    )


def bias_new_gelu(inp, bias, compute_dtype=torch.float32):
    return new_gelu(inp.to(compute_dtype) + bias.to(compute_dtype))


def bias_dropout_residual(x, bias, residual=None, p=0.0, keep_mask=None,
                          compute_dtype=torch.float32):
    """dropout(x + bias, p) [+ residual] with inverted-dropout scaling 1/(1-p)."""
    z = x.to(compute_dtype) + bias.to(compute_dtype)
    if p > 0:
        assert keep_mask is not None, "dropout needs an explicit keep-mask"
        z = z.masked_fill(~keep_mask.reshape(z.shape), 0.0) * (1.0 / (1.0 - p))
    if residual is not None:
        z = z + residual.to(compute_dtype)
    return z


def bias_dropout_residual_bwd(g, p=0.0, keep_mask=None, compute_dtype=torch.float32):
    """(dx, dbias, dresidual) of the function above."""
    g = g.to(compute_dtype)
    dx = g
    if p > 0:
        dx = g.masked_fill(~keep_mask.reshape(g.shape), 0.0) * (1.0 / (1.0 - p))
    return dx, dx.reshape(-1, dx.shape[-1]).sum(0), g


def bias_dropout_residual_layer_norm(x, bias, residual, weight, ln_bias, eps=1e-5, p=0.0,
                                     keep_mask=None, compute_dtype=torch.float32, z_dtype=None):
    """(y, z, mean, rstd) with z = dropout(x + bias) + residual and y = (z - mean) rstd weight +
    ln_bias over the last dimension; variance is the biased one, rstd = 1 / sqrt(var + eps)
    (torch.nn.LayerNorm).  z_dtype: round z to this type before the statistics, as a module that
    stores the sum in the tensor type does."""
    zero = torch.zeros(x.shape[-1], dtype=compute_dtype)
    z = bias_dropout_residual(x, bias if bias is not None else zero, residual, p, keep_mask,
                              compute_dtype)
    if z_dtype is not None:
        z = z.to(z_dtype).to(compute_dtype)
    n = z.shape[-1]
    mean = z.sum(-1, keepdim=True) / n
    var = ((z - mean) ** 2).sum(-1, keepdim=True) / n
    rstd = 1.0 / torch.sqrt(var + eps)
    y = (z - mean) * rstd * weight.to(compute_dtype) + ln_bias.to(compute_dtype)
    return y, z, mean.squeeze(-1), rstd.squeeze(-1)


def bias_dropout_residual_layer_norm_bwd(g, z, mean, rstd, weight, p=0.0, keep_mask=None,
                                         compute_dtype=torch.float32):
    """(dx, dbias, dresidual, dweight, dln_bias) of the function above, in closed form:
    with xh = (z - mean) rstd and gw = g weight,
    dz = rstd (gw - mean_c(gw) - xh mean_c(gw xh))."""
    g = g.to(compute_dtype)
    z = z.to(compute_dtype)
    xh = (z - mean.to(compute_dtype).unsqueeze(-1)) * rstd.to(compute_dtype).unsqueeze(-1)
    gw = g * weight.to(compute_dtype)
    dz = rstd.to(compute_dtype).unsqueeze(-1) * (
        gw - gw.mean(-1, keepdim=True) - xh * (gw * xh).mean(-1, keepdim=True))
    dx, dbias, dres = bias_dropout_residual_bwd(dz, p, keep_mask, compute_dtype)
    cols = z.shape[-1]
    return dx, dbias, dres, (g * xh).reshape(-1, cols).sum(0), g.reshape(-1, cols).sum(0)
