"""CPU restatement of the reference's fused-bias epilogues (test infrastructure; see
oracle/__init__.py for what pins it).  Follows slapo/op/fused_bias.py line by line in meaning:
`bias_gelu` (:18-21), `bias_gelu_back` (:26-34), `new_gelu` (:49-60), `bias_new_gelu` (:63-64),
`bias_dropout` (:67-74), and the residual fusion pattern of tests/test_fusion.py:179-180.
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
