"""Bias epilogues fused with the following activation / dropout, on hand-written HIP kernels.

Same public names and call signatures as the reference's slapo/op/fused_bias.py
(`BiasGeLUFunction` :13-46, `new_gelu` :49-60, `bias_new_gelu` :63-64, `bias_dropout` :67-74); each runs as ONE
streaming kernel per direction instead of a TorchScript / functorch fusion.  Two modules,
`HipBiasGeLU` and `HipBiasDropoutResidual`, package them with the positional signatures
(`forward(x, bias)`, `forward(x, bias, residual)`) that `sch.replace(module, subgraph)` needs
for the fusion patterns of tests/test_fusion.py:118-204.
"""
from __future__ import annotations

import torch
from torch import nn

from ..random import draw_philox_state
from . import _kernels as K


class BiasGeLUFunction(torch.autograd.Function):
    """gelu_tanh(inp + bias); backward is the closed form of fused_bias.py:26-34 and returns the
    bias gradient already reduced to the bias shape."""

    # pylint: disable=arguments-differ, abstract-method
    @staticmethod
    def forward(ctx, inp, bias):
        ctx.save_for_backward(inp, bias)
        return K.bias_gelu_fwd(inp, bias)

    @staticmethod
    def backward(ctx, grad_output):
        inp, bias = ctx.saved_tensors
        dx, dbias = K.bias_gelu_bwd(grad_output, inp, bias, need_dbias=ctx.needs_input_grad[1])
        if dbias is not None and dbias.dtype != bias.dtype:
            dbias = dbias.to(bias.dtype)
        return (dx if ctx.needs_input_grad[0] else None), dbias


def bias_gelu(inp: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    return BiasGeLUFunction.apply(inp, bias)


class _NewGeLU(torch.autograd.Function):
    """The same kernels with a zero bias and no bias gradient."""

    # pylint: disable=arguments-differ, abstract-method
    @staticmethod
    def forward(ctx, inp):
        zero = inp.new_zeros(inp.shape[-1])
        ctx.save_for_backward(inp, zero)
        return K.bias_gelu_fwd(inp, zero)

    @staticmethod
    def backward(ctx, grad_output):
        inp, zero = ctx.saved_tensors
        dx, _ = K.bias_gelu_bwd(grad_output, inp, zero, need_dbias=False)
        return dx


def new_gelu(inp: torch.Tensor) -> torch.Tensor:
    """HF `gelu_new` (fused_bias.py:49-60) as one kernel per direction."""
    return _NewGeLU.apply(inp)


def bias_new_gelu(inp: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """HF `gelu_new` on inp + bias.  Its constant sqrt(2/pi) equals the 0.79788456 of
    `BiasGeLUFunction` to 8 digits, so both names share one kernel."""
    return BiasGeLUFunction.apply(inp, bias)


class _BiasDropoutResidual(torch.autograd.Function):
    # pylint: disable=arguments-differ, abstract-method
    @staticmethod
    def forward(ctx, x, bias, residual, p):
        plan, seed, offset, rng_state = None, 0, 0, None
        if x.numel() == 0:
            p = 0.0  # nothing to drop, and F.dropout leaves the generator alone for an empty tensor
        if 0.0 < p:
            plan = K.dropout_plan(x.numel(), x.element_size(), x.device)
            if p < 1.0:
                # The generator moves exactly as it would for F.dropout on this tensor.
                seed, offset, rng_state = draw_philox_state(plan.offset_increment, x.device)
        ctx.p, ctx.seed, ctx.offset, ctx.plan = p, seed, offset, plan
        ctx.rng_state = rng_state  # a non-differentiable two-element tensor, or None
        ctx.bias_like = bias
        ctx.has_residual = residual is not None
        return K.bias_dropout_residual_fwd(x, bias, residual, p, seed, offset, plan,
                                           rng_state=rng_state)

    @staticmethod
    def backward(ctx, grad_output):
        need_dx, need_dbias = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        dx = dbias = None
        if need_dx or need_dbias:
            if ctx.p == 0.0 and not need_dbias:
                dx = grad_output
            else:
                dx, dbias = K.bias_dropout_residual_bwd(
                    grad_output, ctx.bias_like, ctx.p, ctx.seed, ctx.offset, ctx.plan,
                    need_dx=need_dx, need_dbias=need_dbias, rng_state=ctx.rng_state)
        dres = grad_output if (ctx.has_residual and ctx.needs_input_grad[2]) else None
        return dx, dbias, dres, None


def bias_dropout(x: torch.Tensor, bias: torch.Tensor, p: float = 0.5, training: bool = True,
                 inplace: bool = False) -> torch.Tensor:
    """dropout(x + bias).  `inplace` is accepted for signature compatibility; the reference's
    in-place target is the temporary x + bias, which this kernel never materialises."""
    del inplace
    _check_p(p)
    return _BiasDropoutResidual.apply(x, bias, None, float(p) if training else 0.0)


def bias_dropout_residual(x: torch.Tensor, bias: torch.Tensor, residual: torch.Tensor,
                          p: float = 0.5, training: bool = True) -> torch.Tensor:
    """dropout(x + bias) + residual, the pattern of tests/test_fusion.py:179-180."""
    _check_p(p)
    return _BiasDropoutResidual.apply(x, bias, residual, float(p) if training else 0.0)


class _BiasDropoutResidualLayerNorm(torch.autograd.Function):
    # pylint: disable=arguments-differ, abstract-method
    @staticmethod
    def forward(ctx, x, bias, residual, weight, ln_bias, p, eps):
        plan, seed, offset, rng_state = None, 0, 0, None
        if x.numel() == 0:
            p = 0.0  # nothing to drop, and F.dropout leaves the generator alone for an empty tensor
        if 0.0 < p:
            plan = K.dropout_plan(x.numel(), x.element_size(), x.device)
            if p < 1.0:
                # The generator moves exactly as it would for F.dropout on this tensor.
                seed, offset, rng_state = draw_philox_state(plan.offset_increment, x.device)
        need_grad = any(ctx.needs_input_grad[:5])
        y, z, mean, rstd = K.bias_dropout_residual_ln_fwd(
            x, bias, residual, weight, ln_bias, eps, p, seed, offset, plan,
            save_for_backward=need_grad, rng_state=rng_state)
        ctx.rng_state = rng_state  # a non-differentiable two-element tensor, or None
        ctx.cfg = (p, seed, offset, plan, bias is not None, residual is not None)
        ctx.dtypes = tuple(t.dtype if t is not None else None for t in (bias, weight, ln_bias))
        ctx.save_for_backward(z, mean, rstd, weight)
        return y

    @staticmethod
    def backward(ctx, grad_output):
        z, mean, rstd, weight = ctx.saved_tensors
        p, seed, offset, plan, has_bias, has_residual = ctx.cfg
        need = ctx.needs_input_grad
        dx, dres, dw, dlb, db = K.bias_dropout_residual_ln_bwd(
            grad_output, z, mean, rstd, weight, p, seed, offset, plan, need_dx=need[0],
            need_dres=has_residual and need[2], need_dweight=need[3], need_dln_bias=need[4],
            need_dbias=has_bias and need[1], rng_state=ctx.rng_state)
        cast = lambda t, dt: t if t is None or t.dtype == dt else t.to(dt)
        return (dx, cast(db, ctx.dtypes[0]), dres, cast(dw, ctx.dtypes[1]),
                cast(dlb, ctx.dtypes[2]), None, None)


def bias_dropout_residual_layer_norm(x: torch.Tensor, bias, residual, weight: torch.Tensor,
                                     ln_bias: torch.Tensor, p: float = 0.5, eps: float = 1e-5,
                                     training: bool = True) -> torch.Tensor:
    """layer_norm(dropout(x + bias) + residual) over the last dimension, the pattern of
    tests/test_fusion.py:184-185 (bias and residual may be None)."""
    _check_p(p)
    return _BiasDropoutResidualLayerNorm.apply(x, bias, residual, weight, ln_bias,
                                               float(p) if training else 0.0, float(eps))


def _check_p(p):
    if p < 0.0 or p > 1.0:
        raise ValueError(f"dropout probability has to be between 0 and 1, but got {p}")


class HipBiasGeLU(nn.Module):
    """Replacement payload for a matched `gelu(x + bias)` subgraph."""

    def forward(self, x, bias):
        return BiasGeLUFunction.apply(x, bias)


class HipBiasDropoutResidual(nn.Module):
    """Replacement payload for a matched `dropout(x + bias) + residual` subgraph."""

    def __init__(self, p: float = 0.5):
        super().__init__()
        _check_p(p)
        self.p = p

    def forward(self, x, bias, residual):
        return bias_dropout_residual(x, bias, residual, self.p, self.training)

    def extra_repr(self):
        return f"p={self.p}"


class HipBiasDropoutResidualLayerNorm(nn.Module):
    """Replacement payload for a matched `layer_norm(dropout(x + bias) + residual)` subgraph;
    owns the LayerNorm parameters under the names of `nn.LayerNorm` (`weight`, `bias`)."""

    def __init__(self, normalized_shape: int, p: float = 0.5, eps: float = 1e-5, device=None,
                 dtype=None):
        super().__init__()
        _check_p(p)
        if not isinstance(normalized_shape, int):
            if len(normalized_shape) != 1:
                raise NotImplementedError("only the last dimension can be normalized")
            normalized_shape = int(normalized_shape[0])
        self.normalized_shape = (normalized_shape,)
        self.p, self.eps = p, eps
        self.weight = nn.Parameter(torch.ones(normalized_shape, device=device, dtype=dtype))
        self.bias = nn.Parameter(torch.zeros(normalized_shape, device=device, dtype=dtype))

    @classmethod
    def from_layer_norm(cls, ln: nn.LayerNorm, p: float):
        """Takes over the parameters of an existing nn.LayerNorm (shared, not copied)."""
        if not ln.elementwise_affine or ln.bias is None:
            raise NotImplementedError("LayerNorm without affine parameters")
        mod = cls(ln.normalized_shape, p, ln.eps, device=ln.weight.device, dtype=ln.weight.dtype)
        mod.weight, mod.bias = ln.weight, ln.bias
        return mod

    def forward(self, x, bias, residual):
        return bias_dropout_residual_layer_norm(x, bias, residual, self.weight, self.bias,
                                                self.p, self.eps, self.training)

    def extra_repr(self):
        return f"{self.normalized_shape}, p={self.p}, eps={self.eps}"
