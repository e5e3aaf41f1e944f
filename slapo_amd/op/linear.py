"""Linear layers whose bias is applied by a fused HIP epilogue after the GEMM.

Interface-compatible with the reference's slapo/op/linear.py: `LinearWithSeparateBias` (:60-68),
`LinearWithSyncFunc` (:71-131), `LinearWithAct` (:134-191), `LinearWithDropout` (:194-264) and
`FusedQKV` (:20-57).  The GEMM stays on the vendor BLAS (F.linear without bias); what follows it
-- optional `sync_fn`, then bias + activation or bias + dropout -- is one kernel launch.
"""
from __future__ import annotations

from functools import partial

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from .fused_bias import BiasGeLUFunction, bias_dropout, bias_new_gelu


class FusedQKV(nn.Module):
    """One GEMM for Q, K and V with the [heads, head_size, 3] output interleave of the
    reference (linear.py:41-57); `world_size` divides the heads held by this rank."""

    def __init__(self, hidden_size, num_heads, world_size) -> None:
        super().__init__()
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.head_size = hidden_size // num_heads
        self.world_size = world_size
        self.fused_linear = nn.Linear(hidden_size, self.num_heads * self.head_size * 3)

    def reshape_for_scores(self, x):
        shape = x.size()[:-1] + (self.num_heads // self.world_size, self.head_size, 3)
        return x.view(shape).contiguous()

    def forward(self, hidden_states):
        packed = self.reshape_for_scores(self.fused_linear(hidden_states))
        return [t.squeeze(-1).contiguous() for t in torch.split(packed, 1, dim=-1)]


class LinearWithSeparateBias(nn.Linear):
    """nn.Linear computed as GEMM then `+ bias`, so a tracer sees the bias add as its own node
    (what `.decompose()` installs before `.fuse()`)."""

    def forward(self, x: Tensor) -> Tensor:
        return F.linear(x, self.weight, None) + self.bias


class LinearWithSyncFunc(nn.Linear):
    """nn.Linear with a hook (`sync_fn`, e.g. a tensor-parallel all-reduce) between the GEMM
    and the bias addition.  `sync_fn` is a plain mutable attribute: schedules assign it later."""

    def __init__(self, in_features, out_features, bias=True, device=None, dtype=None,
                 sync_fn=None):
        super().__init__(in_features, out_features, bias, device, dtype)
        self.traceable = False
        self.sync_fn = sync_fn

    def _gemm_and_sync(self, x):
        x = F.linear(x, self.weight, None)
        return self.sync_fn(x) if self.sync_fn is not None else x

    def forward(self, x):
        x = self._gemm_and_sync(x)
        return x if self.bias is None else x + self.bias

    def _sync_fn_repr(self):
        fn = self.sync_fn
        if fn is None:
            return "None"
        if hasattr(fn, "__name__"):
            return fn.__name__
        if isinstance(fn, partial):
            fixed = ", ".join(str(a) for a in fn.args)
            if fn.keywords:
                fixed += ", ".join(f"{k}={v}" for k, v in fn.keywords.items())
            return f"partial({fn.func.__name__}, {fixed})"
        return str(fn)

    def extra_repr(self):
        return f"{super().extra_repr()}, sync_fn={self._sync_fn_repr()}"


class LinearWithAct(LinearWithSyncFunc):
    """GEMM -> sync_fn -> fused bias + GeLU.  `act_fn` is "gelu" or "gelu_new"; both are the
    tanh formulation and run the same kernel.  Requires a bias (ValueError otherwise), rejects
    other activations with NotImplementedError, as the reference does (linear.py:166-182)."""

    def __init__(self, in_features, out_features, bias=True, act_fn="gelu", device=None,
                 dtype=None, sync_fn=None):
        super().__init__(in_features, out_features, bias, device, dtype, sync_fn)
        self.act_fn = act_fn
        if not bias:
            raise ValueError(
                "LinearWithAct requires bias. Please set bias=True or simply use nn.Linear"
            )
        if act_fn == "gelu":
            self.act = BiasGeLUFunction.apply
        elif act_fn == "gelu_new":
            self.act = bias_new_gelu
        else:
            raise NotImplementedError(f"Unsupported activation: {self.act_fn}")

    def forward(self, x: Tensor) -> Tensor:
        return self.act(self._gemm_and_sync(x), self.bias)

    def extra_repr(self):
        return f"{super().extra_repr()}, act_fn={self.act_fn}"


class LinearWithDropout(LinearWithSyncFunc):
    """GEMM -> sync_fn -> fused bias + dropout.  The mask is the one torch's own dropout would
    draw from the same generator state.  `use_torchscript` is kept for signature compatibility
    and only echoed by `extra_repr`: there is a single kernel path here."""

    def __init__(self, in_features, out_features, bias=True, p=0.5, inplace=False, device=None,
                 dtype=None, sync_fn=None, use_torchscript=False):
        super().__init__(in_features, out_features, bias, device, dtype, sync_fn)
        if not bias:
            raise ValueError(
                "LinearWithDropout requires bias. Please set bias=True or simply use nn.Linear"
            )
        self.p = p
        self.inplace = inplace
        self.use_torchscript = use_torchscript
        self.dropout = bias_dropout

    def forward(self, x: Tensor) -> Tensor:
        return self.dropout(self._gemm_and_sync(x), self.bias, self.p, self.training,
                            self.inplace)

    def extra_repr(self):
        return (f"{super().extra_repr()}, p={self.p}, inplace={self.inplace}, "
                f"use_torchscript={self.use_torchscript}")
