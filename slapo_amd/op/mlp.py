"""Transformer MLP block on the fused epilogues (reference: slapo/op/mlp.py:10-50)."""
from __future__ import annotations

import torch

from .linear import LinearWithAct, LinearWithDropout


class FusedMLP(torch.nn.Module):
    """fc_in (GEMM + bias-GeLU kernel) -> fc_out (GEMM + bias-dropout kernel).

    Same constructor as the reference.  There, `orig_act` lands in the `bias` slot of
    `LinearWithAct` (mlp.py:39 against linear.py:156-165), so every `orig_act` string runs the
    tanh GeLU of `BiasGeLUFunction`; that behaviour is kept: `orig_act` selects nothing.
    Child names `fc_in` / `fc_out` are what schedules address (model_schedule/gpt2.py:505-520).
    """

    def __init__(self, hidden_size, intermediate_size, orig_act, resid_pdrop,
                 use_torchscript=False):
        super().__init__()
        self.orig_act = orig_act
        self.fc_in = LinearWithAct(hidden_size, intermediate_size, bias=True, act_fn="gelu")
        self.fc_out = LinearWithDropout(intermediate_size, hidden_size, p=resid_pdrop,
                                        use_torchscript=use_torchscript)

    def forward(self, hidden_states):
        return self.fc_out(self.fc_in(hidden_states))
