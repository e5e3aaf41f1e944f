"""Fused ops with the reference's names (slapo/op/__init__.py:4-8) on HIP kernels."""
from .attention import FlashAttention, FlashAttentionOp, hip_attention
from .cross_entropy import ParallelCrossEntropy, vocab_parallel_cross_entropy
from .fused_bias import (BiasGeLUFunction, HipBiasDropoutResidual,
                         HipBiasDropoutResidualLayerNorm, HipBiasGeLU, bias_dropout,
                         bias_dropout_residual, bias_dropout_residual_layer_norm, bias_gelu,
                         bias_new_gelu, new_gelu)
from .linear import (FusedQKV, LinearWithAct, LinearWithDropout, LinearWithSeparateBias,
                     LinearWithSyncFunc)
from .mlp import FusedMLP
