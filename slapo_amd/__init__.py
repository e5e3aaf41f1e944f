"""slapo_amd: MI355X (gfx950) kernels behind Slapo's fused-op interface.

`slapo_amd.op` mirrors `slapo.op` (FlashAttention, FlashAttentionOp, FusedMLP, LinearWith*),
`slapo_amd.random` mirrors `slapo.random`, `slapo_amd.checkpoint` mirrors `slapo.checkpoint`.  Importing the package loads nothing native; the
first kernel call loads libslapo_amd.so and fails loudly when it has not been built.
"""
from . import op
from .checkpoint import checkpoint
from .random import (get_cuda_rng_tracker, is_random_seed_set, model_parallel_cuda_manual_seed,
                     set_random_seed)

__version__ = "0.1.0"
