"""CPU oracle for the Slapo fused-op hot path.  TEST INFRASTRUCTURE ONLY.

This package restates, on the CPU, the arithmetic of the reference's native PyTorch path
(awslabs/slapo, slapo/op/attention.py, slapo/op/fused_bias.py, slapo/op/cross_entropy.py and
the LayerNorm fusion pattern of tests/test_fusion.py:157-204) and of the Philox dropout
mask that torch.nn.functional.dropout draws on a ROCm device.  Only tests/, the smoke check in
__graft_entry__.py and the cpu_baseline leg of bench.py may import it; the product package
(slapo_amd) never does and has no CPU path of its own.

What pins each function (none of them is pinned by retyping its own formula):

  attention.attention_bmk / xformers_ref / flash_attn_ref (forward)
      torch.nn.functional.scaled_dot_product_attention on CPU (library routine), a pure-Python
      triple loop on tiny shapes, and closed forms (Q = 0 under a causal mask gives prefix
      means of V; window = 1 returns V; a per-row constant bias is a no-op).
  attention backward (autograd of the restatement)
      torch.autograd.gradcheck in fp64 and the identities dV = P^T dO,
      dS = P * (dP - rowsum(dO * O)).
  epilogue.bias_gelu / bias_gelu_back / new_gelu
      torch.nn.functional.gelu(approximate="tanh") (library routine) and fp64 autograd of the
      forward against the literal backward formula.
  epilogue.bias_dropout(_residual)
      identity at p = 0; at p > 0 the explicit-mask semantics of flash_attn_ref
      (masked_fill(~mask, 0) and scaling by 1/(1-p), slapo/op/attention.py:118-125).
  epilogue.bias_dropout_residual_layer_norm(_bwd)
      torch.nn.functional.layer_norm (library routine) and autograd through it, with an eps large
      enough that leaving it out shows; constant rows (exactly ln_bias).
  cross_entropy.forward / backward / shard_stats / combine
      torch.nn.functional.cross_entropy (library routine; its label smoothing equals the
      reference's at alpha K / (K - 1)), autograd, and the identity between the whole-vocabulary
      loss and the loss combined from shard statistics for several cuts.
  philox.philox4x32_10
      the Random123 known-answer vectors for Philox4x32-10.
  philox.aten_dropout_mask (element -> subsequence/counter/lane mapping)
      PARITY UNPINNED on the CPU: the mapping is fixed by ATen's device kernel, whose source is
      not available offline.  It is pinned on the GPU by comparing against the mask that
      torch.nn.functional.dropout itself produces under the same generator state (the
      reference calls exactly that function, slapo/op/fused_bias.py:74, attention.py:180).

Third-party kernels the reference calls on this path (xformers @48a77cc, jfc4050/flash-attention
@3676bd2) are not vendored under the reference tree; their arithmetic is anchored on the
reference's own native restatements named above.
"""
