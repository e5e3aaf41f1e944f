"""Self-attention on a hand-written gfx950 flash-attention kernel.

Interface-compatible with the reference's slapo/op/attention.py: `FlashAttentionOp`
(:245-367) and `FlashAttention` (:370-522) keep their constructor and forward signatures,
attribute names and child-module names, so schedules that build them and address
`module.qkv`, `module.out_proj`, `module.attn_op` keep working.  The kernel registry gains one
name, "hip_cdna4", which takes the place of every third-party choice:

    "hip_cdna4", "auto"                     -> the HIP kernel
    "cutlass", "flash", "triton", "cuda",   -> accepted as aliases of "hip_cdna4" (one warning);
    "small_k"                                  the reference's schedules fall back to "cutlass"
                                               when a constructor fails (model_schedule/gpt2.py:229-239)
    "native_xformers", "native_flash_attn"  -> ValueError: the native PyTorch restatements are
                                               test oracles, not part of this package

The op reads an additive mask in the compact [B,1,1,Sk] layout (`bias_layout == "b11k"`, no
[B,H,S,S] expansion), broadcasts it in-kernel, applies the causal triangle (and an optional
local window) by index arithmetic, and draws its dropout mask from the device's default
generator -- the mask torch.nn.functional.dropout would draw for the dense [B*H,Sq,Sk]
probability tensor in `xformers_ref` (:178-181).
"""
from __future__ import annotations

import logging
from typing import Optional

import torch
import torch.nn.functional as F
from torch import nn

from ..random import draw_philox  # noqa: F401  (kept importable from here for direct launches)
from ..random import draw_philox_state
from . import _kernels as K
from .fused_bias import bias_dropout

logger = logging.getLogger("slapo_amd")

ATTN_GLOBAL_MSGS = set()

HIP_OP_NAMES = ("hip_cdna4", "auto")
ALIASED_OP_NAMES = ("cutlass", "flash", "triton", "cuda", "small_k")
ORACLE_OP_NAMES = ("native_xformers", "native_flash_attn")


def warning_once(msg):
    if msg not in ATTN_GLOBAL_MSGS:
        logger.warning(msg)
        ATTN_GLOBAL_MSGS.add(msg)


# With dropout, the forward hands the keep bits (1 bit per score) to the backward, which then reads
# them instead of regenerating every Philox block in both of its kernels.  Same gradients, bit
# for bit; False trades the buffer (B*H*Sq*Sk/8 bytes) for the regeneration.
SAVE_DROPOUT_MASK = True
# ... up to this size per call; beyond it (long sequences: the bits grow with Sq * Sk) the backward
# regenerates the mask and nothing of that size is kept between the passes.
SAVE_DROPOUT_MASK_MAX_BYTES = 512 << 20


class _HipAttention(torch.autograd.Function):
    """Forward saves (q, k, v, bias, out, lse), the Philox (seed, offset) and, with dropout, the
    keep bits; backward recomputes the probabilities from lse and reads (or regenerates) the
    dropout mask -- it never draws."""

    # pylint: disable=arguments-differ, abstract-method
    @staticmethod
    def forward(ctx, q, k, v, bias, causal, window, scale, p):
        b, sq, h, _ = q.shape
        sk = k.shape[1]
        plan, seed, offset, rng_state = None, 0, 0, None
        if b * h * sq * sk == 0:
            p = 0.0  # nothing to drop, and F.dropout leaves the generator alone for an empty tensor
        if p > 0.0:
            plan = K.dropout_plan(b * h * sq * sk, 4, q.device)
            if p < 1.0:
                seed, offset, rng_state = draw_philox_state(plan.offset_increment, q.device)
        save_mask = SAVE_DROPOUT_MASK and 0.0 < p < 1.0 and any(ctx.needs_input_grad[:3])
        if save_mask:
            mask_bytes = b * h * ((sk + 31) // 32) * ((sq + 3) // 4 * 4) * 4
            save_mask = mask_bytes <= SAVE_DROPOUT_MASK_MAX_BYTES
        out, lse, (q, k, v), keep_mask = K.attn_fwd(q, k, v, bias, causal, window, scale, p, seed,
                                                    offset, plan, save_mask=save_mask,
                                                    rng_state=rng_state)
        ctx.save_for_backward(q, k, v, bias, out, lse, keep_mask, rng_state)
        ctx.cfg = (causal, window, scale, p, seed, offset, plan)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, bias, out, lse, keep_mask, rng_state = ctx.saved_tensors
        causal, window, scale, p, seed, offset, plan = ctx.cfg
        dq, dk, dv = K.attn_bwd(dout, q, k, v, bias, out, lse, causal, window, scale, p, seed,
                                offset, plan, keep_mask, rng_state)
        return dq, dk, dv, None, None, None, None, None


def hip_attention(q, k, v, attention_mask=None, causal=False, p=0.0, scale=None, window=0):
    """q, k, v: [B, S, H, D] (head_dim contiguous; outer dims may be strided views).
    attention_mask: additive, 4-D, broadcastable to [B, H, Sq, Sk].  Returns [B, Sq, H, D]."""
    if q.ndim != 4 or k.ndim != 4 or v.ndim != 4:
        raise ValueError("q, k, v must be [batch, seqlen, heads, head_dim]")
    if k.shape != v.shape or q.shape[0] != k.shape[0] or q.shape[2:] != k.shape[2:]:
        raise ValueError(f"inconsistent q/k/v shapes {tuple(q.shape)} {tuple(k.shape)} "
                         f"{tuple(v.shape)}")
    if not (q.dtype == k.dtype == v.dtype):
        raise ValueError("q, k, v must share a dtype")
    if p < 0.0 or p > 1.0:
        raise ValueError(f"dropout probability has to be between 0 and 1, but got {p}")
    b, sq, h, d = q.shape
    bias = None
    if attention_mask is not None:
        if attention_mask.requires_grad:
            warning_once("WARNING: bias gradient is not supported yet. "
                         "The mask is applied but receives no gradient")
        bias = K.prepare_bias(attention_mask.detach(), b, h, sq, k.shape[1])
    scale = float(scale) if scale is not None else float(d) ** -0.5
    return _HipAttention.apply(q, k, v, bias, bool(causal), int(window or 0), scale, float(p))


class FlashAttentionOp(nn.Module):
    """Core attention: softmax(Q K^T * scale + mask) V with dropout on the probabilities.

    Parameters
    ----------
    attn_op_name : str
        "hip_cdna4" (or "auto"); the third-party names of the reference are aliases.
    apply_causal_mask : bool
        Restrict query i to keys j <= i.
    scale : Optional[float]
        Softmax scale; None means head_dim ** -0.5.
    window : Optional[int]
        Not in the reference: local causal attention (HF GPT-Neo), key j is visible to query i
        only if i - j < window.  None / 0 disables it.
    """

    def __init__(self, attn_op_name, apply_causal_mask, scale=None, window=None):
        super().__init__()
        if attn_op_name in ORACLE_OP_NAMES:
            raise ValueError(
                f"attn_op_name '{attn_op_name}' names a native PyTorch restatement, which this "
                "package keeps only as a test oracle; use 'hip_cdna4'"
            )
        if attn_op_name in ALIASED_OP_NAMES:
            warning_once(f"attn_op_name '{attn_op_name}' is served by the 'hip_cdna4' kernel")
        elif attn_op_name not in HIP_OP_NAMES:
            raise ValueError(f"Unknown attention op name: {attn_op_name}")
        if window is not None and window < 0:
            raise ValueError("window must be positive")
        self.attn_op_name = attn_op_name
        self.apply_causal_mask = apply_causal_mask
        self.scale = scale
        self.window = window
        self.pkg = "hip"
        self.attn_fn = hip_attention
        # The kernel broadcasts a [B,1,1,Sk] mask itself.
        self.bias_layout = "b11k"

    def forward(self, query_layer, key_layer, value_layer, attention_mask, p):
        ret = self.attn_fn(query_layer, key_layer, value_layer, attention_mask,
                           causal=self.apply_causal_mask, p=p, scale=self.scale,
                           window=self.window or 0)
        return ret.to(query_layer.dtype)

    def extra_repr(self):
        return (f"attn_op_name={self.attn_op_name}, causal={self.apply_causal_mask}, "
                f"scale={self.scale}, window={self.window}")


def _has_hooks(module):
    """True if any per-module or global forward / backward hook would run on `module(...)`."""
    # pylint: disable=protected-access
    from torch.nn.modules import module as M
    return bool(module._forward_hooks or module._forward_pre_hooks or module._backward_hooks
                or module._backward_pre_hooks or M._global_forward_hooks
                or M._global_forward_pre_hooks or M._global_backward_hooks
                or M._global_backward_pre_hooks)


class FlashAttention(nn.Module):
    """HF-style self-attention block: QKV projection(s) -> FlashAttentionOp -> optional output
    projection + residual dropout.  Restrictions are the reference's: no cross attention, no
    head mask, no attention-probability output (NotImplementedError)."""

    def __init__(self, hidden_size, num_attention_heads, attn_pdrop=0.0, resid_pdrop=0.0,
                 attn_op_name="auto", bias=True, output_proj=True, fused_qkv=False,
                 window=None):
        super().__init__()
        if hidden_size % num_attention_heads != 0:
            raise ValueError(
                f"The hidden size ({hidden_size}) is not a multiple "
                f"of the number of attention heads ({num_attention_heads})"
            )
        self.hidden_size = hidden_size
        self.num_attention_heads = num_attention_heads
        self.attention_head_size = hidden_size // num_attention_heads
        self.all_head_size = self.num_attention_heads * self.attention_head_size

        self.fused_qkv = fused_qkv
        if fused_qkv:
            self.qkv = nn.Linear(hidden_size, 3 * self.all_head_size, bias=bias)
        else:
            self.query = nn.Linear(hidden_size, self.all_head_size, bias=bias)
            self.key = nn.Linear(hidden_size, self.all_head_size, bias=bias)
            self.value = nn.Linear(hidden_size, self.all_head_size, bias=bias)

        self.output_proj = output_proj
        self.attn_pdrop = attn_pdrop
        if output_proj:
            self.out_proj = nn.Linear(hidden_size, hidden_size, bias=bias)
            self.resid_dropout = nn.Dropout(resid_pdrop)

        self.attn_op_name = attn_op_name
        # Causality follows output_proj, as in the reference (attention.py:428): encoder models
        # (BERT) are built with output_proj=False, decoder models with True.
        self.attn_op = FlashAttentionOp(attn_op_name, self.output_proj, window=window)
        self.bias_layout = self.attn_op.bias_layout

    @staticmethod
    def layout_attention_mask(mask, num_attention_heads):
        """(B,1,1,S) -> dense (B,H,S,S); only needed by ops whose bias_layout is "bhqk"."""
        return mask.expand(-1, num_attention_heads, mask.shape[-1], -1).contiguous()

    def reshape_for_scores(self, x: torch.Tensor):
        """[B, S, heads*head_size] -> [B, S, heads, head_size]; -1 covers sharded head counts."""
        return x.view(x.size()[:-1] + (-1, self.attention_head_size))

    def _project_qkv(self, hidden_states):
        if self.fused_qkv:
            # Head-interleaved packing [.., heads, 3*head_size]: q, k, v of one head are adjacent,
            # which keeps a tensor-parallel shard of the weight a set of whole heads.  The three
            # results are strided views; the kernel reads them in place.
            packed = self.qkv(hidden_states)
            packed = packed.view(packed.size()[:-1] + (-1, 3 * self.attention_head_size))
            return packed.split(self.attention_head_size, dim=-1)
        return tuple(self.reshape_for_scores(proj(hidden_states))
                     for proj in (self.query, self.key, self.value))

    def _tail_can_fuse(self, x):
        """The fused out_proj-bias + resid_dropout pass stands in for the two child calls only when
        nothing could tell the difference: both children are the plain torch modules, carry no
        hooks (a schedule's `.sync(mode="fwd_post")` is a forward hook on `out_proj`,
        slapo/sharding/shard_ops.py:436-440; `.replace` moves hooks along, primitives/replace.py:254),
        and the input is a real device tensor (not an fx Proxy during tracing)."""
        proj, drop = self.out_proj, self.resid_dropout
        return (type(x) is torch.Tensor and x.is_cuda
                and type(proj) is nn.Linear and proj.bias is not None
                and type(drop) is nn.Dropout and not drop.inplace
                and not _has_hooks(proj) and not _has_hooks(drop))

    def forward(
        self,
        hidden_states: Optional[tuple[torch.FloatTensor]],
        attention_mask: Optional[torch.FloatTensor] = None,
        layer_past: Optional[tuple[torch.Tensor]] = None,
        head_mask: Optional[torch.FloatTensor] = None,
        encoder_hidden_states: Optional[torch.Tensor] = None,
        encoder_attention_mask: Optional[torch.FloatTensor] = None,
        use_cache: Optional[bool] = False,
        output_attentions: Optional[bool] = False,
    ) -> tuple[torch.Tensor]:
        if encoder_hidden_states is not None or encoder_attention_mask is not None:
            raise NotImplementedError("FlashAttention does not support cross attention yet.")
        if output_attentions:
            raise NotImplementedError("FlashAttention does not support output attention yet.")
        if head_mask is not None:
            raise NotImplementedError("FlashAttention does not support head mask yet.")

        query_layer, key_layer, value_layer = self._project_qkv(hidden_states)

        if layer_past is not None:
            past_key, past_value = layer_past
            key_layer = torch.cat((past_key, key_layer), dim=-2)
            value_layer = torch.cat((past_value, value_layer), dim=-2)

        if attention_mask is not None and self.bias_layout == "bhqk":
            attention_mask = self.layout_attention_mask(attention_mask, self.num_attention_heads)

        context_layer = self.attn_op(query_layer, key_layer, value_layer, attention_mask,
                                     p=self.attn_pdrop)
        context_layer = context_layer.contiguous()
        context_layer = context_layer.view(context_layer.size()[:-2] + (-1,))

        if self.output_proj:
            if self._tail_can_fuse(context_layer):
                # out_proj's bias and resid_dropout ride on one pass over [B, S, hidden] (the
                # reference runs the GEMM with bias, then nn.Dropout: slapo/op/attention.py:514-516).
                # The mask is the one nn.Dropout would draw; p and training are read from the child.
                context_layer = bias_dropout(
                    F.linear(context_layer, self.out_proj.weight, None), self.out_proj.bias,
                    self.resid_dropout.p, self.resid_dropout.training)
            else:
                context_layer = self.resid_dropout(self.out_proj(context_layer))

        return (context_layer, (key_layer, value_layer) if use_cache else None)
