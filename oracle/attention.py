"""CPU restatement of the reference's native attention path (test infrastructure; see
oracle/__init__.py for what pins it).

Follows slapo/op/attention.py: `attention_bmk` / `xformers_ref` (:134-196), `flash_attn_ref`
(:39-131) and the mask conventions of `FlashAttentionOp.forward` (:305-367).  Two things are
added that the reference gets from elsewhere: the dense form of xformers'
`LowerTriangularMask` (-inf strictly above the diagonal) and the HF GPT-Neo local window
(key j visible to query i iff 0 <= i - j < window).  Dropout takes an explicit boolean keep-mask
(the semantics of flash_attn_ref :118-125), so the same function serves any mask source.
"""
from __future__ import annotations

import math
from typing import Optional

import torch


def visibility(seqlen_q: int, seqlen_k: int, causal: bool, window: int = 0) -> torch.Tensor:
    """Boolean [Sq, Sk]: True where key j may be attended by query i."""
    i = torch.arange(seqlen_q)[:, None]
    j = torch.arange(seqlen_k)[None, :]
    vis = torch.ones(seqlen_q, seqlen_k, dtype=torch.bool)
    if causal:
        vis &= j <= i
    if window and window > 0:
        vis &= (i - j) < window
    return vis


def attention_bmk(q, k, v, attn_bias=None, keep_mask=None, p=0.0, scale=None,
                  compute_dtype=torch.float32):
    """slapo/op/attention.py:163-181 on [B*H, S, D] operands: upcast, scale q, q k^T, + bias,
    softmax, inverted dropout with an explicit keep-mask, @ v."""
    assert q.ndim == 3
    q = q.to(compute_dtype)
    k = k.to(compute_dtype)
    v = v.to(compute_dtype)
    scale = scale if scale is not None else (1 / q.shape[-1] ** 0.5)
    q = q * scale
    attn = q @ k.transpose(-2, -1)
    if attn_bias is not None:
        if attn_bias.ndim == 4:
            attn_bias = attn_bias.reshape([-1, *attn_bias.shape[2:]])
        attn = attn + attn_bias.to(compute_dtype)
    attn = attn.softmax(-1)
    if p > 0:
        assert keep_mask is not None, "dropout needs an explicit keep-mask"
        attn = attn.masked_fill(~keep_mask.reshape(attn.shape), 0.0) * (1.0 / (1.0 - p))
    return attn @ v


def dense_bias(batch, heads, seqlen_q, seqlen_k, attention_mask=None, causal=False, window=0,
               dtype=torch.float32):
    """[B, H, Sq, Sk] additive bias: broadcast HF-style mask + (-inf) where not visible."""
    bias = torch.zeros(batch, heads, seqlen_q, seqlen_k, dtype=dtype)
    if attention_mask is not None:
        bias = bias + attention_mask.to(dtype)
    if causal or (window and window > 0):
        vis = visibility(seqlen_q, seqlen_k, causal, window)
        bias = bias.masked_fill(~vis, float("-inf"))
    return bias


def xformers_ref(q, k, v, attention_mask=None, causal=False, window=0, p=0.0, keep_mask=None,
                 scale=None, compute_dtype=torch.float32):
    """slapo/op/attention.py:183-196 with the bias materialised as FlashAttentionOp.forward
    builds it (:307-311).  q, k, v: [B, S, H, D]; returns [B, Sq, H, D] in compute_dtype."""
    assert q.ndim == 4
    b, sq, h, d = q.shape
    sk = k.shape[1]

    def T(t):
        return t.permute((0, 2, 1, 3)).reshape([t.shape[0] * t.shape[2], t.shape[1], t.shape[3]])

    bias = None
    if attention_mask is not None or causal or (window and window > 0):
        bias = dense_bias(b, h, sq, sk, attention_mask, causal, window, compute_dtype)
        bias = bias.reshape(b * h, sq, sk)
    out = attention_bmk(T(q), T(k), T(v), bias, keep_mask, p, scale, compute_dtype)
    out = out.reshape([b, h, sq, v.shape[3]])
    return out.permute((0, 2, 1, 3))


def flash_attn_ref(q, k, v, bias=None, causal=False, dropout_p=0.0, key_padding_mask=None,
                   dropout_mask=None, compute_dtype=torch.float32):
    """slapo/op/attention.py:97-131: einsum formulation, q pre-divided by sqrt(d), -inf fills
    for key padding and the causal triangle, explicit dropout mask, v scaled by 1/(1-p)."""
    q, k, v = q.to(compute_dtype), k.to(compute_dtype), v.to(compute_dtype)
    seqlen_q, seqlen_k = q.shape[1], k.shape[1]
    d = q.shape[-1]
    scores = torch.einsum("bthd,bshd->bhts", q / math.sqrt(d), k)
    if bias is not None:
        scores = (scores + bias.to(compute_dtype)).to(dtype=scores.dtype)
    if key_padding_mask is not None:
        scores = scores.masked_fill(~key_padding_mask[:, None, None, :], float("-inf"))
    if causal:
        causal_mask = torch.triu(torch.ones(seqlen_q, seqlen_k, dtype=torch.bool), 1)
        scores = scores.masked_fill(causal_mask, float("-inf"))
    attention = torch.softmax(scores, dim=-1)
    dropout_scaling = 1.0 / (1 - dropout_p)
    if dropout_mask is not None:
        attention_drop = attention.masked_fill(~dropout_mask, 0.0)
    else:
        attention_drop = attention
    return torch.einsum("bhts,bshd->bthd", attention_drop, v * dropout_scaling)


def attention_fwd_bwd(q, k, v, dout, attention_mask=None, causal=False, window=0, p=0.0,
                      keep_mask=None, scale=None, compute_dtype=torch.float32):
    """Forward + autograd backward of xformers_ref; returns (out, dq, dk, dv) in compute_dtype."""
    q = q.detach().to(compute_dtype).requires_grad_(True)
    k = k.detach().to(compute_dtype).requires_grad_(True)
    v = v.detach().to(compute_dtype).requires_grad_(True)
    out = xformers_ref(q, k, v, attention_mask, causal, window, p, keep_mask, scale, compute_dtype)
    out.backward(dout.to(compute_dtype))
    return out.detach(), q.grad, k.grad, v.grad


def attended_pairs(seqlen_q: int, seqlen_k: int, causal: bool, window: int = 0,
                   valid_len: Optional[int] = None) -> int:
    """Number of (query, key) pairs with non-masked score for one (batch, head); keys beyond
    valid_len are key-padding.  This is the N of the algorithmic-work formula 14*D*N."""
    vis = visibility(seqlen_q, seqlen_k, causal, window)
    if valid_len is not None:
        vis = vis & (torch.arange(seqlen_k)[None, :] < valid_len)
    return int(vis.sum())
