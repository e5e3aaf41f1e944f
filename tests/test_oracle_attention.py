"""Pins for oracle/attention.py (CPU only): library routine, brute force, closed forms,
gradcheck and the backward identities."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import attention as OA


def _qkv(b, s, h, d, sk=None, dtype=torch.float64, seed=0):
    g = torch.Generator().manual_seed(seed)
    sk = sk or s
    return (torch.randn(b, s, h, d, generator=g, dtype=dtype),
            torch.randn(b, sk, h, d, generator=g, dtype=dtype),
            torch.randn(b, sk, h, d, generator=g, dtype=dtype))


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("with_mask", [False, True])
def test_matches_library_sdpa(causal, with_mask):
    b, s, h, d = 2, 33, 3, 16
    q, k, v = _qkv(b, s, h, d)
    mask = torch.randn(b, 1, 1, s, dtype=torch.float64) if with_mask else None
    out = OA.xformers_ref(q, k, v, mask, causal, compute_dtype=torch.float64)
    attn_mask = None
    if with_mask or causal:
        attn_mask = torch.zeros(b, h, s, s, dtype=torch.float64)
        if with_mask:
            attn_mask = attn_mask + mask
        if causal:
            attn_mask = attn_mask.masked_fill(~torch.ones(s, s, dtype=torch.bool).tril(), -math.inf)
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2),
                                         attn_mask=attn_mask).transpose(1, 2)
    torch.testing.assert_close(out, ref, atol=1e-12, rtol=1e-10)


def test_matches_brute_force_loops_with_window_padding_and_dropout():
    b, s, h, d, window, p = 2, 9, 2, 4, 3, 0.25
    q, k, v = _qkv(b, s, h, d, seed=1)
    lens = [8, 9]  # every query keeps at least one visible key
    mask = torch.zeros(b, 1, 1, s, dtype=torch.float64)
    for bi, L in enumerate(lens):
        mask[bi, 0, 0, L:] = -math.inf
    keep = torch.rand(b * h, s, s, generator=torch.Generator().manual_seed(2)) > p
    out = OA.xformers_ref(q, k, v, mask, True, window, p, keep, None, torch.float64)
    for bi in range(b):
        for hi in range(h):
            for i in range(s):
                scores = []
                for j in range(s):
                    ok = j <= i and i - j < window and j < lens[bi]
                    scores.append(sum(q[bi, i, hi, t] * k[bi, j, hi, t] for t in range(d)).item()
                                  / math.sqrt(d) if ok else -math.inf)
                mx = max(scores)
                w = [math.exp(x - mx) for x in scores]
                z = sum(w)
                for t in range(d):
                    acc = sum((w[j] / z) * (1 / (1 - p) if keep[bi * h + hi, i, j] else 0.0)
                              * v[bi, j, hi, t].item() for j in range(s))
                    assert abs(out[bi, i, hi, t].item() - acc) < 1e-12


def test_flash_attn_ref_and_xformers_ref_agree():
    b, s, h, d = 2, 17, 2, 8
    q, k, v = _qkv(b, s, h, d, seed=3)
    lens = torch.tensor([11, 17])
    kpm = torch.arange(s)[None, :] < lens[:, None]
    bias = torch.zeros(b, 1, 1, s, dtype=torch.float64).masked_fill(~kpm[:, None, None, :], -math.inf)
    a = OA.flash_attn_ref(q, k, v, None, True, key_padding_mask=kpm, compute_dtype=torch.float64)
    x = OA.xformers_ref(q, k, v, bias, True, compute_dtype=torch.float64)
    torch.testing.assert_close(a, x, atol=1e-12, rtol=1e-10)


def test_closed_forms():
    b, s, h, d = 1, 12, 2, 4
    q, k, v = _qkv(b, s, h, d, seed=4)
    # Q = 0 under a causal mask: uniform weights over the visible prefix -> prefix means of V
    out = OA.xformers_ref(torch.zeros_like(q), k, v, None, True, compute_dtype=torch.float64)
    prefix_mean = v.cumsum(1) / torch.arange(1, s + 1, dtype=torch.float64)[None, :, None, None]
    torch.testing.assert_close(out, prefix_mean, atol=1e-12, rtol=1e-10)
    # window = 1: each query sees only itself -> V
    out = OA.xformers_ref(q, k, v, None, True, window=1, compute_dtype=torch.float64)
    torch.testing.assert_close(out, v, atol=1e-12, rtol=1e-10)
    # window >= S is plain causal; a bias constant along keys is a no-op
    base = OA.xformers_ref(q, k, v, None, True, compute_dtype=torch.float64)
    torch.testing.assert_close(OA.xformers_ref(q, k, v, None, True, window=s,
                                               compute_dtype=torch.float64), base)
    row_const = torch.randn(b, h, s, 1, dtype=torch.float64).expand(b, h, s, s)
    torch.testing.assert_close(OA.xformers_ref(q, k, v, row_const, True,
                                               compute_dtype=torch.float64), base,
                               atol=1e-12, rtol=1e-10)
    # permuting keys and values together leaves unmasked attention unchanged
    perm = torch.randperm(s, generator=torch.Generator().manual_seed(5))
    full = OA.xformers_ref(q, k, v, None, False, compute_dtype=torch.float64)
    torch.testing.assert_close(OA.xformers_ref(q, k[:, perm], v[:, perm], None, False,
                                               compute_dtype=torch.float64), full,
                               atol=1e-12, rtol=1e-10)


def test_gradcheck_and_backward_identities():
    b, s, h, d, p = 1, 6, 2, 3, 0.3
    q, k, v = _qkv(b, s, h, d, seed=6)
    keep = torch.rand(b * h, s, s, generator=torch.Generator().manual_seed(7)) > p
    fn = lambda q_, k_, v_: OA.xformers_ref(q_, k_, v_, None, True, 0, p, keep, None, torch.float64)
    assert torch.autograd.gradcheck(fn, [t.clone().requires_grad_(True) for t in (q, k, v)])
    dout = torch.randn(b, s, h, d, dtype=torch.float64, generator=torch.Generator().manual_seed(8))
    out, dq, dk, dv = OA.attention_fwd_bwd(q, k, v, dout, None, True, 0, p, keep, None, torch.float64)
    # closed-form backward: dV = Pd^T dO, dS = P * (dPd*M/(1-p) - rowsum(dO * O)), dQ = dS K / sqrt(d)
    scale = d ** -0.5
    qh, kh, vh, gh, oh = (t.permute(0, 2, 1, 3).reshape(b * h, s, d) for t in (q, k, v, dout, out))
    sc = (qh * scale) @ kh.transpose(1, 2)
    sc = sc.masked_fill(~OA.visibility(s, s, True), -math.inf)
    pr = sc.softmax(-1)
    m = keep.double() / (1 - p)
    dv_ref = (pr * m).transpose(1, 2) @ gh
    dp = (gh @ vh.transpose(1, 2)) * m
    delta = (gh * oh).sum(-1, keepdim=True)
    ds = pr * (dp - delta)
    back = lambda t: t.reshape(b, h, s, d).permute(0, 2, 1, 3)
    torch.testing.assert_close(dv, back(dv_ref), atol=1e-12, rtol=1e-10)
    torch.testing.assert_close(dq, back(ds @ kh * scale), atol=1e-12, rtol=1e-10)
    torch.testing.assert_close(dk, back(ds.transpose(1, 2) @ qh * scale), atol=1e-12, rtol=1e-10)


def test_attended_pairs_formulas():
    s = 64
    assert OA.attended_pairs(s, s, False) == s * s
    assert OA.attended_pairs(s, s, True) == s * (s + 1) // 2
    w = 10
    assert OA.attended_pairs(s, s, True, w) == w * (w + 1) // 2 + (s - w) * w
    L = 40
    assert OA.attended_pairs(s, s, True, 0, L) == L * (L + 1) // 2 + (s - L) * L
    # the GPT-2-medium benchmark shape: 524800 pairs per head at S = 1024
    assert OA.attended_pairs(1024, 1024, True) == 524800
