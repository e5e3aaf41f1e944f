"""Tensor-level wrappers over the C ABI: argument checking, output/workspace allocation with
torch's caching allocator, stream selection.  No arithmetic happens here."""
from __future__ import annotations

import ctypes
import functools

import torch

from .. import _lib
from .._lib import AttnParams, DropoutPlan


def _require_device(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "slapo_amd kernels run on a gfx950 device only; got a tensor on "
                f"'{t.device}'.  There is no CPU implementation in this package."
            )


# The wrappers below sit on the critical path of every training step, so the per-call host work
# is kept small: raw stream and data pointers as plain integers (ctypes converts them through the
# declared argtypes), a device switch only when the tensor lives on another device than the
# current one, and parameter structs cached per problem geometry.
def _stream():
    return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device())


def _ptr(t):
    return t.data_ptr() if t is not None else None


class _on:
    """`with _on(device):` -- like torch.cuda.device(device), without the cost when the device
    is already current."""

    __slots__ = ("idx", "prev")

    def __init__(self, device):
        self.idx = torch.device(device).index
        self.prev = -1

    def __enter__(self):
        if self.idx is not None:
            cur = torch.cuda.current_device()
            if cur != self.idx:
                self.prev = cur
                torch.cuda.set_device(self.idx)
        return self

    def __exit__(self, *exc):
        if self.prev >= 0:
            torch.cuda.set_device(self.prev)
        return False


@functools.lru_cache(maxsize=4096)
def _plan_cached(numel: int, elem_bytes: int, device_index: int):
    plan = DropoutPlan()
    rc = _lib.load().slapo_amd_dropout_plan(numel, elem_bytes, 256, device_index,
                                            ctypes.byref(plan))
    _lib.check(rc, "slapo_amd_dropout_plan")
    return plan


def dropout_plan(numel: int, elem_bytes: int, device) -> DropoutPlan:
    """Launch plan torch.nn.functional.dropout would use for a fresh dense tensor."""
    idx = torch.device(device).index
    if idx is None:
        idx = torch.cuda.current_device()
    return _plan_cached(int(numel), int(elem_bytes), int(idx))


def _plan_ref(plan, rng_state=None):
    """The plan as a call argument.  `rng_state` (a device tensor of two 64-bit integers, {seed,
    offset}) makes the kernels read the pair from device memory when they run -- what a captured
    graph needs -- instead of taking the call's seed / offset values."""
    if plan is None:
        return None
    if rng_state is None:
        return ctypes.byref(plan)
    if (rng_state.dtype not in (torch.int64, torch.uint64) or rng_state.numel() != 2
            or not rng_state.is_cuda or not rng_state.is_contiguous()):
        raise ValueError("rng_state must be a contiguous device tensor of two 64-bit integers")
    own = DropoutPlan.from_buffer_copy(plan)
    own.rng_state = rng_state.data_ptr()
    return ctypes.byref(own)


def _rows_cols(x, bias):
    cols = x.shape[-1]
    if bias.ndim != 1 or bias.shape[0] != cols:
        raise ValueError(f"bias must have shape [{cols}], got {tuple(bias.shape)}")
    return x.numel() // cols, cols


def _same_dtype(x, *others):
    return [o if o is None or o.dtype == x.dtype else o.to(x.dtype) for o in others]


def bias_gelu_fwd(y, bias):
    _require_device(y, bias)
    y = y.contiguous()
    (bias,) = _same_dtype(y, bias.contiguous())
    rows, cols = _rows_cols(y, bias)
    out = torch.empty_like(y)
    if y.numel() == 0:
        return out
    with _on(y.device):
        rc = _lib.load().slapo_amd_bias_gelu_fwd(_ptr(y), _ptr(bias), _ptr(out), rows, cols,
                                                 _lib.dtype_code(y.dtype), _stream())
    _lib.check(rc, "slapo_amd_bias_gelu_fwd")
    return out


def _colsum_ws(rows, cols, device):
    nbytes = _lib.load().slapo_amd_colsum_workspace_bytes(rows, cols)
    return torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device=device), nbytes


def bias_gelu_bwd(grad, y, bias, need_dbias=True):
    _require_device(grad, y, bias)
    y = y.contiguous()
    grad, bias = _same_dtype(y, grad.contiguous(), bias.contiguous())
    rows, cols = _rows_cols(y, bias)
    dx = torch.empty_like(y)
    dbias = torch.empty_like(bias) if need_dbias else None
    if y.numel() == 0:
        return dx, (dbias.zero_() if dbias is not None else None)
    with _on(y.device):
        ws, nbytes = _colsum_ws(rows, cols, y.device) if need_dbias else (None, 0)
        rc = _lib.load().slapo_amd_bias_gelu_bwd(_ptr(grad), _ptr(y), _ptr(bias), _ptr(dx),
                                                 _ptr(dbias), _ptr(ws), nbytes, rows, cols,
                                                 _lib.dtype_code(y.dtype), _stream())
    _lib.check(rc, "slapo_amd_bias_gelu_bwd")
    return dx, dbias


def bias_dropout_residual_fwd(x, bias, residual, p, seed, offset, plan, rng_state=None):
    _require_device(x, bias, residual)
    x = x.contiguous()
    bias, residual = _same_dtype(x, bias.contiguous(),
                                 residual.contiguous() if residual is not None else None)
    if residual is not None and residual.shape != x.shape:
        raise ValueError("residual must have the shape of x")
    rows, cols = _rows_cols(x, bias)
    out = torch.empty_like(x)
    if x.numel() == 0:
        return out
    with _on(x.device):
        rc = _lib.load().slapo_amd_bias_dropout_residual_fwd(
            _ptr(x), _ptr(bias), _ptr(residual), _ptr(out), rows, cols,
            _lib.dtype_code(x.dtype), float(p), seed, offset,
            _plan_ref(plan, rng_state), _stream())
    _lib.check(rc, "slapo_amd_bias_dropout_residual_fwd")
    return out


def bias_dropout_residual_bwd(grad, bias_like, p, seed, offset, plan, need_dx=True,
                              need_dbias=True, rng_state=None):
    _require_device(grad)
    grad = grad.contiguous()
    cols = grad.shape[-1]
    rows = grad.numel() // cols
    dx = torch.empty_like(grad) if need_dx else None
    dbias = torch.empty(cols, dtype=grad.dtype, device=grad.device) if need_dbias else None
    if grad.numel() == 0 or not (need_dx or need_dbias):
        return dx, (dbias.zero_() if dbias is not None else None)
    with _on(grad.device):
        ws, nbytes = _colsum_ws(rows, cols, grad.device) if need_dbias else (None, 0)
        rc = _lib.load().slapo_amd_bias_dropout_residual_bwd(
            _ptr(grad), _ptr(dx), _ptr(dbias), _ptr(ws), nbytes, rows, cols,
            _lib.dtype_code(grad.dtype), float(p), seed, offset,
            _plan_ref(plan, rng_state), _stream())
    _lib.check(rc, "slapo_amd_bias_dropout_residual_bwd")
    if dbias is not None and dbias.dtype != bias_like.dtype:
        dbias = dbias.to(bias_like.dtype)
    return dx, dbias


def bias_dropout_residual_ln_fwd(x, bias, residual, weight, ln_bias, eps, p, seed, offset, plan,
                                 save_for_backward=True, rng_state=None):
    """Returns (y, z, mean, rstd); the last three are None without save_for_backward."""
    _require_device(x, bias, residual, weight, ln_bias)
    x = x.contiguous()
    bias, residual, weight, ln_bias = _same_dtype(
        x, bias.contiguous() if bias is not None else None,
        residual.contiguous() if residual is not None else None, weight.contiguous(),
        ln_bias.contiguous())
    if residual is not None and residual.shape != x.shape:
        raise ValueError("residual must have the shape of x")
    cols = x.shape[-1]
    if weight.shape != (cols,) or ln_bias.shape != (cols,) or (
            bias is not None and bias.shape != (cols,)):
        raise ValueError("bias, weight and ln_bias must be 1-D of the last dimension of x")
    rows = x.numel() // max(cols, 1)
    y = torch.empty_like(x)
    z = mean = rstd = None
    if save_for_backward:
        z = torch.empty_like(x)
        mean = torch.empty(rows, dtype=torch.float32, device=x.device)
        rstd = torch.empty(rows, dtype=torch.float32, device=x.device)
    if x.numel() == 0:
        return y, z, mean, rstd
    with _on(x.device):
        rc = _lib.load().slapo_amd_bias_dropout_residual_ln_fwd(
            _ptr(x), _ptr(bias), _ptr(residual), _ptr(weight), _ptr(ln_bias), _ptr(z), _ptr(y),
            _ptr(mean), _ptr(rstd), rows, cols, _lib.dtype_code(x.dtype), float(eps), float(p),
            seed, offset, _plan_ref(plan, rng_state), _stream())
    _lib.check(rc, "slapo_amd_bias_dropout_residual_ln_fwd")
    return y, z, mean, rstd


def bias_dropout_residual_ln_bwd(grad, z, mean, rstd, weight, p, seed, offset, plan, need_dx=True,
                                 need_dres=True, need_dweight=True, need_dln_bias=True,
                                 need_dbias=True, rng_state=None):
    """Returns (dx, dresidual, dweight, dln_bias, dbias); entries not asked for are None."""
    _require_device(grad, z, mean, rstd, weight)
    grad = grad.contiguous()
    (weight,) = _same_dtype(z, weight.contiguous())
    cols = z.shape[-1]
    rows = z.numel() // max(cols, 1)
    vec = lambda need: torch.empty(cols, dtype=z.dtype, device=z.device) if need else None
    dx = torch.empty_like(z) if need_dx else None
    dres = torch.empty_like(z) if need_dres else None
    dw, dlb, db = vec(need_dweight), vec(need_dln_bias), vec(need_dbias)
    outs = (dx, dres, dw, dlb, db)
    if z.numel() == 0 or all(o is None for o in outs):
        for o in (dw, dlb, db):
            if o is not None:
                o.zero_()
        return outs
    lib = _lib.load()
    with _on(z.device):
        ws, nbytes = None, 0
        if need_dweight or need_dln_bias or need_dbias:
            nbytes = lib.slapo_amd_ln_bwd_workspace_bytes(rows, cols)
            ws = torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device=z.device)
        rc = lib.slapo_amd_bias_dropout_residual_ln_bwd(
            _ptr(grad), _ptr(z), _ptr(mean), _ptr(rstd), _ptr(weight), _ptr(dx), _ptr(dres),
            _ptr(dw), _ptr(dlb), _ptr(db), _ptr(ws), nbytes, rows, cols,
            _lib.dtype_code(z.dtype), float(p), seed, offset,
            _plan_ref(plan, rng_state), _stream())
    _lib.check(rc, "slapo_amd_bias_dropout_residual_ln_bwd")
    return outs


def vocab_ce_fwd(logits, target, vocab_start=0):
    """Per-row (row_max, sum_exp, predicted, sum_logits) of one vocabulary shard, fp32 [rows]."""
    _require_device(logits, target)
    logits = logits.contiguous()
    vocab = logits.shape[-1]
    rows = logits.numel() // max(vocab, 1)
    target = target.contiguous().view(-1).to(torch.int64)
    if target.numel() != rows:
        raise ValueError("target must have the shape of the logits without the vocabulary dim")
    stats = torch.empty(4, max(rows, 1), dtype=torch.float32, device=logits.device)
    if rows:
        with _on(logits.device):
            rc = _lib.load().slapo_amd_vocab_ce_fwd(
                _ptr(logits), _ptr(target), _ptr(stats[0]), _ptr(stats[1]), _ptr(stats[2]),
                _ptr(stats[3]), rows, vocab, int(vocab_start), _lib.dtype_code(logits.dtype),
                _stream())
        _lib.check(rc, "slapo_amd_vocab_ce_fwd")
    return stats[0, :rows], stats[1, :rows], stats[2, :rows], stats[3, :rows], logits, target


def vocab_ce_bwd(logits, target, row_max, inv_sum_exp, grad_loss, vocab_start=0,
                 label_smoothing=0.0):
    _require_device(logits, target, row_max, inv_sum_exp, grad_loss)
    vocab = logits.shape[-1]
    rows = logits.numel() // max(vocab, 1)
    grad = torch.empty_like(logits)
    grad_loss = grad_loss.contiguous().view(-1).float()
    if rows:
        with _on(logits.device):
            rc = _lib.load().slapo_amd_vocab_ce_bwd(
                _ptr(logits), _ptr(target), _ptr(row_max.contiguous()),
                _ptr(inv_sum_exp.contiguous()), _ptr(grad_loss), _ptr(grad), rows, vocab,
                int(vocab_start), float(label_smoothing), _lib.dtype_code(logits.dtype),
                _stream())
        _lib.check(rc, "slapo_amd_vocab_ce_bwd")
    return grad


def dropout_mask(numel, elem_bytes, p, seed, offset, device, rng_state=None):
    """Boolean keep-mask [numel] drawn on the device (debugging / test aid)."""
    plan = dropout_plan(numel, elem_bytes, device)
    mask = torch.empty(numel, dtype=torch.uint8, device=device)
    with _on(device):
        rc = _lib.load().slapo_amd_dropout_mask(_ptr(mask), _plan_ref(plan, rng_state), float(p),
                                                seed, offset, _stream())
    _lib.check(rc, "slapo_amd_dropout_mask")
    return mask.bool()


# ------------------------------------------------------------------------------------------
# attention
# ------------------------------------------------------------------------------------------
@functools.lru_cache(maxsize=1024)
def _stride_array(s0, s1, s2):
    return (ctypes.c_int64 * 3)(s0, s1, s2)


def _bshd_strides(t):
    if t.ndim != 4:
        raise ValueError("attention operands must be [batch, seqlen, heads, head_dim]")
    st = t.stride()
    if t.shape[-1] > 1 and st[3] != 1:
        raise ValueError("head_dim must be contiguous")
    return _stride_array(st[0], st[1], st[2])


def _usable_layout(t):
    """Strided [B,S,H,D] views are consumed as they are when rows stay 16-byte aligned."""
    if t.stride(-1) != 1 and t.shape[-1] > 1:
        return t.contiguous()
    esz = t.element_size()
    if (t.data_ptr() % 16) or any((s * esz) % 16 for s in t.stride()[:3]):
        return t.contiguous()
    return t


_PARAMS_CACHE = {}


def make_attn_params(q, k, v, o, bias, causal, window, scale, p, seed, offset, plan,
                     keep_mask=None, rng_state=None):
    """The parameter struct of one attention call.  Everything but (seed, offset, keep_mask) is a
    function of the problem geometry and is cached."""
    key = (q.dtype, q.shape, k.shape[1], q.stride(), k.stride(), v.stride(), o.stride(),
           bias.stride() if bias is not None else None, bool(causal), int(window or 0),
           float(scale), float(p), id(plan))
    entry = _PARAMS_CACHE.get(key)
    if entry is None:
        prm = AttnParams()
        b, sq, h, d = q.shape
        prm.dtype = _lib.dtype_code(q.dtype)
        prm.batch, prm.heads, prm.seqlen_q, prm.seqlen_k, prm.head_dim = b, h, sq, k.shape[1], d
        prm.causal = 1 if causal else 0
        prm.window = int(window) if window else 0
        prm.scale = float(scale)
        prm.p_drop = float(p)
        prm.q_strides = _bshd_strides(q)
        prm.k_strides = _bshd_strides(k)
        prm.v_strides = _bshd_strides(v)
        prm.o_strides = _bshd_strides(o)
        if bias is not None:
            prm.bias_strides = (ctypes.c_int64 * 4)(*bias.stride())
        if plan is not None:
            prm.plan = plan
        if len(_PARAMS_CACHE) >= 1024:
            _PARAMS_CACHE.clear()
        # the plan object is kept alive with the entry, so that its id stays unique
        entry = _PARAMS_CACHE[key] = (prm, plan)
    prm = AttnParams.from_buffer_copy(entry[0])
    prm.seed = int(seed)
    prm.offset = int(offset)
    if keep_mask is not None:
        prm.keep_mask = keep_mask.data_ptr()
    if rng_state is not None:
        if (rng_state.dtype not in (torch.int64, torch.uint64) or rng_state.numel() != 2
                or not rng_state.is_cuda or not rng_state.is_contiguous()):
            raise ValueError("rng_state must be a contiguous device tensor of two 64-bit integers")
        prm.plan.rng_state = rng_state.data_ptr()
    return prm


def prepare_bias(attention_mask, b, h, sq, sk):
    """Additive mask -> fp32 tensor viewed as [B,H,Sq,Sk] with stride 0 on broadcast dims."""
    if attention_mask is None:
        return None
    m = attention_mask
    if m.ndim != 4:
        raise ValueError("attention_mask must be 4-D ([B,1,1,Sk] or [B,H,Sq,Sk])")
    m = m.float() if m.dtype != torch.float32 else m
    return m.expand(b, h, sq, sk)


def attn_fwd(q, k, v, bias, causal, window, scale, p, seed, offset, plan, save_mask=None,
             rng_state=None):
    """Returns (o, lse, (q, k, v) as consumed); when save_mask is given (True / False) a fourth
    item: the dropout keep bits for attn_bwd, or None (save_mask False, p == 0, fp32)."""
    _require_device(q, k, v, bias)
    q, k, v = _usable_layout(q), _usable_layout(k), _usable_layout(v)
    b, sq, h, d = q.shape
    o = torch.empty((b, sq, h, d), dtype=q.dtype, device=q.device)
    lse = torch.empty((b, h, sq), dtype=torch.float32, device=q.device)
    prm = make_attn_params(q, k, v, o, bias, causal, window, scale, p, seed, offset, plan,
                           rng_state=rng_state)
    keep_mask = None
    if save_mask and o.numel():
        nbytes = _lib.load().slapo_amd_attn_keep_mask_bytes(ctypes.byref(prm))
        if nbytes:
            keep_mask = torch.empty(nbytes // 4, dtype=torch.int32, device=q.device)
            prm.keep_mask = keep_mask.data_ptr()
    if o.numel():
        with _on(q.device):
            rc = _lib.load().slapo_amd_attn_fwd(ctypes.byref(prm), _ptr(q), _ptr(k), _ptr(v),
                                                _ptr(bias), _ptr(o), _ptr(lse), _stream())
        _lib.check(rc, "slapo_amd_attn_fwd")
    if save_mask is not None:
        return o, lse, (q, k, v), keep_mask
    return o, lse, (q, k, v)


def attn_bwd(dout, q, k, v, bias, o, lse, causal, window, scale, p, seed, offset, plan,
             keep_mask=None, rng_state=None):
    _require_device(dout, q, k, v, o, lse, bias)
    dout = dout if dout.stride() == o.stride() else dout.contiguous()
    if dout.stride() != o.stride():
        o = o.contiguous()
    dq = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    dk = torch.empty(k.shape, dtype=k.dtype, device=k.device)
    dv = torch.empty(v.shape, dtype=v.dtype, device=v.device)
    prm = make_attn_params(q, k, v, o, bias, causal, window, scale, p, seed, offset, plan,
                           keep_mask, rng_state)
    if dq.numel() and dk.numel():
        lib = _lib.load()
        nbytes = lib.slapo_amd_attn_bwd_workspace_bytes(ctypes.byref(prm))
        with _on(q.device):
            ws = torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device=q.device)
            rc = lib.slapo_amd_attn_bwd(
                ctypes.byref(prm), _ptr(q), _ptr(k), _ptr(v), _ptr(bias), _ptr(o), _ptr(dout),
                _ptr(lse), _ptr(dq), _ptr(dk), _ptr(dv), _bshd_strides(dq), _bshd_strides(dk),
                _bshd_strides(dv), _ptr(ws), nbytes, _stream())
        _lib.check(rc, "slapo_amd_attn_bwd")
    else:
        dq.zero_(), dk.zero_(), dv.zero_()
    return dq, dk, dv
