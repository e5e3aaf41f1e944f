"""ctypes binding of libslapo_amd.so (the C ABI declared in include/slapo_amd.h).

The library is loaded lazily on first use and never built at import time.  If it is missing
the loader raises: there is no eager / CPU substitute for the kernels in this package.
"""
from __future__ import annotations

import ctypes
import os
import threading

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "libslapo_amd.so")

SLAPO_F32, SLAPO_F16, SLAPO_BF16 = 0, 1, 2

c_i64 = ctypes.c_int64
c_u64 = ctypes.c_uint64
c_vp = ctypes.c_void_p


class DropoutPlan(ctypes.Structure):
    _fields_ = [
        ("numel", ctypes.c_int64),
        ("total_threads", ctypes.c_int64),
        ("vec", ctypes.c_int32),
        ("calls_per_iter", ctypes.c_int32),
        ("offset_increment", ctypes.c_int64),
        ("rng_state", ctypes.c_void_p),
    ]

    def as_dict(self):
        """The launch geometry (everything but the optional device-state pointer)."""
        return {name: getattr(self, name) for name, _ in self._fields_ if name != "rng_state"}


class AttnParams(ctypes.Structure):
    _fields_ = [
        ("dtype", ctypes.c_int32),
        ("batch", ctypes.c_int32),
        ("heads", ctypes.c_int32),
        ("seqlen_q", ctypes.c_int32),
        ("seqlen_k", ctypes.c_int32),
        ("head_dim", ctypes.c_int32),
        ("causal", ctypes.c_int32),
        ("window", ctypes.c_int32),
        ("scale", ctypes.c_float),
        ("p_drop", ctypes.c_float),
        ("seed", ctypes.c_uint64),
        ("offset", ctypes.c_uint64),
        ("q_strides", ctypes.c_int64 * 3),
        ("k_strides", ctypes.c_int64 * 3),
        ("v_strides", ctypes.c_int64 * 3),
        ("o_strides", ctypes.c_int64 * 3),
        ("bias_strides", ctypes.c_int64 * 4),
        ("plan", DropoutPlan),
        ("keep_mask", ctypes.c_void_p),
    ]


# name -> (restype, argtypes); this table is also what the symbol-export test walks.
PROTOTYPES = {
    "slapo_amd_abi_version": (ctypes.c_int, []),
    "slapo_amd_status_string": (ctypes.c_char_p, [ctypes.c_int]),
    "slapo_amd_philox4x32_10": (
        None,
        [ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(ctypes.c_uint32),
         ctypes.POINTER(ctypes.c_uint32)],
    ),
    "slapo_amd_dropout_plan_for": (
        ctypes.c_int,
        [c_i64, ctypes.c_int, c_i64, ctypes.c_int, ctypes.c_int, ctypes.POINTER(DropoutPlan)],
    ),
    "slapo_amd_dropout_plan": (
        ctypes.c_int, [c_i64, ctypes.c_int, c_i64, ctypes.c_int, ctypes.POINTER(DropoutPlan)]
    ),
    "slapo_amd_dropout_threshold": (
        ctypes.c_uint32,
        [ctypes.c_double, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)],
    ),
    "slapo_amd_dropout_mask_host": (
        ctypes.c_int, [c_vp, ctypes.POINTER(DropoutPlan), ctypes.c_double, c_u64, c_u64]
    ),
    "slapo_amd_dropout_mask": (
        ctypes.c_int, [c_vp, ctypes.POINTER(DropoutPlan), ctypes.c_double, c_u64, c_u64, c_vp]
    ),
    "slapo_amd_bias_gelu_fwd": (
        ctypes.c_int, [c_vp, c_vp, c_vp, c_i64, c_i64, ctypes.c_int, c_vp]
    ),
    "slapo_amd_colsum_workspace_bytes": (ctypes.c_size_t, [c_i64, c_i64]),
    "slapo_amd_bias_gelu_bwd": (
        ctypes.c_int,
        [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, ctypes.c_size_t, c_i64, c_i64, ctypes.c_int, c_vp],
    ),
    "slapo_amd_bias_dropout_residual_fwd": (
        ctypes.c_int,
        [c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, ctypes.c_int, ctypes.c_double, c_u64, c_u64,
         ctypes.POINTER(DropoutPlan), c_vp],
    ),
    "slapo_amd_bias_dropout_residual_bwd": (
        ctypes.c_int,
        [c_vp, c_vp, c_vp, c_vp, ctypes.c_size_t, c_i64, c_i64, ctypes.c_int, ctypes.c_double,
         c_u64, c_u64, ctypes.POINTER(DropoutPlan), c_vp],
    ),
    "slapo_amd_bias_dropout_residual_ln_fwd": (
        ctypes.c_int,
        [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, ctypes.c_int,
         ctypes.c_double, ctypes.c_double, c_u64, c_u64, ctypes.POINTER(DropoutPlan), c_vp],
    ),
    "slapo_amd_ln_bwd_workspace_bytes": (ctypes.c_size_t, [c_i64, c_i64]),
    "slapo_amd_bias_dropout_residual_ln_bwd": (
        ctypes.c_int,
        [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, ctypes.c_size_t,
         c_i64, c_i64, ctypes.c_int, ctypes.c_double, c_u64, c_u64,
         ctypes.POINTER(DropoutPlan), c_vp],
    ),
    "slapo_amd_vocab_ce_fwd": (
        ctypes.c_int,
        [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, ctypes.c_int, c_vp],
    ),
    "slapo_amd_vocab_ce_bwd": (
        ctypes.c_int,
        [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, ctypes.c_double, ctypes.c_int,
         c_vp],
    ),
    "slapo_amd_attn_fwd": (
        ctypes.c_int, [ctypes.POINTER(AttnParams), c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp]
    ),
    "slapo_amd_attn_bwd_workspace_bytes": (ctypes.c_size_t, [ctypes.POINTER(AttnParams)]),
    "slapo_amd_attn_keep_mask_bytes": (ctypes.c_size_t, [ctypes.POINTER(AttnParams)]),
    "slapo_amd_attn_bwd": (
        ctypes.c_int,
        [ctypes.POINTER(AttnParams), c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp,
         ctypes.POINTER(c_i64), ctypes.POINTER(c_i64), ctypes.POINTER(c_i64), c_vp,
         ctypes.c_size_t, c_vp],
    ),
    "slapo_amd_attn_bwd_static_scratch": (
        ctypes.c_int,
        [ctypes.POINTER(AttnParams), c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp,
         ctypes.POINTER(c_i64), ctypes.POINTER(c_i64), ctypes.POINTER(c_i64), c_vp],
    ),
    "slapo_amd_attn_bwd_stages": (
        ctypes.c_int,
        [ctypes.POINTER(AttnParams), c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp,
         ctypes.POINTER(c_i64), ctypes.POINTER(c_i64), ctypes.POINTER(c_i64), c_vp,
         ctypes.c_size_t, ctypes.c_int, c_vp],
    ),
}

BWD_PREPARE, BWD_DKDV, BWD_DQ, BWD_ALL = 1, 2, 4, 7

_lib = None
_lock = threading.Lock()


class SlapoAmdError(RuntimeError):
    """A C-ABI call returned a negative status."""


def load():
    """Return the loaded library, loading it on first use.  Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m slapo_amd.build` "
                "(hipcc, gfx950).  slapo_amd has no fallback implementation."
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def check(status: int, what: str):
    if status != 0:
        msg = load().slapo_amd_status_string(status).decode()
        exc = ValueError if status in (-1, -2, -3, -4) else SlapoAmdError
        raise exc(f"{what} failed: {msg} (status {status})")


def dtype_code(torch_dtype) -> int:
    import torch

    table = {torch.float32: SLAPO_F32, torch.float16: SLAPO_F16, torch.bfloat16: SLAPO_BF16}
    if torch_dtype not in table:
        raise ValueError(f"unsupported dtype {torch_dtype}; expected float32, float16 or bfloat16")
    return table[torch_dtype]
