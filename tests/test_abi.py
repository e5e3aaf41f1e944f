"""C-ABI checks that need no GPU: the library loads, exports every symbol the header declares,
and its pure-host entry points (Philox, launch plan, keep threshold, host mask) agree with the
oracle.  No kernel is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest

from oracle import philox as OP
from slapo_amd import _lib
from slapo_amd._lib import DropoutPlan

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "slapo_amd.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(slapo_amd_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    declared = _declared_symbols()
    assert len(declared) >= 16
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/slapo_amd.h but not exported"
    # and the Python prototype table covers the same set
    assert sorted(_lib.PROTOTYPES) == declared


def test_abi_version_and_status_strings():
    lib = _lib.load()
    assert lib.slapo_amd_abi_version() == 3
    assert lib.slapo_amd_status_string(0) == b"ok"
    for code in range(-7, 0):
        assert lib.slapo_amd_status_string(code) not in (b"ok", b"unknown status")


def test_struct_layout_matches_header():
    # sizes the C compiler produces for the two PODs (natural alignment, no packing)
    assert ctypes.sizeof(DropoutPlan) == 40
    assert ctypes.sizeof(_lib.AttnParams) == 4 * 8 + 2 * 4 + 2 * 8 + 16 * 8 + 40 + 8


def test_host_philox_known_answers():
    lib = _lib.load()
    from tests.test_oracle_philox import KAT
    for ctr, key, expect in KAT:
        c = (ctypes.c_uint32 * 4)(*ctr)
        k = (ctypes.c_uint32 * 2)(*key)
        out = (ctypes.c_uint32 * 4)()
        lib.slapo_amd_philox4x32_10(c, k, out)
        assert tuple(out) == expect


@pytest.mark.parametrize("elem_bytes", [2, 4])
def test_plan_matches_oracle(elem_bytes):
    lib = _lib.load()
    rng = np.random.default_rng(0)
    sizes = [1, 2, 3, 4, 255, 256, 257, 1000, 4096, 4098, 4100, 524288, 524296, 2097168,
             8388608, 12582913, 12582914, 4 * 16 * 2048 * 2048]
    sizes += [int(x) for x in rng.integers(1, 1 << 26, size=40)]
    for n in sizes:
        plan = DropoutPlan()
        assert lib.slapo_amd_dropout_plan_for(n, elem_bytes, 256, 256, 2048, ctypes.byref(plan)) == 0
        assert plan.as_dict() == OP.aten_launch_plan(n, elem_bytes, 256, 2048)


def test_plan_rejects_bad_arguments():
    lib = _lib.load()
    plan = DropoutPlan()
    assert lib.slapo_amd_dropout_plan_for(0, 4, 256, 256, 2048, ctypes.byref(plan)) == -4
    assert lib.slapo_amd_dropout_plan_for(16, 3, 256, 256, 2048, ctypes.byref(plan)) == -1
    assert lib.slapo_amd_dropout_plan_for(16, 4, 256, 256, 2048, None) == -4


@pytest.mark.parametrize("p", [0.0, 0.1, 0.2, 0.5, 0.9, 1.0 - 2.0 ** -20, 1.0])
def test_keep_threshold_matches_float_comparison(p):
    lib = _lib.load()
    all_, none = ctypes.c_int(0), ctypes.c_int(0)
    thr = lib.slapo_amd_dropout_threshold(p, ctypes.byref(all_), ctypes.byref(none))
    pkeep = np.float32(1.0 - p)
    if none.value:
        assert not (OP.uniform_from_u32(np.array([0], dtype=np.uint32))[0] < pkeep)
        return
    probe = np.array(sorted({0, max(thr, 1) - 1, thr, min(thr + 1, 2 ** 32 - 1), 2 ** 32 - 1}),
                     dtype=np.uint64).astype(np.uint32)
    keep = OP.uniform_from_u32(probe) < pkeep
    for v, k in zip(probe.tolist(), keep.tolist()):
        assert k == (v <= thr), (p, v, thr)
    assert bool(all_.value) == bool(keep[-1])


@pytest.mark.parametrize("numel,elem_bytes,p,seed,offset", [
    (1000, 4, 0.1, 2013, 0),
    (4098, 4, 0.25, 7, 8),          # vec 2
    (4097, 4, 0.5, 11, 4),          # vec 1
    (4096, 2, 0.1, 2013, 40),       # vec 8
    (4100, 2, 0.2, 99, 0),          # vec 4 on a 2-byte type
    (2 * 64 * 64, 4, 0.1, 5, 0),
    (4096, 1, 0.3, 3, 0),           # vec 16
    (5000, 4, 0.1, (1 << 40) + 3, 1 << 33),
])
def test_host_mask_matches_oracle(numel, elem_bytes, p, seed, offset):
    lib = _lib.load()
    plan = DropoutPlan()
    # a tiny "device" (2 CUs) so that several loop trips occur even at these sizes
    assert lib.slapo_amd_dropout_plan_for(numel, elem_bytes, 256, 2, 512, ctypes.byref(plan)) == 0
    mask = np.zeros(numel, dtype=np.uint8)
    rc = lib.slapo_amd_dropout_mask_host(mask.ctypes.data_as(ctypes.c_void_p), ctypes.byref(plan),
                                         p, seed, offset)
    assert rc == 0
    ref = OP.aten_dropout_mask(OP.aten_launch_plan(numel, elem_bytes, 2, 512), p, seed, offset)
    assert np.array_equal(mask.astype(bool), ref)


def test_compute_entry_points_validate_before_touching_the_device():
    """Argument errors are reported from host code; nothing is launched for them."""
    lib = _lib.load()
    assert lib.slapo_amd_bias_gelu_fwd(None, None, None, 4, 4, 0, None) == -4
    assert lib.slapo_amd_bias_gelu_fwd(1, 1, 1, 0, 4, 0, None) == -2
    assert lib.slapo_amd_bias_gelu_fwd(16, 16, 16, 4, 4, 9, None) == -1
    assert lib.slapo_amd_colsum_workspace_bytes(8192, 4096) == 128 * 4096 * 4
    prm = _lib.AttnParams()
    prm.dtype, prm.batch, prm.heads, prm.seqlen_q, prm.seqlen_k, prm.head_dim = 1, 1, 1, 8, 8, 136
    assert lib.slapo_amd_attn_fwd(ctypes.byref(prm), 16, 16, 16, None, 16, 16, None) == -2
    prm.head_dim = 20  # not a multiple of 8 for a 16-bit type
    assert lib.slapo_amd_attn_fwd(ctypes.byref(prm), 16, 16, 16, None, 16, 16, None) == -2
    prm.head_dim, prm.dtype = 64, 7
    assert lib.slapo_amd_attn_fwd(ctypes.byref(prm), 16, 16, 16, None, 16, 16, None) == -1
    prm.dtype = 2
    prm.q_strides[1] = 68  # rows not 16-byte aligned
    assert lib.slapo_amd_attn_fwd(ctypes.byref(prm), 16, 16, 16, None, 16, 16, None) == -3
    prm.q_strides[1] = 1 << 24  # row stride beyond the 32-bit tile offsets of the 16-bit kernels
    assert lib.slapo_amd_attn_fwd(ctypes.byref(prm), 16, 16, 16, None, 16, 16, None) == -2
    prm.q_strides[1] = 64
    prm.p_drop = 0.5  # dropout without a valid plan
    assert lib.slapo_amd_attn_fwd(ctypes.byref(prm), 16, 16, 16, None, 16, 16, None) == -4
    prm.p_drop, prm.dtype = 0.0, 1
    for bad in (float("nan"), float("inf"), -float("inf")):  # a softmax scale that is no number
        prm.scale = bad
        assert lib.slapo_amd_attn_fwd(ctypes.byref(prm), 16, 16, 16, None, 16, 16, None) == -4
    prm.scale = 0.125
    assert lib.slapo_amd_attn_bwd_workspace_bytes(ctypes.byref(prm)) == 8 * 4
    # keep-bit buffer: one uint32 per (batch*head, 32 keys, query rounded up to 4); none without
    # dropout or for fp32
    assert lib.slapo_amd_attn_keep_mask_bytes(ctypes.byref(prm)) == 0
    prm.p_drop, prm.batch, prm.heads, prm.seqlen_q, prm.seqlen_k = 0.1, 2, 3, 70, 65
    assert lib.slapo_amd_attn_keep_mask_bytes(ctypes.byref(prm)) == 2 * 3 * 3 * 72 * 4
    prm.dtype = 0
    assert lib.slapo_amd_attn_keep_mask_bytes(ctypes.byref(prm)) == 0


def test_host_mask_mirror_refuses_a_device_resident_pair():
    """plan.rng_state names device memory; the host mirror cannot read it and says so."""
    lib = _lib.load()
    plan = DropoutPlan()
    assert lib.slapo_amd_dropout_plan_for(64, 2, 256, 256, 2048, ctypes.byref(plan)) == 0
    assert plan.rng_state is None
    host = np.zeros(64, dtype=np.uint8)
    assert lib.slapo_amd_dropout_mask_host(host.ctypes.data_as(ctypes.c_void_p),
                                           ctypes.byref(plan), 0.5, 1, 0) == 0
    plan.rng_state = 0x1000
    assert lib.slapo_amd_dropout_mask_host(host.ctypes.data_as(ctypes.c_void_p),
                                           ctypes.byref(plan), 0.5, 1, 0) == -4
