"""numpy restatement of the dropout RNG (test infrastructure; see oracle/__init__.py).

Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11) with the
counter/key layout ATen documents in ATen/core/PhiloxRNGEngine.h (key = seed lo/hi; counter =
[offset lo, offset hi, subsequence lo, subsequence hi]) and the element mapping of ATen's fused
dropout kernels, which is what torch.nn.functional.dropout -- called by the reference at
slapo/op/fused_bias.py:74 and slapo/op/attention.py:179-180 -- runs on a device.
"""
from __future__ import annotations

import numpy as np

M0 = np.uint64(0xD2511F53)
M1 = np.uint64(0xCD9E8D57)
W0 = 0x9E3779B9
W1 = 0xBB67AE85
MASK32 = np.uint64(0xFFFFFFFF)


def philox4x32_10(counter: np.ndarray, key: np.ndarray) -> np.ndarray:
    """counter: [...,4] uint32, key: [...,2] uint32 -> [...,4] uint32 (10 rounds)."""
    c = np.asarray(counter, dtype=np.uint64)
    k = np.asarray(key, dtype=np.uint64)
    c0, c1, c2, c3 = (c[..., i].copy() for i in range(4))
    k0, k1 = k[..., 0].copy(), k[..., 1].copy()
    for _ in range(10):
        p0 = M0 * c0
        p1 = M1 * c2
        n0 = (p1 >> np.uint64(32)) ^ c1 ^ k0
        n1 = p1 & MASK32
        n2 = (p0 >> np.uint64(32)) ^ c3 ^ k1
        n3 = p0 & MASK32
        c0, c1, c2, c3 = n0, n1, n2, n3
        k0 = (k0 + np.uint64(W0)) & MASK32
        k1 = (k1 + np.uint64(W1)) & MASK32
    return np.stack([c0, c1, c2, c3], axis=-1).astype(np.uint32)


def uniform_from_u32(v: np.ndarray) -> np.ndarray:
    """rocRAND's conversion (rocrand_uniform.h): 2^-32 + float(v) * 2^-32, in fp32, (0, 1]."""
    inv = np.float32(2.3283064365386963e-10)
    return (np.asarray(v).astype(np.float32) * inv + inv).astype(np.float32)


def aten_launch_plan(numel: int, elem_bytes: int, num_cus: int, max_threads_per_cu: int,
                     ptr_align: int = 256) -> dict:
    """Launch geometry of ATen's fused dropout for a dense tensor (block 256, capped grid,
    widest vector that the type/alignment allows and that divides numel)."""
    block = 256
    grid = min(num_cus * (max_threads_per_cu // block), (numel + block - 1) // block)
    if elem_bytes == 1 and ptr_align % 16 == 0:
        vec = 16
    elif elem_bytes <= 2 and ptr_align % (8 * elem_bytes) == 0:
        vec = 8
    elif ptr_align % (4 * elem_bytes) == 0:
        vec = 4
    elif ptr_align % (2 * elem_bytes) == 0:
        vec = 2
    else:
        vec = 1
    while vec > 1 and numel % vec:
        vec //= 2
    return {
        "numel": numel,
        "total_threads": grid * block,
        "vec": vec,
        "calls_per_iter": 1 if vec == 1 else (vec + 3) // 4,
        "offset_increment": ((numel - 1) // (block * grid * 4) + 1) * 4,
    }


def aten_dropout_mask(plan: dict, p: float, seed: int, offset: int) -> np.ndarray:
    """Boolean keep-mask [numel] for drop probability p under generator state (seed, offset)."""
    n = plan["numel"]
    T = plan["total_threads"]
    vec = plan["vec"]
    e = np.arange(n, dtype=np.uint64)
    if vec == 1:
        thread = e % np.uint64(T)
        q = e // np.uint64(T)
        call = q // np.uint64(4)
        lane = (q % np.uint64(4)).astype(np.int64)
    else:
        v = e // np.uint64(vec)
        sub = e % np.uint64(vec)
        thread = v % np.uint64(T)
        trip = v // np.uint64(T)
        call = trip * np.uint64(plan["calls_per_iter"]) + sub // np.uint64(4)
        lane = (sub % np.uint64(4)).astype(np.int64)
    ctr = np.uint64(offset // 4) + call
    counter = np.stack(
        [ctr & MASK32, ctr >> np.uint64(32), thread & MASK32, thread >> np.uint64(32)], axis=-1
    )
    key = np.array([seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF], dtype=np.uint64)
    key = np.broadcast_to(key, counter.shape[:-1] + (2,))
    words = philox4x32_10(counter, key)
    w = np.take_along_axis(words, lane[:, None], axis=-1)[:, 0]
    pkeep = np.float32(1.0 - p)
    return uniform_from_u32(w) < pkeep
