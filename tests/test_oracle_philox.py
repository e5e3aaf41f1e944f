"""Pins for oracle/philox.py (CPU only)."""
import hashlib
import json
import os

import numpy as np
import pytest

from oracle import philox as P

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")

# Known-answer vectors of Philox4x32-10 from the Random123 distribution (kat_vectors).
KAT = [
    ((0x00000000, 0x00000000, 0x00000000, 0x00000000), (0x00000000, 0x00000000),
     (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)),
    ((0xFFFFFFFF, 0xFFFFFFFF, 0xFFFFFFFF, 0xFFFFFFFF), (0xFFFFFFFF, 0xFFFFFFFF),
     (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)),
    ((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0),
     (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)),
]


@pytest.mark.parametrize("ctr,key,expect", KAT)
def test_philox_known_answers(ctr, key, expect):
    out = P.philox4x32_10(np.array(ctr, dtype=np.uint32), np.array(key, dtype=np.uint32))
    assert tuple(int(x) for x in out) == expect


def test_philox_is_a_bijection_on_counters():
    # A block cipher in counter mode: distinct counters give distinct blocks.
    ctr = np.zeros((4096, 4), dtype=np.uint32)
    ctr[:, 0] = np.arange(4096)
    out = P.philox4x32_10(ctr, np.broadcast_to(np.array([7, 9], dtype=np.uint32), (4096, 2)))
    assert len({tuple(r) for r in out.tolist()}) == 4096


def test_uniform_conversion_range_and_monotone():
    v = np.array([0, 1, 2 ** 31, 2 ** 32 - 1], dtype=np.uint64).astype(np.uint32)
    u = P.uniform_from_u32(v)
    assert u.dtype == np.float32
    assert u[0] == np.float32(2.0 ** -32) and u[-1] == np.float32(1.0)
    assert np.all(np.diff(u.astype(np.float64)) >= 0)


def test_launch_plan_arithmetic():
    # 256 CUs x 2048 threads: the grid saturates at 2048 blocks = 524288 subsequences.
    p = P.aten_launch_plan(8192 * 1024, 2, 256, 2048)
    assert p == {"numel": 8388608, "total_threads": 524288, "vec": 8, "calls_per_iter": 2,
                 "offset_increment": 16}
    p = P.aten_launch_plan(1000, 4, 256, 2048)
    assert (p["total_threads"], p["vec"], p["offset_increment"]) == (1024, 4, 4)
    p = P.aten_launch_plan(4098, 2, 256, 2048)
    assert (p["total_threads"], p["vec"]) == (4352, 2)
    p = P.aten_launch_plan(12582913, 4, 256, 2048)
    assert (p["vec"], p["calls_per_iter"], p["offset_increment"]) == (1, 1, 28)


def test_keep_fraction_is_one_minus_p():
    plan = P.aten_launch_plan(1 << 16, 4, 256, 2048)
    for p in (0.1, 0.5):
        keep = P.aten_dropout_mask(plan, p, seed=123, offset=0)
        assert abs(keep.mean() - (1 - p)) < 0.01


def _golden_files():
    if not os.path.isdir(GOLDEN):
        return []
    return sorted(f for f in os.listdir(GOLDEN) if f.startswith("aten_dropout_") and f.endswith(".json"))


@pytest.mark.parametrize("fname", _golden_files())
def test_mask_matches_masks_recorded_from_torch_dropout(fname):
    """Fixtures hold masks that torch.nn.functional.dropout produced on an MI355X (the function
    the reference calls); the oracle must reproduce every bit and the offset advance."""
    with open(os.path.join(GOLDEN, fname)) as f:
        g = json.load(f)
    plan = P.aten_launch_plan(g["numel"], g["elem_bytes"], g["num_cus"], g["max_threads_per_cu"])
    assert plan["offset_increment"] == g["offset_after"] - g["offset_before"]
    keep = P.aten_dropout_mask(plan, g["p"], g["seed"], g["offset_before"])
    assert int(keep.sum()) == g["keep_count"]
    packed = np.packbits(keep, bitorder="little").tobytes()
    assert hashlib.sha256(packed).hexdigest() == g["mask_sha256"]
    if "mask_hex" in g:
        expect = np.unpackbits(np.frombuffer(bytes.fromhex(g["mask_hex"]), dtype=np.uint8),
                               bitorder="little")[: g["numel"]].astype(bool)
        assert np.array_equal(keep, expect)
