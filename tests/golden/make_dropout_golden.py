"""Writes the aten_dropout_*.json fixtures: masks drawn by torch.nn.functional.dropout (the call
the reference makes at slapo/op/fused_bias.py:74 and slapo/op/attention.py:180) on the device
this script runs on, with the generator state they were drawn under.  Run on an MI355X:

    python tests/golden/make_dropout_golden.py <output-dir>

Only torch is used; nothing from the reference or from this repository's kernels."""
import hashlib
import json
import os
import sys

import numpy as np
import torch

CASES = [
    # (name, dtype, numel, p, seed, offset)
    ("f32_n1000", torch.float32, 1000, 0.1, 2013, 0),
    ("f32_n4098_vec2", torch.float32, 4098, 0.25, 7, 8),
    ("f32_n4097_vec1", torch.float32, 4097, 0.5, 11, 4),
    ("bf16_n4096_vec8", torch.bfloat16, 4096, 0.1, 2013, 40),
    ("f16_n4100_vec4", torch.float16, 4100, 0.2, 99, 0),
    ("f32_attn_2x64x64", torch.float32, 2 * 64 * 64, 0.1, 5, 0),
    ("f32_multi_trip", torch.float32, 524288 * 4 + 64, 0.1, 1, 12),
    ("bf16_multi_trip", torch.bfloat16, 524288 * 8 + 128, 0.3, (1 << 40) + 3, 1 << 33),
]


def main(out_dir):
    os.makedirs(out_dir, exist_ok=True)
    props = torch.cuda.get_device_properties(0)
    gen = torch.cuda.default_generators[0]
    for name, dtype, numel, p, seed, offset in CASES:
        torch.cuda.manual_seed(seed)
        gen.set_offset(offset)
        y = torch.nn.functional.dropout(torch.ones(numel, device="cuda", dtype=dtype), p)
        after = gen.get_offset()
        keep = (y != 0).cpu().numpy()
        rec = {
            "numel": numel, "elem_bytes": y.element_size(), "p": p, "seed": seed,
            "offset_before": offset, "offset_after": after,
            "num_cus": props.multi_processor_count,
            "max_threads_per_cu": props.max_threads_per_multi_processor,
            "torch": torch.__version__,
        }
        packed = np.packbits(keep, bitorder="little").tobytes()
        rec["mask_sha256"] = hashlib.sha256(packed).hexdigest()
        rec["keep_count"] = int(keep.sum())
        if numel <= 16384:  # small cases carry every bit; large ones a digest of all bits
            rec["mask_hex"] = packed.hex()
        with open(os.path.join(out_dir, f"aten_dropout_{name}.json"), "w") as f:
            json.dump(rec, f)
        print(name, "keep fraction", keep.mean(), "offset", offset, "->", after, flush=True)


if __name__ == "__main__":
    if len(sys.argv) != 2:
        sys.exit(__doc__)
    main(sys.argv[1])
