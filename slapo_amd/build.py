"""Build recipe for libslapo_amd.so: hipcc cross-compiles every csrc/*.hip for gfx950.

The library is built in-tree (slapo_amd/libslapo_amd.so) so that it travels with the source
tree; nothing is compiled at import time.  `python -m slapo_amd.build` rebuilds it.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.join(PKG_DIR, "csrc")
OBJ_DIR = os.path.join(CSRC_DIR, "build")
LIB_PATH = os.path.join(PKG_DIR, "libslapo_amd.so")

ARCH = "gfx950"

# -packed-fp32-ops is switched off on purpose: the compiler must not form v_pk_*_f32.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=fast",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-unknown-attributes",
]


# The MFMA attention kernels never compute with NaNs on their defined paths (masked scores are
# -inf, guarded before every subtraction); telling the compiler so removes the canonicalising
# v_max x,x it would otherwise put in front of every max of an MFMA result.
PER_FILE_FLAGS = {
    "attn_fwd_f16.hip": ["-fno-honor-nans"],
    "attn_fwd_bf16.hip": ["-fno-honor-nans"],
    "attn_bwd_f16.hip": ["-fno-honor-nans"],
    "attn_bwd_bf16.hip": ["-fno-honor-nans"],
    "attn_bwd_dq_f16.hip": ["-fno-honor-nans"],
    "attn_bwd_dq_bf16.hip": ["-fno-honor-nans"],
}


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libslapo_amd.so cannot be built")
    return exe


def sources() -> list[str]:
    return sorted(
        os.path.join(CSRC_DIR, f) for f in os.listdir(CSRC_DIR) if f.endswith(".hip")
    )


def _compile_one(src: str, extra: list[str]) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    per_file = PER_FILE_FLAGS.get(os.path.basename(src), [])
    cmd = [_hipcc(), *HIPCC_FLAGS, *per_file, *extra, "-c", src, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{proc.stdout}\n{proc.stderr}")
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build_library(verbose: bool = False, extra_flags: list[str] | None = None) -> str:
    """Compile all kernels and link the shared library; always recompiles."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    extra = list(extra_flags or [])
    srcs = sources()
    if verbose:
        print(f"[slapo_amd.build] compiling {len(srcs)} files for {ARCH}", flush=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        objs = list(pool.map(lambda s: _compile_one(s, extra), srcs))
    tmp = LIB_PATH + ".tmp"
    cmd = [_hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp, *objs]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[slapo_amd.build] wrote {LIB_PATH}", flush=True)
    return LIB_PATH


if __name__ == "__main__":
    build_library(verbose=True)
