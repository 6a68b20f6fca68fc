"""Builds the gfx950 shared library `libkhm_gqa_sdpa.so` in-tree with hipcc.

Run as `python -m khalamari_amd.build` (or through `__graft_entry__.build()`).  hipcc cross-compiles
for gfx950 without a GPU present; the built library is loaded by `khalamari_amd._lib`.
"""
from __future__ import annotations

import os
import subprocess
import sys

PACKAGE_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.join(PACKAGE_DIR, "csrc")
LIB_DIR = os.path.join(PACKAGE_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libkhm_gqa_sdpa.so")

SOURCES = [
    "common.cpp",
    "fp8_codec.cpp",
    "sdpa_registry.cpp",
    "replay_bucket_policy.cpp",
    "selector.cpp",
    "batch_metadata.cpp",
    "bidi_block_metadata.cpp",
    "components.hip",
    "kv_page_write.hip",
    "bidi_block_sdpa.hip",
    "rms_norm_rope.hip",
    "projection_split.hip",
]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-Wall",
    "-Wno-unused-function",
    # packed-FP32 VALU forms are kept off for every device function in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def build_bench_aid(verbose: bool = False) -> str:
    """The read-only slab reader bench.py times beside the bandwidth-bound Map kernels: a library of its own at the
    repository root, not part of `libkhm_gqa_sdpa.so`."""
    root = os.path.dirname(PACKAGE_DIR)
    sources = [os.path.join(root, "bench_slab_read.hip")]
    output = os.path.join(root, "libbench_slab_read.so")
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    command = [hipcc, *HIPCC_FLAGS, "-x", "hip", *sources, "-o", output]
    if verbose:
        print(" ".join(command), flush=True)
    result = subprocess.run(command, capture_output=True, text=True)
    if result.returncode != 0:
        raise RuntimeError(f"hipcc failed ({result.returncode}):\n{result.stderr}")
    return output


def build(verbose: bool = False, extra_flags=(), output: str = LIB_PATH) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    sources = [os.path.join(CSRC_DIR, name) for name in SOURCES if os.path.exists(os.path.join(CSRC_DIR, name))]
    command = [hipcc, *HIPCC_FLAGS, *extra_flags, "-x", "hip", *sources, "-o", output]
    if verbose:
        print(" ".join(command), flush=True)
    result = subprocess.run(command, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    stderr = "\n".join(line for line in result.stderr.splitlines() if noise not in line)
    if result.returncode != 0:
        raise RuntimeError(f"hipcc failed ({result.returncode}):\n{stderr}")
    if verbose and stderr.strip():
        print(stderr, file=sys.stderr)
    return output


if __name__ == "__main__":
    print(build(verbose=True))
    print(build_bench_aid(verbose=True))
