"""Compiles the HIP sources of this package into ``_lib/libbnb_amd.so`` for gfx950.

Run as ``python boost-and-broadside_amd/build.py``; also called by the repository's
build entry point.  hipcc cross-compiles, so no GPU is needed.
"""

from __future__ import annotations

import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
INCLUDE = os.path.join(os.path.dirname(PKG_DIR), "include")
LIB_DIR = os.path.join(PKG_DIR, "_lib")
LIB_PATH = os.path.join(LIB_DIR, "libbnb_amd.so")
SOURCES = ("abi.hip", "conv_step.hip", "elementwise.hip", "ffn_bwd.hip", "ffn_fused.hip", "linear_f32.hip", "linear_wgrad.hip",
    "norm_train.hip", "norm_linear.hip", "probe.hip", "rglru_step.hip", "sdpa_bwd.hip", "sdpa_cross_bwd.hip", "sdpa_cross_f32.hip", "sdpa_env.hip", "sdpa_masked.hip", "team_pool.hip", "temporal_seq.hip", "temporal_step.hip")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    # packed-fp32 VALU forms are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-command-line-argument",
    # the direct-to-LDS asm statements write M0 and say so in their clobber lists; clang only warns that M0 is a reserved register
    "-Wno-inline-asm",
]

# Per-source additions.  The fused FFN keeps 64 accumulators live across its chunk loop next
# to two more MFMA results that the vector ALU consumes at once: with MFMA results in AGPRs
# the compiler copies accumulators between the two register files every iteration, in VGPR
# form it does not.
EXTRA_FLAGS = {
    "ffn_fused.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    "ffn_bwd.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
}


def build(verbose: bool = False) -> str:
    """Compile every source and link the shared library; returns its path."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(LIB_DIR, exist_ok=True)
    objects = []
    for src in SOURCES:
        obj = os.path.join(LIB_DIR, src.replace(".hip", ".o"))
        cmd = [hipcc, *HIPCC_FLAGS, *EXTRA_FLAGS.get(src, []), "-I", INCLUDE, "-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj]
        _run(cmd, verbose)
        objects.append(obj)
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objects], verbose)
    return LIB_PATH


def _run(cmd: list[str], verbose: bool) -> None:
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(line for line in proc.stderr.splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)


if __name__ == "__main__":
    print(build(verbose=True))
