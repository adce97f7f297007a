"""Builds runnburn_amd/librnb_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python -m runnburn_amd.build            # compile every source, link
"""
from __future__ import annotations

import concurrent.futures as cf
import os
import shutil
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(PKG, "librnb_hip.so")

SOURCES = ["state.cpp", "residency.cpp", "api.cpp", "gguf.cpp", "quantize_act.hip", "gemv.hip", "gemm_q4k.hip", "gemm_blocks.hip", "moe.hip", "moe_mfma.hip", "static_scratch.hip", "calib.hip", "norm_route.hip", "gemv_iq.hip", "dequant.hip"]

# -ffp-contract=off: the activation quantisers must perform single IEEE multiplies (no FMA fusion).
# packed-fp32 ops are disabled for every kernel in this library.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-align-mismatch", "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found (expected on PATH or at /opt/rocm/bin/hipcc)")
    return exe


def _compile(src: str) -> str:
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc(), *HIPCC_FLAGS, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass does not know the device-only target feature; that line is harmless
    noise = ("is not a recognized feature for this target", "unknown and will be ignored")
    err = "\n".join(line for line in proc.stderr.splitlines() if not any(n in line for n in noise))
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    with cf.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(_compile, SOURCES))
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    if verbose:
        print(f"built {LIB}")
    return LIB


if __name__ == "__main__":
    build()
