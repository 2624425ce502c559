"""Compile libksana_sage_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

``python -m ksanadit_amd.build`` rebuilds the library in-tree next to this file.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_NAME = "libksana_sage_hip.so"
LIB_PATH = PKG_DIR / LIB_NAME
SOURCES = ("sage_capi.hip", "sage_quant.hip", "sage_attn.hip", "sage_sla.hip", "sage_probe.hip")

HIPCC_FLAGS = (
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-ffp-contract=off",  # the quantizer's arithmetic is specified to the bit; FMAs are written explicitly
    "-fhip-fp32-correctly-rounded-divide-sqrt",  # `/` and sqrtf round correctly (hipcc's default, stated here)
    "-fno-gpu-rdc",
    # packed fp32 VALU forms are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
)


def hipcc_path() -> str:
    found = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(found):
        raise RuntimeError("hipcc not found: the HIP library cannot be built on this host")
    return found


def build_library(verbose: bool = True, extra_flags: tuple[str, ...] = ()) -> Path:
    """Always recompiles; raises ``RuntimeError`` with the compiler output on failure."""
    cmd = [hipcc_path(), *HIPCC_FLAGS, *extra_flags, "-o", str(LIB_PATH), *[str(CSRC / s) for s in SOURCES]]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "packed-fp32-ops' is not a recognized feature"
    log = "\n".join(l for l in (proc.stdout + proc.stderr).splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{log}")
    if verbose and log.strip():
        print(log)
    return LIB_PATH


if __name__ == "__main__":
    build_library()
    print(f"built {LIB_PATH}")
    sys.exit(0)
