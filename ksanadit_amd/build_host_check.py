"""Build ``host_args_check``: the C ABI's argument validation driven from C++, with AddressSanitizer on the HOST pass
of every source (the device code is compiled as usual and never launched).  Runs without a GPU.

``python -m ksanadit_amd.build_host_check`` builds and runs it.
"""

from __future__ import annotations

import os
import subprocess
import sys

from .build import CSRC, HIPCC_FLAGS, PKG_DIR, SOURCES, hipcc_path

EXE_PATH = PKG_DIR / "host_args_check"


def build_host_check(verbose: bool = True):
    flags = [f for f in HIPCC_FLAGS if f not in ("-shared", "-fPIC", "-O3")]
    cmd = [hipcc_path(), *flags, "-O1", "-g", "-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fno-omit-frame-pointer",
           "-o", str(EXE_PATH), str(CSRC / "host_args_check.cpp"), *[str(CSRC / s) for s in SOURCES]]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        noise = "packed-fp32-ops' is not a recognized feature"
        log = "\n".join(l for l in (proc.stdout + proc.stderr).splitlines() if noise not in l)
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{log}")
    return EXE_PATH


def run_host_check() -> subprocess.CompletedProcess:
    """Run the check (leak detection off: the HIP runtime's own start-up allocations are not ours to judge)."""
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0")
    return subprocess.run([str(EXE_PATH)], capture_output=True, text=True, env=env, timeout=120)


if __name__ == "__main__":
    build_host_check()
    r = run_host_check()
    print(r.stdout, r.stderr)
    sys.exit(r.returncode)
