"""Device probes for the attention path.

The reference decides "is this a GPU host" by looking for ``nvidia-smi`` on PATH
(ksana/accelerator/platform.py:21-23), which is False on an AMD machine.  Here a GPU is a
HIP device visible to PyTorch-ROCm; there is no NPU branch.
"""

from __future__ import annotations

import functools

import torch


@functools.lru_cache(maxsize=None)
def is_gpu() -> bool:
    return bool(torch.cuda.is_available()) and torch.version.hip is not None


def is_npu() -> bool:
    return False


@functools.lru_cache(maxsize=None)
def gcn_arch(index: int = 0) -> str:
    """``gfx950`` on MI355X; empty string when no HIP device is present."""
    if not is_gpu():
        return ""
    return torch.cuda.get_device_properties(index).gcnArchName.split(":")[0]


SAGE_ARCH = "gfx950"  # the only architecture libksana_sage_hip.so holds code for


def is_sage_device() -> bool:
    """True when the HIP library's kernels can run here: a HIP device of the architecture it was compiled for.
    On any other device the selector moves on to the next backend, as the reference's availability probe makes it
    (ksana/operations/attention/backends/sage_attn.py:21-27,36-38), instead of failing at the first launch."""
    return gcn_arch() == SAGE_ARCH
