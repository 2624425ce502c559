"""Seeded synthetic q/k/v for the five attention shapes the path is measured on.

Shapes come from the reference's model settings (heads/head_dim in
ksana/settings/wan/modules/14b.yaml:18-22, 5b.yaml:18-22, ksana/settings/qwen/modules/20b.yaml:20-22;
sequence length rule ``L = f*h*w/(p_h*p_w)`` in ksana/models/wan/wan_model.py:775-783; Qwen joint
sequences are text tokens first, then image tokens, ksana/models/qwen/attention.py:355-357).

Values are drawn on the CPU in fp32 from one ``torch.Generator`` per workload, in the fixed order
q, k, v, k_offset, q_outlier_mask, k_outlier_mask, then cast to the requested half dtype.
"N(0, s)" means standard deviation ``s``.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    seed: int
    B: int
    H: int
    L: int
    D: int = 128
    k_offset_std: float = 2.0
    outlier_p: float = 0.0
    outlier_gain: float = 20.0
    text_tokens: int = 0
    text_std: float = 1.0

    @property
    def flops(self) -> float:
        """Attention flops of one call: QK^T and PV, a multiply-add counted as 2."""
        return 4.0 * self.B * self.H * self.L * self.L * self.D

    @property
    def elements(self) -> int:
        return self.B * self.H * self.L * self.D


WORKLOADS = {
    w.name: w
    for w in (
        Workload("cpu_plumbing", 1001, 1, 40, 1560),
        Workload("wan5b_720p", 1002, 1, 24, 27280),
        Workload("wan14b_480p", 1003, 1, 40, 32760, outlier_p=1e-3),
        Workload("wan14b_720p", 1004, 1, 40, 75600, outlier_p=1e-3),
        Workload("qwen_cfg", 1005, 2, 24, 4352, text_tokens=256, text_std=3.0),
    )
}
HEADLINE = "wan14b_480p"


def make_inputs(w: Workload | str, dtype=torch.bfloat16, device="cpu", heads: int | None = None, seq: int | None = None):
    """Return (q, k, v), each ``[B, L, H, D]``.  ``heads``/``seq`` shrink the workload (same
    distributions, same seed) for tests and bounded CPU timings."""
    if isinstance(w, str):
        w = WORKLOADS[w]
    H = w.H if heads is None else heads
    L = w.L if seq is None else seq
    shape = (w.B, L, H, w.D)
    g = torch.Generator().manual_seed(w.seed)
    q = torch.randn(shape, generator=g, dtype=torch.float32)
    k = torch.randn(shape, generator=g, dtype=torch.float32)
    v = torch.randn(shape, generator=g, dtype=torch.float32)
    off = torch.randn((H, w.D), generator=g, dtype=torch.float32) * w.k_offset_std
    if w.text_tokens:
        t = min(w.text_tokens, L)
        q[:, :t] *= w.text_std
        k[:, :t] *= w.text_std
        v[:, :t] *= w.text_std
    k += off[None, None]
    if w.outlier_p > 0:
        qm = torch.rand(shape, generator=g) < w.outlier_p
        km = torch.rand(shape, generator=g) < w.outlier_p
        q = torch.where(qm, q * w.outlier_gain, q)
        k = torch.where(km, k * w.outlier_gain, k)
    return tuple(t.to(dtype).to(device) for t in (q, k, v))
