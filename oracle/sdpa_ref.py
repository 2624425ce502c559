"""Oracle: the reference's torch-SDPA attention backend, restated.  Test infrastructure only.

Follows ksana/operations/attention/backends/sdpa.py:47-79: tensors arrive ``[B, L, H, D]``,
are transposed to ``[B, H, L, D]``, go through ``F.scaled_dot_product_attention`` and are
transposed back.  ``enable_gqa`` is set when the head counts differ (sdpa.py:66-75).
"""

from __future__ import annotations

import torch
import torch.nn.functional as F


def sdpa_ref(q, k, v, *, scale=None, causal=False):
    """``[B, L, H, D]`` in, ``[B, L, H, D]`` out, in the input dtype (sdpa.py:62-79)."""
    qt, kt, vt = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
    if qt.shape[1] != kt.shape[1]:
        out = F.scaled_dot_product_attention(qt, kt, vt, dropout_p=0.0, is_causal=causal, scale=scale, enable_gqa=True)
    else:
        out = F.scaled_dot_product_attention(qt, kt, vt, dropout_p=0.0, is_causal=causal, scale=scale)
    return out.transpose(1, 2)


def sdpa_ref_fp32(q, k, v, *, scale=None, causal=False):
    """Same computation with fp32 operands: the error budget's zero point."""
    return sdpa_ref(q.float(), k.float(), v.float(), scale=scale, causal=causal)


def attention_bruteforce_f64(q, k, v, *, scale=None, causal=False):
    """Textbook ``softmax(Q K^T * scale) V`` in float64; used only to pin ``sdpa_ref``."""
    B, Lq, H, D = q.shape
    Hkv = k.shape[2]
    scale = D**-0.5 if scale is None else scale
    q64 = q.double().permute(0, 2, 1, 3)
    k64 = k.double().permute(0, 2, 1, 3).repeat_interleave(H // Hkv, dim=1)
    v64 = v.double().permute(0, 2, 1, 3).repeat_interleave(H // Hkv, dim=1)
    s = torch.einsum("bhqd,bhkd->bhqk", q64, k64) * scale
    if causal:
        Lk = k.shape[1]
        mask = torch.ones(Lq, Lk, dtype=torch.bool).tril()
        s = s.masked_fill(~mask, float("-inf"))
    p = torch.softmax(s, dim=-1)
    return torch.einsum("bhqk,bhkd->bhqd", p, v64).permute(0, 2, 1, 3)
