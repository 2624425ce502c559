"""Oracle: the reference's torch-SDPA attention backend, restated.  Test infrastructure only.

Follows ksana/operations/attention/backends/sdpa.py:47-79: tensors arrive ``[B, L, H, D]``,
are transposed to ``[B, H, L, D]``, go through ``F.scaled_dot_product_attention`` and are
transposed back.  ``enable_gqa`` is set when the head counts differ (sdpa.py:66-75).
"""

from __future__ import annotations

import torch
import torch.nn.functional as F


def sdpa_ref(q, k, v, *, scale=None, causal=False, k_lens=None, block_mask=None):
    """``[B, L, H, D]`` in, ``[B, L, H, D]`` out, in the input dtype (sdpa.py:62-79).

    ``k_lens`` (one int per batch entry) follows the reference's variable-length backend, which cuts
    batch ``b`` down to ``key[b, :k_lens[b]]`` / ``value[b, :k_lens[b]]`` before attending
    (flash_attn.py:131-139); here the same keys are kept by a boolean mask.  A batch entry without
    keys gives zeros.

    ``block_mask`` (``[B, H, ceil(Lq/128), ceil(Lk/64)]``, leading dims may be 1): entry ``(i, j)`` non-zero lets
    query rows ``128 i ..`` see keys ``64 j ..``; the meaning of ``mask_id`` in the reference's block-sparse call
    (radial_sage_attn.py:150-176, blocks of 128 x 64).  Rows that see no key give zeros."""
    if block_mask is not None:
        return _sdpa_ref_block_mask(q, k, v, scale, causal, k_lens, block_mask)
    if k_lens is not None:
        return _sdpa_ref_k_lens(q, k, v, scale, causal, k_lens)
    qt, kt, vt = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
    if qt.shape[1] != kt.shape[1]:
        out = F.scaled_dot_product_attention(qt, kt, vt, dropout_p=0.0, is_causal=causal, scale=scale, enable_gqa=True)
    else:
        out = F.scaled_dot_product_attention(qt, kt, vt, dropout_p=0.0, is_causal=causal, scale=scale)
    return out.transpose(1, 2)


def _sdpa_ref_k_lens(q, k, v, scale, causal, k_lens):
    B, Lq, Lk = k.shape[0], q.shape[1], k.shape[1]
    lens = torch.as_tensor(k_lens, dtype=torch.int64).clamp(0, Lk)
    keep = (torch.arange(Lk)[None, :] < lens[:, None])[:, None, None, :]  # [B, 1, 1, Lk]
    if causal:  # the triangle anchored at the top-left corner, as is_causal=True defines it
        keep = keep & torch.ones(Lq, Lk, dtype=torch.bool).tril()
    qt, kt, vt = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
    gqa = qt.shape[1] != kt.shape[1]
    out = F.scaled_dot_product_attention(qt, kt, vt, attn_mask=keep.to(q.device), dropout_p=0.0,
                                         scale=scale, **({"enable_gqa": True} if gqa else {}))
    out = out.transpose(1, 2)
    empty = (lens == 0).to(q.device)
    if bool(empty.any()):
        out = out.clone()
        out[empty] = 0
    return out


def _sdpa_ref_block_mask(q, k, v, scale, causal, k_lens, block_mask, blk_q=128, blk_k=64):
    B, Lq, H, _ = q.shape
    Lk = k.shape[1]
    m = torch.as_tensor(block_mask) != 0
    while m.dim() < 4:
        m = m.unsqueeze(0)
    keep = m.repeat_interleave(blk_q, dim=2)[:, :, :Lq].repeat_interleave(blk_k, dim=3)[:, :, :, :Lk]
    keep = keep.expand(B, H, Lq, Lk)
    if causal:
        keep = keep & torch.ones(Lq, Lk, dtype=torch.bool).tril()
    if k_lens is not None:
        lens = torch.as_tensor(k_lens, dtype=torch.int64).clamp(0, Lk)
        keep = keep & (torch.arange(Lk)[None, :] < lens[:, None])[:, None, None, :]
    qt, kt, vt = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
    gqa = qt.shape[1] != kt.shape[1]
    out = F.scaled_dot_product_attention(qt, kt, vt, attn_mask=keep.to(q.device), dropout_p=0.0, scale=scale,
                                         **({"enable_gqa": True} if gqa else {}))
    dead = ~keep.any(dim=-1)  # [B, H, Lq]
    out = torch.where(dead[..., None].to(q.device), torch.zeros((), dtype=out.dtype, device=out.device), out)
    return out.transpose(1, 2)


def sdpa_ref_fp32(q, k, v, *, scale=None, causal=False, k_lens=None):
    """Same computation with fp32 operands: the error budget's zero point."""
    return sdpa_ref(q.float(), k.float(), v.float(), scale=scale, causal=causal, k_lens=k_lens)


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
