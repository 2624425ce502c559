"""Sparse-linear attention ("SLA") backend on the MI355X HIP library.

Drop-in for ksana/operations/attention/backends/sage_sla.py:100-292.  Per call (unless ``dense_only``):

1. a block map: q and the mean-centred k are averaged over blocks of 128 query rows / 64 keys, the block
   averages are multiplied, and every query block keeps its ``topk`` share of the key blocks with the largest
   products (sage_sla.py:43-90, 189);
2. block-sparse quantized attention over the kept blocks (sage_sla.py:196-271) - here this package's masked
   kernel, which takes the int8 map as it is;
3. a linear-attention branch on softmax feature maps of q and k, passed through the block's ``proj_l`` layer, added
   to the sparse result (sage_sla.py:273-287).

Steps 1 and 3 are a handful of dense torch operations and stay torch operations; step 2 is the hot part.
Block averages are fp32 sums divided by the block's row count, rounded to the input type, as the reference's
pooling kernel computes them (sage_sla.py:43-63); which of two key blocks with (nearly) equal products makes the
cut may differ from the reference, whose pooling runs in another summation order.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

from .. import _capi, platform
from ..config import KsanaAttentionBackend, KsanaSageSLAConfig
from ..sage_ops import MASK_BLKK, MASK_BLKQ, block_sparse_sage2_attn
from .base import KsanaAttentionBackendImpl


def block_means(x: torch.Tensor, rows: int) -> torch.Tensor:
    """``[B, H, L, D]`` -> ``[B, H, ceil(L / rows), D]``: mean over each run of ``rows`` positions (the last run may be
    shorter), accumulated in fp32 and rounded to ``x.dtype``."""
    B, H, L, D = x.shape
    nblk = -(-L // rows)
    pad = nblk * rows - L
    xf = x.float()
    if pad:
        xf = F.pad(xf, (0, 0, 0, pad))
    sums = xf.view(B, H, nblk, rows, D).sum(dim=3)
    counts = torch.full((nblk,), float(rows), device=x.device)
    counts[-1] = rows - pad
    return (sums / counts.view(1, 1, nblk, 1)).to(x.dtype)


def topk_block_map(q: torch.Tensor, k: torch.Tensor, topk_ratio: float, blk_q: int = MASK_BLKQ,
                   blk_k: int = MASK_BLKK) -> tuple[torch.Tensor, int]:
    """int8 ``[B, H, ceil(Lq / blk_q), ceil(Lk / blk_k)]`` with ``topk`` ones per row, and ``topk``
    (``get_block_map``, sage_sla.py:78-90).  q, k are ``[B, H, L, D]``."""
    centred = k - torch.mean(k, dim=-2, keepdim=True)
    score = block_means(q, blk_q) @ block_means(centred, blk_k).transpose(-1, -2)
    nk = score.shape[-1]
    keep = min(nk, int(topk_ratio * nk))
    picked = torch.topk(score, keep, dim=-1, sorted=False).indices
    block_map = torch.zeros_like(score, dtype=torch.int8)
    block_map.scatter_(-1, picked, 1)
    return block_map, keep


def linear_branch(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """Linear attention on softmax feature maps over the channel axis (sage_sla.py:135-139, 273-282); ``[B, H, L, D]``."""
    fq = F.softmax(q, dim=-1).contiguous().to(q.dtype)
    fk = F.softmax(k, dim=-1).contiguous().to(q.dtype)
    kv = fk.transpose(-1, -2) @ v
    ksum = torch.sum(fk, dim=-2, keepdim=True)
    return (fq @ kv) / (1e-5 + (fq * ksum).sum(dim=-1, keepdim=True))


class SageSLAAttentionImpl(KsanaAttentionBackendImpl):
    @staticmethod
    def type() -> KsanaAttentionBackend:
        return KsanaAttentionBackend.SAGE_SLA

    @staticmethod
    def supports(**kwargs) -> bool:
        if not platform.is_sage_device():
            return False
        _capi.load()
        head_size = kwargs.get("head_size")
        return head_size is None or head_size == 128

    def __init__(self, attention_config: KsanaSageSLAConfig, num_heads: int, head_size: int, causal: bool,
                 softmax_scale: float, num_kv_heads: int | None = None, **extra_impl_args) -> None:
        if not platform.is_gpu():
            raise RuntimeError("SageSLA backend requested but no HIP device is available.")
        if not isinstance(attention_config, KsanaSageSLAConfig):
            raise ValueError("KsanaSageSLAConfig must be provided")
        self.attention_config = attention_config
        self.topk = attention_config.topk
        self.softmax_scale = softmax_scale
        from ..attention_op import KsanaAttentionOp  # lazy: the op imports this package's backends

        self.dense_attn = KsanaAttentionOp(num_heads, head_size, causal=causal, softmax_scale=softmax_scale,
                                           num_kv_heads=num_kv_heads,
                                           attention_config=attention_config.dense_attention_config)
        self.check_config()

    def forward(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, *, dense_only: bool = False,
                proj_l: torch.nn.Module | None = None, **kwargs) -> torch.Tensor:
        if dense_only:
            return self.dense_attn(query, key, value, **kwargs)
        return self.sla_forward(query, key, value, proj_l)

    def sla_forward(self, query, key, value, proj_l, return_sparsity: bool = False):
        """``[B, L, H, D]`` in and out; ``proj_l`` is the block's linear layer for the linear branch."""
        dtype = query.dtype
        q, k, v = (t.transpose(1, 2) for t in (query, key, value))  # [B, H, L, D] views
        block_map, kept = topk_block_map(q, k, self.topk)
        o_sparse = block_sparse_sage2_attn(query, key, value, block_map, tensor_layout="NHD",
                                           sm_scale=q.shape[-1] ** -0.5)
        o_linear = linear_branch(q, k, v)
        with torch.amp.autocast("cuda", dtype=dtype):
            o_linear = proj_l(o_linear)
        out = (o_sparse.transpose(1, 2) + o_linear).to(dtype).transpose(1, 2)
        if return_sparsity:
            return out, kept / block_map.shape[-1]
        return out
