"""Sparse-linear attention ("SLA") backend on the MI355X HIP library.

Drop-in for ksana/operations/attention/backends/sage_sla.py:100-292.  Per call (unless ``dense_only``):

1. a block map: q and the mean-centred k are averaged over blocks of 128 query rows / 64 keys (the reference's one
   in-repo GPU kernel, ``compress_kernel`` / ``mean_pool``, sage_sla.py:43-75 - here the averages ride in the
   quantizers of q and k, whose workgroups are exactly those blocks: ``ksana_sage_quant_qk_pooled``; the stand-alone
   kernel is ``ksana_sage_block_means``), the block averages are multiplied, and every query block keeps its ``topk``
   share of the key blocks with the largest products (sage_sla.py:78-90, 189);
2. block-sparse quantized attention over the kept blocks (sage_sla.py:196-271) - this package's masked kernel, which
   takes the int8 map as it is, on the operands quantized once for both steps;
3. a linear-attention branch on softmax feature maps of q and k, passed through the block's ``proj_l`` layer, added
   to the sparse result (sage_sla.py:273-287) - the HIP kernels behind ``ksana_sage_sla_linear``: one pass over k and
   v, one over q, with ``proj_l`` (when it is a plain ``torch.nn.Linear``) and the final sum folded in.

The product of the block averages and the top-k selection are one HIP kernel (``ksana_sage_sla_block_map``; of two key
blocks with equal products the lower index makes the cut - ``torch.topk``, which the reference calls, leaves that open).
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

from .. import _capi, platform, sage_ops
from ..config import KsanaAttentionBackend, KsanaSageSLAConfig
from ..sage_ops import MASK_BLKK, MASK_BLKQ
from .base import KsanaAttentionBackendImpl


def block_map_from_pooled(pooled_q: torch.Tensor, pooled_k: torch.Tensor, topk_ratio: float) -> tuple[torch.Tensor, int]:
    """int8 ``[B, H, nq, nk]`` with ``topk`` ones per row, and ``topk`` (the second half of ``get_block_map``,
    sage_sla.py:83-90).  ``pooled_*``: block averages ``[B, H, n, D]``, k's taken after centring.  On a HIP device with
    at most 1024 key blocks this is one kernel (``ksana_sage_sla_block_map``); otherwise the reference's four torch calls."""
    nk = pooled_k.shape[-2]
    keep = min(nk, int(topk_ratio * nk))
    if pooled_q.is_cuda and nk <= 1024 and pooled_q.shape[-1] == 128 and pooled_q.dtype in (torch.bfloat16, torch.float16):
        return sage_ops.sla_block_map(pooled_q, pooled_k, keep), keep
    score = pooled_q @ pooled_k.transpose(-1, -2)
    picked = torch.topk(score, keep, dim=-1, sorted=False).indices
    block_map = torch.zeros_like(score, dtype=torch.int8)
    block_map.scatter_(-1, picked, 1)
    return block_map, keep


def topk_block_map(query: torch.Tensor, key: torch.Tensor, k_mean: torch.Tensor, topk_ratio: float,
                   blk_q: int = MASK_BLKQ, blk_k: int = MASK_BLKK) -> tuple[torch.Tensor, int]:
    """``get_block_map`` (sage_sla.py:78-90) for ``[B, L, H, D]`` tensors on a HIP device.  ``k_mean``: fp32
    ``[B, H, D]``, k's mean over the sequence rounded to k's dtype - what the K quantizer leaves in its workspace."""
    pooled_q = sage_ops.block_means(query, blk_q)
    pooled_k = sage_ops.block_means(key, blk_k, centre=k_mean)
    return block_map_from_pooled(pooled_q, pooled_k, topk_ratio)


def linear_branch(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """Linear attention on softmax feature maps over the channel axis (sage_sla.py:135-139, 273-282); ``[B, H, L, D]``.
    The reference's five library calls as they stand - what ``sage_ops.sla_linear`` replaces; kept for measurements."""
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
        if dtype not in (torch.float16, torch.bfloat16):
            query, key, value = (t.to(torch.bfloat16) for t in (query, key, value))
        # quantize once; the block map is built next to the quantized operands and drives the attention over them
        ws = sage_ops.workspace_for(query, key)
        pooled_q, pooled_k = sage_ops.quant_qk_pooled(query, key, ws, query.shape[-1] ** -0.5)  # averages ride along
        sage_ops.quant_v(value, ws)
        block_map, kept = block_map_from_pooled(pooled_q, pooled_k, self.topk)
        o_sparse = sage_ops.attn_fwd(ws, torch.empty_like(query), block_mask=block_map)
        if isinstance(proj_l, torch.nn.Linear) and tuple(proj_l.weight.shape) == (query.shape[-1],) * 2:
            # the layer and the sum of the two branches ride along in the linear branch's second pass
            out = sage_ops.sla_linear(query, key, value, proj_l.weight, proj_l.bias, add=o_sparse, out=o_sparse)
        else:
            o_linear = sage_ops.sla_linear(query, key, value)
            with torch.amp.autocast("cuda", dtype=query.dtype):
                o_linear = proj_l(o_linear)
            out = o_sparse + o_linear.to(o_sparse.dtype)
        out = out.to(dtype)
        if return_sparsity:
            return out, kept / block_map.shape[-1]
        return out
