"""torch SDPA backend: the accuracy anchor of the path and the one backend that runs on a CPU.

Same computation as ksana/operations/attention/backends/sdpa.py:47-79.  ``supports()`` is true on
any host: the reference's version is ``torch.cuda.is_available()`` (sdpa.py:27-29), which leaves a
GPU-less host with no backend at all (base.py:71-73).
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

from ..config import KsanaAttentionBackend, KsanaAttentionConfig
from .base import KsanaAttentionBackendImpl


class SDPAImpl(KsanaAttentionBackendImpl):
    @staticmethod
    def type() -> KsanaAttentionBackend:
        return KsanaAttentionBackend.TORCH_SDPA

    @staticmethod
    def supports(**_) -> bool:
        return True

    def __init__(
        self,
        attention_config: KsanaAttentionConfig,
        num_heads: int,
        head_size: int,
        causal: bool,
        softmax_scale: float,
        num_kv_heads: int | None = None,
        **extra_impl_args,
    ) -> None:
        self.attention_config = attention_config
        self.causal = causal
        self.softmax_scale = softmax_scale
        self.dropout = float(extra_impl_args.get("dropout_p", 0.0))
        self.check_config()

    def forward(
        self,
        query: torch.Tensor,
        key: torch.Tensor,
        value: torch.Tensor,
        *,
        q_lens: torch.Tensor = None,
        k_lens: torch.Tensor = None,
        dropout_p: float = None,
        softmax_scale: float = None,
        **_,
    ) -> torch.Tensor:
        p = self.dropout if dropout_p is None else dropout_p
        s = self.softmax_scale if softmax_scale is None else softmax_scale
        q, k, v = (t.transpose(1, 2) for t in (query, key, value))
        extra = {"enable_gqa": True} if q.shape[1] != k.shape[1] else {}
        out = F.scaled_dot_product_attention(q, k, v, dropout_p=p, is_causal=self.causal, scale=s, **extra)
        return out.transpose(1, 2)
