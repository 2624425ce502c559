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
    """``[B, L, H, D]`` in and out around ``torch.nn.functional.scaled_dot_product_attention``; grouped-query
    attention is switched on when the head counts differ (sdpa.py:66-75)."""

    def __init__(self, attention_config: KsanaAttentionConfig, num_heads: int, head_size: int, causal: bool,
                 softmax_scale: float, num_kv_heads: int | None = None, **extra_impl_args) -> None:
        self.attention_config = attention_config
        self.check_config()
        self.causal, self.softmax_scale = causal, softmax_scale
        self.dropout = float(extra_impl_args.get("dropout_p", 0.0))

    @staticmethod
    def type() -> KsanaAttentionBackend:
        return KsanaAttentionBackend.TORCH_SDPA

    @staticmethod
    def supports(**_) -> bool:
        return True  # torch runs this anywhere

    def forward(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, *, q_lens: torch.Tensor = None,
                k_lens: torch.Tensor = None, dropout_p: float = None, softmax_scale: float = None, **_) -> torch.Tensor:
        # the per-call values win over the constructor's (sdpa.py:58-60); q_lens / k_lens are accepted and unused
        options = {
            "dropout_p": self.dropout if dropout_p is None else dropout_p,
            "scale": self.softmax_scale if softmax_scale is None else softmax_scale,
            "is_causal": self.causal,
        }
        if query.shape[2] != key.shape[2]:
            options["enable_gqa"] = True
        heads_first = [t.transpose(1, 2) for t in (query, key, value)]
        return F.scaled_dot_product_attention(*heads_first, **options).transpose(1, 2)
