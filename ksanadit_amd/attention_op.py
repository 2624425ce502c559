"""The attention operator the DiT blocks hold: ``op(q, k, v, **kwargs) -> o`` on ``[B, L, H, D]``.

Same contract as ksana/operations/attention/attention_op.py:24-91: the default softmax scale is
``head_size ** -0.5`` (:39), a missing config is a ``ValueError`` (:41-42), the backend object is
built lazily on the first call and rebuilt when the input dtype changes (:53-70), inputs that are
not 4-D are a ``ValueError`` (:80-81), backend kwargs pass through untouched (:86-91), and the
forward is kept out of Dynamo graphs (:72).
"""

from __future__ import annotations

import torch
import torch.nn as nn

from .backends import KsanaAttentionBackendImpl, get_attention_backend_impl
from .config import KsanaAttentionConfig
from .logger import log


class KsanaAttentionOp(nn.Module):
    def __init__(
        self,
        num_heads: int,
        head_size: int,
        *,
        num_kv_heads: int | None = None,
        softmax_scale: float | None = None,
        causal: bool = False,
        attention_config: KsanaAttentionConfig = None,
    ) -> None:
        super().__init__()
        if attention_config is None:
            raise ValueError("attention_config should not be None")
        self.num_heads = num_heads
        self.head_size = head_size
        self.num_kv_heads = num_kv_heads or num_heads
        self.softmax_scale = head_size**-0.5 if softmax_scale is None else softmax_scale
        self.causal = causal
        self.attention_config = attention_config
        self._attn_impl: KsanaAttentionBackendImpl | None = None
        self._attn_impl_dtype: torch.dtype | None = None
        log.debug(f"KsanaAttentionOp with config: {attention_config}")

    @property
    def backend_type(self):
        return None if self._attn_impl is None else self._attn_impl.type()

    def _ensure_impl(self, dtype: torch.dtype) -> None:
        if self._attn_impl is not None and self._attn_impl_dtype == dtype:
            return
        impl_cls = get_attention_backend_impl(
            attention_config=self.attention_config, head_size=self.head_size, dtype=dtype
        )
        self._attn_impl = impl_cls(
            attention_config=self.attention_config,
            num_heads=self.num_heads,
            head_size=self.head_size,
            causal=self.causal,
            softmax_scale=self.softmax_scale,
            num_kv_heads=self.num_kv_heads,
        )
        self._attn_impl_dtype = dtype

    @torch.compiler.disable
    def forward(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, **backend_kwargs) -> torch.Tensor:
        if not (query.dim() == key.dim() == value.dim() == 4):
            raise ValueError("LocalAttentionOp expects tensors shaped [B, L, H, D].")
        self._ensure_impl(query.dtype)
        return self._attn_impl.forward(query, key, value, **backend_kwargs)
