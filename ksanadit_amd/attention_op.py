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
    def __init__(self, num_heads: int, head_size: int, *, num_kv_heads: int | None = None,
                 softmax_scale: float | None = None, causal: bool = False,
                 attention_config: KsanaAttentionConfig = None) -> None:
        super().__init__()
        if attention_config is None:
            raise ValueError("attention_config should not be None")
        log.debug(f"KsanaAttentionOp with config: {attention_config}")
        self.attention_config = attention_config
        self.num_heads, self.head_size, self.causal = num_heads, head_size, causal
        self.num_kv_heads = num_heads if not num_kv_heads else num_kv_heads
        self.softmax_scale = head_size**-0.5 if softmax_scale is None else softmax_scale
        # the backend object and the input dtype it was picked for
        self._attn_impl: KsanaAttentionBackendImpl | None = None
        self._attn_impl_dtype: torch.dtype | None = None

    @property
    def backend_type(self):
        impl = self._attn_impl
        return impl.type() if impl is not None else None

    def _ensure_impl(self, dtype: torch.dtype) -> None:
        """Pick and build the backend on first use, again when the input dtype changes (a backend may support one
        dtype and not another)."""
        if self._attn_impl is None or self._attn_impl_dtype != dtype:
            cls = get_attention_backend_impl(attention_config=self.attention_config, head_size=self.head_size,
                                             dtype=dtype)
            self._attn_impl = cls(attention_config=self.attention_config, num_heads=self.num_heads,
                                  head_size=self.head_size, causal=self.causal, softmax_scale=self.softmax_scale,
                                  num_kv_heads=self.num_kv_heads)
            self._attn_impl_dtype = dtype

    @torch.compiler.disable
    def forward(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, **backend_kwargs) -> torch.Tensor:
        if any(t.dim() != 4 for t in (query, key, value)):
            raise ValueError("LocalAttentionOp expects tensors shaped [B, L, H, D].")
        self._ensure_impl(query.dtype)
        return self._attn_impl.forward(query, key, value, **backend_kwargs)
