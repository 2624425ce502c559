"""Radial (block-sparse) Sage attention backend on the MI355X HIP library.

Drop-in for ksana/operations/attention/backends/radial_sage_attn/radial_sage_attn.py:32-176:

* early denoising steps and the first transformer blocks run dense attention through a nested attention op
  (``step_iter < dense_attn_steps or block_id < dense_blocks_num or dense_only``, :93-100);
* otherwise the block mask of the radial pattern for ``(video_token_num = k_lens[0], num_frame)`` is built once,
  cached per ``(query shape, block size, decay factor, token count, frame count, device)`` with at most 16
  entries, oldest out first (:127-168), adapted to 128-row x 64-key blocks (:150-157) and handed to the
  block-sparse kernel (:170-176);
* ``k_lens`` must be the same for every batch entry (:102-103, 119-120); the latent's height and width must be
  multiples of ``block_size / 8`` (:123-124); causal attention is refused (:55-56).

The block-sparse kernel is this package's own (``sage_ops.block_sparse_sage2_attn``), so the backend is available
whenever the Sage backend is.
"""

from __future__ import annotations

import torch

from .. import _capi, platform
from ..config import KsanaAttentionBackend, KsanaRadialSageAttentionConfig
from ..sage_ops import block_sparse_sage2_attn
from .base import KsanaAttentionBackendImpl
from .radial_mask import kernel_block_mask, radial_block_mask


class RadialSageAttentionImpl(KsanaAttentionBackendImpl):
    _global_cache: dict = {}
    _max_cache_size = 16

    @staticmethod
    def type() -> KsanaAttentionBackend:
        return KsanaAttentionBackend.RADIAL_SAGE_ATTN

    @staticmethod
    def supports(**kwargs) -> bool:
        if not platform.is_sage_device():
            return False
        _capi.load()
        head_size = kwargs.get("head_size")
        return head_size is None or head_size == 128

    def __init__(
        self,
        attention_config: KsanaRadialSageAttentionConfig,
        num_heads: int,
        head_size: int,
        causal: bool,
        softmax_scale: float,
        num_kv_heads: int | None = None,
        **extra_impl_args,
    ) -> None:
        if not platform.is_gpu():
            raise RuntimeError("RadialSageAttention backend requested but no HIP device is available.")
        if causal:
            raise ValueError("RadialSageAttention backend does not support causal attention")
        if not isinstance(attention_config, KsanaRadialSageAttentionConfig):
            raise ValueError("KsanaRadialSageAttentionConfig must be provided")
        self.attention_config = attention_config
        self.block_size = attention_config.block_size
        self.decay_factor = attention_config.decay_factor
        self.dense_blocks_num = attention_config.dense_blocks_num
        self.dense_attn_steps = attention_config.dense_attn_steps
        self.softmax_scale = softmax_scale
        from ..attention_op import KsanaAttentionOp  # lazy: the op imports this package's backends

        self.dense_attn = KsanaAttentionOp(
            num_heads,
            head_size,
            causal=causal,
            softmax_scale=softmax_scale,
            num_kv_heads=num_kv_heads,
            attention_config=attention_config.dense_attention_config,
        )
        self.check_config()

    def forward(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, *, dense_only: bool = False,
                k_lens: torch.Tensor | None = None, step_iter: int = -1, block_id: int = -1,
                latent_shape: list[int] | None = None, **kwargs) -> torch.Tensor:
        if dense_only or step_iter < self.dense_attn_steps or block_id < self.dense_blocks_num:
            return self.dense_attn(query, key, value, **kwargs)
        if k_lens is None or not bool((k_lens == k_lens[0]).all()):
            raise ValueError("k_lens must be the same for all tokens")
        video_token_num = int(k_lens[0])
        _, _, num_frame, l_h, l_w = latent_shape
        if l_h % (self.block_size // 8) != 0 or l_w % (self.block_size // 8) != 0:
            raise ValueError(f"output's width and height must be divisible by block size {self.block_size}")
        mask = self.block_mask_for(query, video_token_num, num_frame)
        return block_sparse_sage2_attn(query, key, value, mask, tensor_layout="NHD", sm_scale=self.softmax_scale)

    def block_mask_for(self, query: torch.Tensor, video_token_num: int, num_frame: int) -> torch.Tensor:
        """int8 ``[ceil(L/128), ceil(L/64)]`` on the query's device, from the cache when the same job comes back."""
        cache = RadialSageAttentionImpl._global_cache
        key = (str(tuple(query.shape)), self.block_size, self.decay_factor, video_token_num, num_frame, str(query.device))
        if key not in cache:
            seq_len = query.shape[1]
            pattern = radial_block_mask(seq_len, video_token_num, num_frame, self.block_size, self.decay_factor)
            if len(cache) >= RadialSageAttentionImpl._max_cache_size:
                del cache[next(iter(cache))]
            cache[key] = kernel_block_mask(pattern, self.block_size, seq_len).to(query.device)
        return cache[key]
