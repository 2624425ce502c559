"""Sage attention backend on the MI355X HIP library.

Drop-in for ksana/operations/attention/backends/sage_attn.py:30-84: same class name, enum type,
constructor and ``forward(query, key, value, **kwargs)``; tensors ``[B, L, H, D]``; inputs that
are not fp16/bf16 are computed in bf16 and the result cast back (sage_attn.py:67-84); every
backend kwarg the model blocks pass (``k_lens``, ``window_size``, ``latent_shape``, ``step_iter``,
``block_id``, ``proj_l``, ``dense_only`` - ksana/models/wan/wan_model.py:182-189,240) is accepted
and ignored, as the reference's adaptor ignores them.

Differences, all deliberate:
* the stored ``softmax_scale`` is USED (the reference stores it and lets the callee default to
  ``D ** -0.5``; the two agree for every caller because attention_op.py:39 defaults to that value);
* ``k_lens``: ignored by default, exactly like the reference's adaptor (sage_attn.py:58-84).  Constructed with
  ``honor_k_lens=True`` the backend limits batch ``b`` to its first ``k_lens[b]`` keys, which is what the reference's
  variable-length backend does with the same argument (flash_attn.py:131-139) and what padded batches need; the same
  switch makes it honour ``q_lens`` (flash_attn.py:120-124): rows of batch ``b`` from ``q_lens[b]`` on are not computed
  and come out as zeros;
* ``out_dtype`` (constructor argument, opt-in): the result is written in that half dtype instead of the query's, which
  folds the cast the Wan block applies before its output projection (wan_model.py:197-204) into the kernel;
* ``smooth_v`` (constructor argument, opt-in): V is quantized around its channel means, which the kernel adds back to
  the output - the option of the same name of the library behind the reference's call;
* ``pwl_exp2`` (constructor argument, opt-in): the kernel's faster form of exp2, about 1.2x the speed at a cosine
  similarity lower by ~1.5e-4;
* availability: no HIP device -> ``supports()`` is False and the selector moves on, like the
  reference without its package (sage_attn.py:21-27,36-38); a HIP device with a missing or stale
  library raises instead of falling back, so a broken build cannot hide behind another backend.
"""

from __future__ import annotations

import torch

from .. import _capi, platform
from ..config import KsanaAttentionBackend, KsanaAttentionConfig
from ..sage_ops import sageattn
from .base import KsanaAttentionBackendImpl

SUPPORTED_HEAD_SIZES = (64, 128)  # 64 runs zero-padded to 128 channels inside the library


class SageAttentionImpl(KsanaAttentionBackendImpl):
    @staticmethod
    def type() -> KsanaAttentionBackend:
        return KsanaAttentionBackend.SAGE_ATTN

    @staticmethod
    def supports(**kwargs) -> bool:
        if not platform.is_sage_device():
            return False
        _capi.load()  # raises SageLibraryError on a GPU host whose library is missing or stale
        head_size = kwargs.get("head_size")
        return head_size is None or head_size in SUPPORTED_HEAD_SIZES

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
        if not platform.is_gpu():
            raise RuntimeError("SageAttention backend requested but no HIP device is available.")
        _capi.load()
        self.causal = causal
        self.softmax_scale = softmax_scale
        self.dropout = float(extra_impl_args.get("dropout_p", 0.0))
        self.honor_k_lens = bool(extra_impl_args.get("honor_k_lens", False))
        # opt-in: the dtype the caller's next layer wants (wan_model.py:197-204 casts the result to the output
        # projection's weight dtype); None keeps the reference's contract, the dtype of the query
        self.out_dtype = extra_impl_args.get("out_dtype")
        # opt-in: the faster piecewise-linear exp2 of the kernel (slightly less accurate, see sage_ops.sageattn)
        self.pwl_exp2 = bool(extra_impl_args.get("pwl_exp2", False))
        # opt-in: V quantized around its channel means (see sage_ops.sageattn)
        self.smooth_v = bool(extra_impl_args.get("smooth_v", False))
        self.attention_config = attention_config
        self.check_config()

    def forward(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, **kwargs) -> torch.Tensor:
        original_dtype = query.dtype
        if original_dtype not in (torch.float16, torch.bfloat16):
            query, key, value = (t.to(torch.bfloat16) for t in (query, key, value))
        k_lens = kwargs.get("k_lens") if self.honor_k_lens else None
        q_lens = kwargs.get("q_lens") if self.honor_k_lens else None
        output = sageattn(query, key, value, tensor_layout="NHD", is_causal=self.causal, sm_scale=self.softmax_scale,
                          k_lens=k_lens, out_dtype=self.out_dtype, pwl_exp2=self.pwl_exp2,
                          smooth_v=self.smooth_v, q_lens=q_lens)
        if self.out_dtype is not None:
            return output
        return output if output.dtype == original_dtype else output.to(original_dtype)
