"""Backend plugin interface and selector for the attention op.

The abstract class and the selection walk restate ksana/operations/attention/backends/base.py:27-128:

* a backend is a class with ``type()``, ``supports(**kwargs)`` (called with ``head_size`` and
  ``dtype``, attention_op.py:57-61), the constructor signature below and ``forward(q, k, v, **kw)``;
* the selector rejects a backend outside the supported list with ``ValueError`` (base.py:54-57),
  then tries the requested backend followed by the supported list in order and returns the first
  class whose ``supports`` is true (base.py:59-69); none -> ``RuntimeError`` (base.py:71-73).

One deliberate difference: when the requested backend is passed over, the walk logs a WARNING
(the reference logs at debug level), so a substitution is never silent.
"""

from __future__ import annotations

from abc import ABC, abstractmethod

import torch

from ..config import KsanaAttentionBackend, KsanaAttentionConfig
from ..logger import log

_ATTN_BACKEND_TO_IMPL: dict | None = None


def get_backend_mapping() -> dict:
    """Lazy enum -> class registry (built on first use to avoid import cycles, base.py:27-48)."""
    global _ATTN_BACKEND_TO_IMPL
    if _ATTN_BACKEND_TO_IMPL is None:
        from .radial_sage_attn import RadialSageAttentionImpl
        from .sage_attn import SageAttentionImpl
        from .sage_sla import SageSLAAttentionImpl
        from .sdpa import SDPAImpl

        _ATTN_BACKEND_TO_IMPL = {
            cls.type(): cls for cls in (SageAttentionImpl, SDPAImpl, RadialSageAttentionImpl, SageSLAAttentionImpl)
        }
    return _ATTN_BACKEND_TO_IMPL


def get_attention_backend_impl(attention_config: KsanaAttentionConfig, **kwargs):
    mapping = get_backend_mapping()
    wanted = attention_config.backend
    if not KsanaAttentionBackend.support(wanted):
        raise ValueError(
            f"attn_backend:{wanted} is not in supported_list:{KsanaAttentionBackend.get_supported_list()}"
        )
    first = True
    for candidate in [wanted] + KsanaAttentionBackend.get_supported_list():
        candidate = KsanaAttentionBackend(candidate)
        impl = mapping.get(candidate)
        if impl is None:
            raise ValueError(f"{candidate} not in {list(mapping.keys())}")
        if impl.supports(**kwargs):
            if not first and candidate != KsanaAttentionBackend(wanted):
                log.warning(f"attention backend {wanted} unavailable for {kwargs}; using {candidate}")
            return impl
        log.debug(f"{impl.type()} backend unavailable for {kwargs}")
        first = False
    raise RuntimeError(
        f"No compatible attention({KsanaAttentionBackend.get_supported_list()}) backend available for {kwargs}. "
    )


class KsanaAttentionBackendImpl(ABC):
    """What a backend provides (base.py:76-128): its enum member, an availability probe that receives ``head_size``
    and ``dtype``, the constructor below, and ``forward(query, key, value, **kwargs)`` on ``[B, L, H, D]``."""

    attention_config: KsanaAttentionConfig

    @abstractmethod
    def __init__(self, attention_config: KsanaAttentionConfig, num_heads: int, head_size: int, causal: bool,
                 softmax_scale: float, num_kv_heads: int | None = None, **extra_impl_args) -> None: ...

    @staticmethod
    @abstractmethod
    def type() -> KsanaAttentionBackend: ...

    @staticmethod
    @abstractmethod
    def supports(**kwargs) -> bool: ...

    @abstractmethod
    def forward(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, **kwargs) -> torch.Tensor: ...

    def check_config(self) -> None:
        """A backend built for another backend's config is a programming error (base.py:102-106)."""
        asked, mine = KsanaAttentionBackend(self.attention_config.backend), self.type()
        if asked != mine:
            raise ValueError(f"Attention config {self.attention_config.backend} does not match implementation type {mine}")

    # identity hooks of the reference's interface (base.py:108-118); no caller uses them
    def preprocess_qkv(self, qkv: torch.Tensor) -> torch.Tensor:
        return qkv

    def postprocess_output(self, output: torch.Tensor) -> torch.Tensor:
        return output
