from .base import KsanaAttentionBackendImpl, get_attention_backend_impl, get_backend_mapping

__all__ = ["KsanaAttentionBackendImpl", "get_attention_backend_impl", "get_backend_mapping"]
