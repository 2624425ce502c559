"""MI355X-native quantized (Sage-style) attention behind KsanaDiT's attention-backend interface."""

from .attention_op import KsanaAttentionOp
from .config import DEFAULT_ATTENTION_BACKEND, KsanaAttentionBackend, KsanaAttentionConfig
from .pick_attn import pick_attn_op

__all__ = [
    "KsanaAttentionOp",
    "KsanaAttentionBackend",
    "KsanaAttentionConfig",
    "DEFAULT_ATTENTION_BACKEND",
    "pick_attn_op",
]
