"""``ops.Attn`` factory: binds a config into the op class (ksana/operations/attention/pick_attn.py:22-23)."""

from functools import partial

from .attention_op import KsanaAttentionOp
from .config import KsanaAttentionConfig


def pick_attn_op(attention_config: KsanaAttentionConfig):
    return partial(KsanaAttentionOp, attention_config=attention_config)
