"""Which attention backend to run, and the settings of the two block-sparse ones.

Same public surface as ksana/config/attention_config.py:23-119 - the enum with the reference's string values, the
frozen config classes with the reference's field names, defaults and ``ValueError`` conditions - so that a
configuration written for the reference selects the same backend here.  Enum members the reference knows but this
package does not build (flash, laser) exist and are refused by ``support()``, the way the reference refuses a backend
that is missing from its platform's list (attention_config.py:62-68, 79-83).
"""

from __future__ import annotations

import dataclasses
from enum import Enum

# member names in the order the selector falls back through them (backends/base.py)
_BUILT_HERE = ("SAGE_ATTN", "TORCH_SDPA", "RADIAL_SAGE_ATTN", "SAGE_SLA")


class KsanaAttentionBackend(Enum):
    SAGE_ATTN = "sage_attention"
    FLASH_ATTN = "flash_attention"
    TORCH_SDPA = "torch_sdpa"
    RADIAL_SAGE_ATTN = "radial_sage_attention"
    SAGE_SLA = "sage_sla"
    LASER_ATTN = "laser_attention"

    @staticmethod
    def _get_gpu_supported() -> list["KsanaAttentionBackend"]:
        return [KsanaAttentionBackend[name] for name in _BUILT_HERE]

    @staticmethod
    def get_supported_list(exclude: list["KsanaAttentionBackend"] | None = None) -> list[str]:
        """String values of the backends built here, minus ``exclude``."""
        left_out = frozenset(exclude) if exclude else frozenset()
        return [member.value for member in KsanaAttentionBackend._get_gpu_supported() if member not in left_out]

    @staticmethod
    def support(type) -> bool:  # noqa: A002 - argument name of the reference
        """An enum member always passes (whether it can run is the selector's business); a string has to name a
        backend built here; anything else, ``None`` included, does not pass."""
        if isinstance(type, KsanaAttentionBackend):
            return True
        return isinstance(type, str) and type in KsanaAttentionBackend.get_supported_list()


DEFAULT_ATTENTION_BACKEND = KsanaAttentionBackend.SAGE_ATTN


def _require_between_0_and_1(name: str, value: float) -> None:
    if not 0 < value < 1:
        raise ValueError(f"{name} must be in range (0, 1), got {value}")


@dataclasses.dataclass(frozen=True)
class KsanaAttentionConfig:
    backend: KsanaAttentionBackend | str | None = DEFAULT_ATTENTION_BACKEND

    def __post_init__(self):
        if KsanaAttentionBackend.support(self.backend):
            return
        known = KsanaAttentionBackend.get_supported_list()
        raise ValueError(f"attention_config {self.backend} not supported in {known}")


_DENSE_SAGE = KsanaAttentionConfig(backend=KsanaAttentionBackend.SAGE_ATTN)


@dataclasses.dataclass(frozen=True)
class KsanaRadialSageAttentionConfig(KsanaAttentionConfig):
    """Radial block-sparse backend (attention_config.py:86-104).  ``dense_blocks_num`` / ``dense_attn_steps``: the
    first transformer blocks / denoising steps that run dense; ``decay_factor``: how fast the spatial window narrows
    with the distance in frames; ``block_size``: mask granularity; ``dense_attention_config``: what runs when dense."""

    backend: KsanaAttentionBackend = dataclasses.field(init=False, default=KsanaAttentionBackend.RADIAL_SAGE_ATTN)
    dense_blocks_num: int = 0
    dense_attn_steps: int = 0
    decay_factor: float = 0.02
    block_size: int = 128
    dense_attention_config: KsanaAttentionConfig = _DENSE_SAGE

    def __post_init__(self):
        if self.block_size != 64 and self.block_size != 128:
            raise ValueError(f"block_size must be 64 or 128, got {self.block_size}")
        _require_between_0_and_1("decay_factor", self.decay_factor)


@dataclasses.dataclass(frozen=True)
class KsanaSageSLAConfig(KsanaAttentionConfig):
    """Sparse-linear backend (attention_config.py:107-119): every query block keeps the ``topk`` share of the key
    blocks for the softmax branch; ``dense_attention_config`` is what runs when the caller asks for dense."""

    backend: KsanaAttentionBackend = dataclasses.field(init=False, default=KsanaAttentionBackend.SAGE_SLA)
    dense_attention_config: KsanaAttentionConfig = _DENSE_SAGE
    topk: float = 0.1

    def __post_init__(self):
        _require_between_0_and_1("topk", self.topk)
