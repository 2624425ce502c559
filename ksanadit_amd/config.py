"""Backend selector for the attention op: enum + frozen config.

Mirrors ksana/config/attention_config.py:23-104 for the backends this package provides.
The enum keeps the reference's string values so a config written for the reference selects the
same backend here; names the reference knows but this package does not build
(flash / laser) are accepted by the enum and rejected by ``support()`` exactly
as the reference rejects a backend missing from its platform list
(attention_config.py:62-68, 79-83).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from enum import Enum


class KsanaAttentionBackend(Enum):
    SAGE_ATTN = "sage_attention"
    FLASH_ATTN = "flash_attention"
    TORCH_SDPA = "torch_sdpa"
    RADIAL_SAGE_ATTN = "radial_sage_attention"
    SAGE_SLA = "sage_sla"
    LASER_ATTN = "laser_attention"

    @staticmethod
    def _get_gpu_supported() -> list["KsanaAttentionBackend"]:
        # order is the fallback order of the selector (backends/base.py)
        return [KsanaAttentionBackend.SAGE_ATTN, KsanaAttentionBackend.TORCH_SDPA, KsanaAttentionBackend.RADIAL_SAGE_ATTN,
                KsanaAttentionBackend.SAGE_SLA]

    @staticmethod
    def get_supported_list(exclude: list["KsanaAttentionBackend"] | None = None) -> list[str]:
        skip = set(exclude or ())
        return [b.value for b in KsanaAttentionBackend._get_gpu_supported() if b not in skip]

    @staticmethod
    def support(type) -> bool:  # noqa: A002 - the reference's argument name
        if isinstance(type, KsanaAttentionBackend):
            return True
        if isinstance(type, str):
            return type in KsanaAttentionBackend.get_supported_list()
        return False


DEFAULT_ATTENTION_BACKEND = KsanaAttentionBackend.SAGE_ATTN


@dataclass(frozen=True)
class KsanaAttentionConfig:
    backend: KsanaAttentionBackend | str | None = field(default=DEFAULT_ATTENTION_BACKEND)

    def __post_init__(self):
        if not KsanaAttentionBackend.support(self.backend):
            raise ValueError(
                f"attention_config {self.backend} not supported in {KsanaAttentionBackend.get_supported_list()}"
            )


@dataclass(frozen=True)
class KsanaRadialSageAttentionConfig(KsanaAttentionConfig):
    """Settings of the radial block-sparse backend (attention_config.py:86-104)."""

    backend: KsanaAttentionBackend = field(init=False, default=KsanaAttentionBackend.RADIAL_SAGE_ATTN)
    dense_blocks_num: int = field(default=0)
    dense_attn_steps: int = field(default=0)
    decay_factor: float = field(default=0.02)
    block_size: int = field(default=128)
    dense_attention_config: KsanaAttentionConfig = field(
        default=KsanaAttentionConfig(backend=KsanaAttentionBackend.SAGE_ATTN)
    )

    def __post_init__(self):
        if self.block_size not in [64, 128]:
            raise ValueError(f"block_size must be 64 or 128, got {self.block_size}")
        if not (0 < self.decay_factor < 1):
            raise ValueError(f"decay_factor must be in range (0, 1), got {self.decay_factor}")


@dataclass(frozen=True)
class KsanaSageSLAConfig(KsanaAttentionConfig):
    """Settings of the sparse-linear backend (attention_config.py:107-119): ``topk`` is the share of key blocks
    every query block keeps."""

    backend: KsanaAttentionBackend = field(init=False, default=KsanaAttentionBackend.SAGE_SLA)
    dense_attention_config: KsanaAttentionConfig = field(
        default=KsanaAttentionConfig(backend=KsanaAttentionBackend.SAGE_ATTN)
    )
    topk: float = field(default=0.1)

    def __post_init__(self):
        if not (0 < self.topk < 1):
            raise ValueError(f"topk must be in range (0, 1), got {self.topk}")
