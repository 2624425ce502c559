"""Backend selector for the attention op: enum + frozen config.

Mirrors ksana/config/attention_config.py:23-83 for the two backends this package provides.
The enum keeps the reference's string values so a config written for the reference selects the
same backend here; names the reference knows but this package does not build
(flash / radial / SLA / laser) are accepted by the enum and rejected by ``support()`` exactly
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
        return [KsanaAttentionBackend.SAGE_ATTN, KsanaAttentionBackend.TORCH_SDPA]

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
