"""Tuning knobs of the fused GEMM+collective operators.

Field-for-field the reference's FusedConfig (iris/ops/config.py:12-104), including its defaults and
its validation messages.  What the fields mean for the HIP kernels:

  block_size_m / block_size_n   size of a *flag tile*: one ready flag (`locks[t]`) and one owner per
                                block_size_m x block_size_n output block, numbered row-major.  The
                                kernels pick their own MFMA macro-tile; flags and ownership always
                                follow these two numbers, so results match the reference bit for bit
                                in where they land.
  block_size_k                  lower bound on K (K_local) checked by the operators; no effect on
                                results.
  all_reduce_variant            "one_shot" or "two_shot" are implemented.
  the remaining fields          accepted and validated, not used by the HIP kernels (tile order and
                                caching are fixed by the kernel).
"""

from dataclasses import dataclass
from typing import Optional

_VARIANTS = ["atomic", "ring", "one_shot", "two_shot", "spinlock"]


@dataclass
class FusedConfig:
    # GEMM
    block_size_m: int = 256
    block_size_n: int = 64
    block_size_k: int = 64
    group_size_m: int = 1
    num_sms: Optional[int] = None
    num_xcds: int = 1
    chunk_size: int = 1
    cache_modifier_a: str = ".ca"
    cache_modifier_b: str = ".ca"
    allow_tf32: bool = True
    # collective
    all_reduce_variant: str = "two_shot"
    all_reduce_num_rings: int = 1

    def validate(self, world_size: Optional[int] = None):
        """Raise ValueError for a setting no kernel could honour."""
        for name in ("block_size_m", "block_size_n", "block_size_k", "group_size_m"):
            value = getattr(self, name)
            if value <= 0:
                raise ValueError(f"{name} must be positive, got {value}")
        if self.num_sms is not None and self.num_sms <= 0:
            raise ValueError(f"num_sms must be positive, got {self.num_sms}")
        for name in ("num_xcds", "chunk_size"):
            value = getattr(self, name)
            if value <= 0:
                raise ValueError(f"{name} must be positive, got {value}")
        if self.all_reduce_variant not in _VARIANTS:
            raise ValueError(f"all_reduce_variant must be one of {_VARIANTS}, got {self.all_reduce_variant}")
        if self.all_reduce_variant == "ring" and world_size is not None:
            if self.block_size_n % world_size != 0:
                raise ValueError(
                    f"For ring variant, block_size_n ({self.block_size_n}) must be "
                    f"divisible by world_size ({world_size})"
                )
        if self.all_reduce_num_rings <= 0:
            raise ValueError(f"all_reduce_num_rings must be positive, got {self.all_reduce_num_rings}")
