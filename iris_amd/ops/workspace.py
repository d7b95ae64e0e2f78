"""Reusable scratch of a fused operator: the aux buffer, the flag array, and what they were sized for.

Same fields and reuse rule as the reference's FusedWorkspace (iris/ops/workspace.py:13-85).
"""

from dataclasses import dataclass
from typing import Optional, Tuple

import torch


@dataclass
class FusedWorkspace:
    operation: str = ""
    shape: Tuple[int, ...] = ()  # (M, N, K)
    dtype: Optional[torch.dtype] = None
    world_size: int = 1
    variant: str = ""
    aux_buffer: Optional[torch.Tensor] = None  # own GEMM tile results, read by the peers
    locks: Optional[torch.Tensor] = None  # int32 ready flag per flag tile
    prepared: bool = False

    def matches(self, operation, shape, dtype, world_size, variant="") -> bool:
        """True when the buffers were prepared for exactly this call and have not been used since."""
        same = (self.operation, self.shape, self.dtype, self.world_size, self.variant) == (
            operation, shape, dtype, world_size, variant)
        return same and self.prepared

    def reset(self):
        self.prepared = False

    def clear(self):
        self.aux_buffer = None
        self.locks = None
        self.prepared = False
