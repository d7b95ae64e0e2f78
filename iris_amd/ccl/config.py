"""Config of the collectives: the fields and checks of iris/ccl/config.py:17-150."""

from dataclasses import dataclass
from typing import Optional

_ALL_REDUCE_VARIANTS = ["atomic", "ring", "two_shot", "one_shot", "spinlock"]


def _require_positive(name, value):
    if value <= 0:
        raise ValueError(f"{name} must be positive, got {value}")


def _detect_num_xcds():
    """XCD count of the current GPU; 8 (an MI355X) where no GPU can be asked."""
    try:
        import torch

        if torch.cuda.is_available():
            from .. import _lib

            return _lib.query(torch.cuda.current_device())[1]
    except Exception:
        pass
    return 8


@dataclass
class Config:
    """Kernel parameters shared by the collectives.

    The tile grid (block_size_m x block_size_n, grouped by swizzle_size tile-rows), comm_sms and
    all_reduce_distribution decide which tiles a rank reduces and in which order the ranks'
    contributions are added; they are honoured exactly.  How many workgroups run is chosen by the
    library for the machine (comm_sms does not limit the launch).  num_stages, num_warps,
    threads_per_warp, waves_per_eu and use_gluon are compiler hints of the reference's Triton kernels:
    they are validated and otherwise unused.
    """

    block_size_m: int = 32
    block_size_n: int = 64
    swizzle_size: int = 4
    comm_sms: int = 64
    num_xcds: Optional[int] = None
    chunk_size: Optional[int] = None
    use_gluon: bool = False
    all_gather_variant: str = "persistent"
    all_reduce_variant: str = "two_shot"
    all_reduce_distribution: int = 1
    all_reduce_num_rings: int = 1
    all_reduce_ring_slice_n: Optional[int] = None
    reduce_scatter_variant: str = "two_shot"
    num_stages: int = 1
    num_warps: int = 4
    threads_per_warp: int = 64
    waves_per_eu: int = 0

    def __post_init__(self):
        if self.num_xcds is None:
            self.num_xcds = _detect_num_xcds()
        if self.chunk_size is None:
            self.chunk_size = min(self.swizzle_size * self.swizzle_size, self.comm_sms // self.num_xcds)
        # Same checks, order and messages as the reference's Config.__post_init__.
        for name in ("block_size_m", "block_size_n", "swizzle_size", "comm_sms", "num_xcds"):
            _require_positive(name, getattr(self, name))
        if self.all_gather_variant not in ("persistent", "partitioned"):
            raise ValueError(
                f"all_gather_variant must be one of: 'persistent', 'partitioned', got {self.all_gather_variant}"
            )
        if self.all_reduce_variant not in _ALL_REDUCE_VARIANTS:
            listed = ", ".join(repr(v) for v in _ALL_REDUCE_VARIANTS)
            raise ValueError(f"all_reduce_variant must be one of: {listed}, got {self.all_reduce_variant}")
        if self.all_reduce_distribution not in (0, 1):
            raise ValueError(
                f"all_reduce_distribution must be 0 (striding) or 1 (block), got {self.all_reduce_distribution}"
            )
        _require_positive("all_reduce_num_rings", self.all_reduce_num_rings)
        slice_n = self.block_size_n if self.all_reduce_ring_slice_n is None else self.all_reduce_ring_slice_n
        self.all_reduce_ring_slice_n = slice_n
        _require_positive("all_reduce_ring_slice_n", slice_n)
        if self.block_size_n % slice_n:
            raise ValueError(
                f"all_reduce_ring_slice_n must divide block_size_n (block_size_n={self.block_size_n}, slice={slice_n})"
            )
        if slice_n & (slice_n - 1):
            raise ValueError(f"all_reduce_ring_slice_n must be a power of two, got {slice_n}")
        if self.reduce_scatter_variant != "two_shot":
            raise ValueError(f"reduce_scatter_variant must be 'two_shot', got '{self.reduce_scatter_variant}'")
        if self.threads_per_warp not in (32, 64):
            raise ValueError(f"threads_per_warp must be 32 (NVIDIA) or 64 (AMD), got {self.threads_per_warp}")
        _require_positive("num_warps", self.num_warps)
