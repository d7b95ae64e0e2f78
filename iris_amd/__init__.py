"""iris_amd: the rank-local compute of Iris's fused GEMM+collective operators on one MI355X.

    import iris_amd as iris
    ctx = iris.iris(heap_size, num_ranks=8)       # W heap slots in one GPU's HBM
    A = ctx.zeros((M, K), dtype=torch.bfloat16)
    ctx.ops.matmul_all_reduce(C, A, B)

The package keeps the reference's Python surface (context, tensor factories, heap_bases, operator
signatures) and runs hand-written gfx950 kernels from libiris_hip.so underneath.
"""

from . import ccl, ops
from .host.bench import do_bench
from .host.iris import Iris, iris
from .host.logging import DEBUG, ERROR, INFO, WARNING, logger, set_logger_level
from .ops import FusedConfig, FusedWorkspace

__all__ = [
    "iris",
    "Iris",
    "ops",
    "ccl",
    "FusedConfig",
    "FusedWorkspace",
    "do_bench",
    "set_logger_level",
    "logger",
    "DEBUG",
    "INFO",
    "WARNING",
    "ERROR",
]
