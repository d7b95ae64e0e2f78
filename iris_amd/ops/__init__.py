"""Fused GEMM+collective operators (rank-local compute on one MI355X).

    import iris_amd as iris
    shmem = iris.iris(heap_size, num_ranks=8)
    shmem.ops.matmul_all_reduce(C, A, B)          # via the context
    iris.ops.matmul_all_reduce(shmem, C, A, B)    # or as free functions

Mirrors iris/ops/__init__.py:43-186 of the reference: matmul_all_reduce, all_gather_matmul,
matmul_all_gather and matmul_reduce_scatter.
"""

from .all_gather_matmul import all_gather_matmul, all_gather_matmul_preamble
from .config import FusedConfig
from .matmul_all_gather import matmul_all_gather, matmul_all_gather_preamble
from .matmul_all_reduce import matmul_all_reduce, matmul_all_reduce_preamble
from .matmul_reduce_scatter import matmul_reduce_scatter, matmul_reduce_scatter_preamble
from .workspace import FusedWorkspace


class OpsNamespace:
    """`ctx.ops`: the free functions with the context bound as first argument."""

    def __init__(self, shmem):
        self._shmem = shmem

    def matmul_all_reduce(self, output_tensor, A, B, bias=None, async_op=False, config=None, workspace=None,
                          **kwargs):
        """output = all_reduce(A @ B).  `bias` is accepted and ignored, as in the reference."""
        return matmul_all_reduce(self._shmem, output_tensor, A, B, async_op, config, workspace, **kwargs)

    def all_gather_matmul(self, output_tensor, A_sharded, B, bias=None, async_op=False, config=None,
                          workspace=None, **kwargs):
        """output = all_gather(A_sharded) @ B + bias[:, None]."""
        return all_gather_matmul(self._shmem, output_tensor, A_sharded, B, bias, async_op, config, workspace,
                                 **kwargs)

    def matmul_all_gather(self, output_tensor, A, B, bias=None, async_op=False, config=None, workspace=None,
                          **kwargs):
        """output = all_gather(A @ B + bias[:, None]) along rows."""
        return matmul_all_gather(self._shmem, output_tensor, A, B, bias, async_op, config, workspace, **kwargs)

    def matmul_reduce_scatter(self, output_tensor, A, B, bias=None, async_op=False, config=None, workspace=None,
                              **kwargs):
        """output = reduce_scatter(A @ B).  `bias` is accepted and ignored.  (The reference forwards
        `bias` as a surplus positional argument here, which raises TypeError; this does not.)"""
        return matmul_reduce_scatter(self._shmem, output_tensor, A, B, async_op, config, workspace, **kwargs)


__all__ = [
    "FusedConfig",
    "FusedWorkspace",
    "OpsNamespace",
    "matmul_all_reduce",
    "matmul_all_reduce_preamble",
    "all_gather_matmul",
    "all_gather_matmul_preamble",
    "matmul_all_gather",
    "matmul_all_gather_preamble",
    "matmul_reduce_scatter",
    "matmul_reduce_scatter_preamble",
]
