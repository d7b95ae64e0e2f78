"""Reduce-scatter over the symmetric heap: the rank reduces the tiles assigned to it and keeps them.

Call contract of iris/ccl/reduce_scatter.py:13-73 and the launch in
iris/ccl/triton/reduce_scatter.py:143-192.
"""

import logging

from ..host.logging import debug_on, log_rank
from ..ops._common import current_stream, dtype_code, iris_launch, require_gpu_tensors
from .all_reduce import _check_tensors, _launch_head
from .config import Config
from .utils import ReduceOp


def reduce_scatter(output_tensor, input_tensor, ctx, op=None, group=None, async_op=False, config=None):
    """output (M, N), own copy only: the tiles config.all_reduce_distribution assigns to this rank hold
    the sum over the group of input; other tiles are left untouched."""
    if op is None:
        op = ReduceOp.SUM
    if op != ReduceOp.SUM:
        raise ValueError(
            f"Only ReduceOp.SUM is currently supported, got {op}. "
            "Support for other operations will be added in a future release."
        )
    if config is None:
        config = Config(block_size_m=32, block_size_n=64, all_reduce_distribution=1)
    if config.use_gluon:
        raise ValueError(
            "reduce_scatter does not support use_gluon=True. "
            "Gluon implementation is not available for reduce_scatter. "
            "Use default config (use_gluon=False)."
        )
    variant = getattr(config, "reduce_scatter_variant", "two_shot")
    if variant != "two_shot":
        raise ValueError(f"reduce_scatter only supports variant='two_shot', got '{variant}'.")
    _check_tensors(ctx, output_tensor, input_tensor)
    M, N = input_tensor.shape[:2]
    if tuple(output_tensor.shape[:2]) != (M, N):
        raise ValueError(
            f"Output tensor shape {tuple(output_tensor.shape[:2])} does not match input shape {(M, N)}. "
            f"For reduce-scatter, output should have the same shape as input."
        )
    code = dtype_code(input_tensor.dtype)
    head, rank_global = _launch_head(ctx, output_tensor, input_tensor, config, group)
    if debug_on():
        log_rank(logging.DEBUG, "ccl.reduce_scatter: shape=(%d,%d) dtype=%s", M, N, input_tensor.dtype,
                 rank=rank_global, num_ranks=ctx.get_num_ranks())
    require_gpu_tensors(ctx, input_tensor=input_tensor, output_tensor=output_tensor)
    iris_launch(
        "iris_hip_reduce_scatter", (config.comm_sms,), *head,
        config.all_reduce_distribution, code, current_stream(ctx),
        algorithm="reduce_scatter", rank=rank_global, dtype=input_tensor.dtype,
    )
    if not async_op:
        ctx.barrier()
