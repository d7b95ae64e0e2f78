"""All-reduce over the symmetric heap: output = sum of the group's inputs, the work of one rank.

Call contract of iris/ccl/all_reduce.py:18-81 and iris/ccl/triton/all_reduce.py:25-117 (workspace and
preamble), :708-956 (launch).  Variants with a HIP kernel: "one_shot", "two_shot", "atomic".
"ring" and "spinlock" pass tiles from rank to rank or serialise ranks through locks; one GPU playing
all ranks in turn cannot run them and they raise NotImplementedError.
"""

import logging
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from .. import _lib
from ..host.logging import debug_on, log_rank
from ..ops._common import current_stream, dtype_code, iris_launch, ptr, require_gpu_tensors
from .config import Config
from .utils import ReduceOp, extract_group_info

_VALID_VARIANTS = ["atomic", "spinlock", "ring", "two_shot", "one_shot"]
_VARIANT_CODES = {"atomic": _lib.VARIANT_ATOMIC, "one_shot": _lib.VARIANT_ONE_SHOT, "two_shot": _lib.VARIANT_TWO_SHOT}


@dataclass
class AllReduceWorkspace:
    """What a call keeps between invocations (iris/ccl/triton/all_reduce.py:25-49).  The variants built
    here need no buffers; ring_buffer, flags and locks stay None."""

    variant: str = ""
    shape: Tuple[int, int] = ()
    dtype: Optional[torch.dtype] = None
    ring_buffer: Optional[torch.Tensor] = None
    flags: Optional[torch.Tensor] = None
    locks: Optional[torch.Tensor] = None
    num_rings: int = 1
    flags_per_tile: int = 0
    prepared: bool = False


def _check_variant(variant):
    if variant not in _VALID_VARIANTS:
        raise ValueError(f"Invalid all_reduce_variant: {variant}. Must be one of: {', '.join(_VALID_VARIANTS)}")
    if variant not in _VARIANT_CODES:
        raise NotImplementedError(
            f"all_reduce_variant {variant!r} has no HIP kernel; use 'atomic', 'one_shot' or 'two_shot'"
        )


def all_reduce_preamble(output_tensor, input_tensor, ctx, config=None, workspace=None):
    """Reset what the variant needs reset: atomic and one_shot zero the output and meet at a barrier,
    two_shot does nothing (iris/ccl/triton/all_reduce.py:83-85,109-110)."""
    if config is None:
        config = Config()
    variant = config.all_reduce_variant.lower()
    _check_variant(variant)
    M, N = input_tensor.shape[:2]
    if workspace is None:
        workspace = AllReduceWorkspace()
    workspace.variant = variant
    workspace.shape = (M, N)
    workspace.dtype = input_tensor.dtype
    workspace.num_rings = getattr(config, "all_reduce_num_rings", 1)
    workspace.prepared = False
    if variant in ("atomic", "one_shot"):
        output_tensor.zero_()
        ctx.barrier()
    workspace.prepared = True
    return workspace


def _check_tensors(ctx, output_tensor, input_tensor):
    if input_tensor.dim() != 2 or output_tensor.dim() != 2:
        raise ValueError(f"input and output must be 2-D, got {tuple(input_tensor.shape)} and {tuple(output_tensor.shape)}")
    if output_tensor.dtype != input_tensor.dtype:
        raise ValueError(f"input and output must have the same dtype, got {input_tensor.dtype} and {output_tensor.dtype}")
    if not ctx.is_symmetric(input_tensor):
        raise RuntimeError("input_tensor must be allocated on the symmetric heap (the peers' copies are read)")


def _launch_head(ctx, output_tensor, input_tensor, config, group):
    rank_in_group, rank_global, world_size, rank_start, rank_stride = extract_group_info(group, ctx)
    M, N = input_tensor.shape[:2]
    head = (
        ptr(input_tensor), ptr(output_tensor), M, N,
        input_tensor.stride(0), input_tensor.stride(1), output_tensor.stride(0), output_tensor.stride(1),
        ptr(ctx.get_heap_bases()), rank_in_group, rank_global, world_size, rank_start, rank_stride,
        config.block_size_m, config.block_size_n, config.swizzle_size, config.comm_sms, config.num_xcds,
        config.chunk_size,
    )
    return head, rank_global


def all_reduce(output_tensor, input_tensor, ctx, op=None, group=None, async_op=False, config=None, workspace=None):
    """All-reduce: the calling rank's share of output = sum over the group of input.

    output_tensor, input_tensor: (M, N) tensors of one dtype (bfloat16, float16 or float32); the input
    must be on the symmetric heap, and so must the output for "two_shot" and "atomic", which write the
    peers' outputs.  op: only ReduceOp.SUM.  group: None, a ProcessGroup, or a list of ranks.
    async_op=False ends with ctx.barrier().  Returns the workspace with prepared=False, as the
    reference does.
    """
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
            "all_reduce does not support use_gluon=True. "
            "Gluon implementation is not available for all_reduce. "
            "Use default config (use_gluon=False)."
        )
    variant = config.all_reduce_variant.lower()
    _check_variant(variant)
    _check_tensors(ctx, output_tensor, input_tensor)
    M, N = input_tensor.shape[:2]
    if tuple(output_tensor.shape[:2]) != (M, N):
        raise ValueError(f"Output tensor shape {tuple(output_tensor.shape[:2])} does not match input shape {(M, N)}.")
    if variant != "one_shot" and not ctx.is_symmetric(output_tensor):
        raise RuntimeError("output_tensor must be allocated on the symmetric heap (every rank's copy is written)")
    code = dtype_code(input_tensor.dtype)

    needs_prepare = (
        workspace is None
        or not getattr(workspace, "prepared", False)
        or workspace.variant != variant
        or workspace.shape != (M, N)
        or workspace.dtype != input_tensor.dtype
    )
    if needs_prepare:
        workspace = all_reduce_preamble(output_tensor, input_tensor, ctx, config=config, workspace=workspace)

    head, rank_global = _launch_head(ctx, output_tensor, input_tensor, config, group)
    if debug_on():
        log_rank(logging.DEBUG, "ccl.all_reduce: shape=(%d,%d) dtype=%s variant=%s", M, N, input_tensor.dtype, variant,
                 rank=rank_global, num_ranks=ctx.get_num_ranks())
    require_gpu_tensors(ctx, input_tensor=input_tensor, output_tensor=output_tensor)
    iris_launch(
        "iris_hip_all_reduce", (config.comm_sms,), *head,
        _VARIANT_CODES[variant], config.all_reduce_distribution, code, current_stream(ctx),
        algorithm="all_reduce", rank=rank_global, dtype=input_tensor.dtype,
    )
    if workspace is not None:
        workspace.prepared = False
    if not async_op:
        ctx.barrier()
    return workspace
