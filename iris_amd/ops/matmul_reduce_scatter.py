"""Fused C = reduce_scatter(A @ B): the work of one rank.

Same call contract as iris/ops/matmul_reduce_scatter.py:121-294 of the reference.  Every rank
computes the whole product into its aux buffer and raises a flag per tile; tile t is then reduced by
rank min(t // (tiles // W), W - 1), which stores the sum into its own C at the tile's coordinates.
"""

import logging
from typing import Optional

import torch

from ..host.logging import debug_on, log_rank
from ._common import (acc_code, current_stream, dtype_code, iris_launch, is_fp8, path_code, ptr,
                      require_gpu_tensors, stage_idle_peers)
from .config import FusedConfig
from .workspace import FusedWorkspace


def _tile_count(M, N, config):
    num_pid_m = (M + config.block_size_m - 1) // config.block_size_m
    num_pid_n = (N + config.block_size_n - 1) // config.block_size_n
    return num_pid_m * num_pid_n


def _too_small(have, need):
    return ValueError(
        f"Lock array too small: have {have} but need {need}. "
        f"Pre-allocate workspace with the smallest block sizes you intend to use."
    )


def matmul_reduce_scatter_preamble(
    shmem,
    C: torch.Tensor,
    A: torch.Tensor,
    B: torch.Tensor,
    config: Optional[FusedConfig] = None,
    workspace: Optional[FusedWorkspace] = None,
) -> FusedWorkspace:
    """Allocate (or reset) flags and aux, zero C, barrier.  A workspace whose flag array is smaller
    than the tile count of `config` is rejected with ValueError."""
    if config is None:
        config = FusedConfig()
    M, K = A.shape[:2]
    N = B.shape[1]
    world_size = shmem.get_num_ranks()
    config.validate(world_size=world_size)
    if workspace is None:
        workspace = FusedWorkspace()
    workspace.operation = "matmul_reduce_scatter"
    workspace.shape = (M, N, K)
    workspace.dtype = A.dtype
    workspace.world_size = world_size
    workspace.variant = "two_shot"
    workspace.prepared = False

    total_tiles = _tile_count(M, N, config)
    if workspace.locks is not None and workspace.locks.numel() < total_tiles:
        raise _too_small(workspace.locks.numel(), total_tiles)
    if workspace.locks is None or workspace.locks.numel() != total_tiles:
        workspace.locks = shmem.zeros((total_tiles,), dtype=torch.int32)
    else:
        workspace.locks.zero_()
    if workspace.aux_buffer is None or workspace.aux_buffer.shape != (M, N):
        workspace.aux_buffer = shmem.zeros((M, N), dtype=C.dtype)
    else:
        workspace.aux_buffer.zero_()
    C.zero_()
    stage_idle_peers(shmem, workspace)
    shmem.barrier()
    workspace.prepared = True
    return workspace


def matmul_reduce_scatter(
    shmem,
    C: torch.Tensor,
    A: torch.Tensor,
    B: torch.Tensor,
    async_op: bool = False,
    config: Optional[FusedConfig] = None,
    workspace: Optional[FusedWorkspace] = None,
    *,
    all_owners: bool = False,
    sum_peers: bool = True,
    scale_a: Optional[float] = None,
    scale_b: Optional[float] = None,
    slot_sum: str = "fp32",
    kernel_path: str = "auto",
    stage=None,
) -> FusedWorkspace:
    """C = reduce_scatter(A @ B) for this rank: C holds the reduced tiles this rank owns.

    Keyword-only additions to the reference signature:
        all_owners: one GPU stands in for every rank's reduce step: each tile t is reduced and stored
            into C of slot owner(t) (with the default 256 x 64 tiles, contiguous row blocks per slot).
        sum_peers: if False, the peers contribute nothing (their flags and aux are not read).
        stage: optional callable `stage(workspace)` run after the preamble (which zeroes the
            workspace on every call) and before the launch - the place to write peers' partial
            results and flags into the other slots when one GPU plays all ranks.
        scale_a, scale_b, slot_sum, kernel_path: as for matmul_all_reduce.
    """
    if config is None:
        config = FusedConfig()
    if A.ndim != 2 or B.ndim != 2:
        raise ValueError(f"A and B must be 2D tensors, got shapes {A.shape} and {B.shape}")
    if A.shape[1] != B.shape[0]:
        raise ValueError(f"Incompatible matrix dimensions: A is {tuple(A.shape)}, B is {tuple(B.shape)}")
    if C.shape != (A.shape[0], B.shape[1]):
        raise ValueError(f"Output tensor shape {C.shape} doesn't match expected ({A.shape[0]}, {B.shape[1]})")
    if is_fp8(A.dtype):
        if A.dtype != B.dtype or C.dtype not in (torch.bfloat16, torch.float16):
            raise ValueError(f"float8 inputs need a bfloat16/float16 output, got A:{A.dtype}, B:{B.dtype}, C:{C.dtype}")
    elif A.dtype != B.dtype or A.dtype != C.dtype:
        raise ValueError(f"All tensors must have same dtype, got A:{A.dtype}, B:{B.dtype}, C:{C.dtype}")
    workspace = matmul_reduce_scatter_preamble(shmem, C, A, B, config, workspace)
    if stage is not None:
        stage(workspace)

    M, K = A.shape[:2]
    N = B.shape[1]
    rank = shmem.get_rank()
    world_size = shmem.get_num_ranks()
    if debug_on():
        log_rank(logging.DEBUG, "matmul_reduce_scatter: shape=(%d,%d,%d) dtype=%s rank=%d/%d", M, N, K, A.dtype, rank,
                 world_size, rank=rank, num_ranks=world_size)

    total_tiles = _tile_count(M, N, config)
    if workspace.locks is not None and workspace.locks.numel() < total_tiles:
        raise _too_small(workspace.locks.numel(), total_tiles)
    grid = (total_tiles,)
    if (M - 1) * C.stride(0) + (N - 1) * C.stride(1) >= workspace.aux_buffer.numel():
        raise ValueError("C's strides address beyond the aux buffer")

    scale = 1.0
    if is_fp8(A.dtype):
        scale = float(1.0 if scale_a is None else scale_a) * float(1.0 if scale_b is None else scale_b)
    elif scale_a is not None or scale_b is not None:
        raise ValueError("scale_a / scale_b only apply to float8 inputs")

    acc, path = acc_code(slot_sum), path_code(kernel_path)
    require_gpu_tensors(shmem, A=A, B=B, C=C)
    iris_launch(
        "iris_hip_matmul_reduce_scatter",
        grid,
        ptr(A), ptr(B), ptr(C), ptr(workspace.aux_buffer), ptr(workspace.locks),
        M, N, K,
        A.stride(0), A.stride(1), B.stride(0), B.stride(1), C.stride(0), C.stride(1),
        ptr(shmem.get_device_context()), rank, world_size,
        config.block_size_m, config.block_size_n, config.block_size_k,
        int(bool(all_owners)), int(bool(sum_peers)),
        dtype_code(A.dtype), dtype_code(C.dtype), scale, acc,
        shmem.spin_limit, ptr(shmem._status), path, current_stream(shmem),
        algorithm="matmul_reduce_scatter",
        rank=rank,
        dtype=A.dtype,
    )

    if not async_op:
        torch.cuda.synchronize()
        shmem.barrier()
    return workspace
