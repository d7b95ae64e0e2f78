"""Fused C = all_reduce(A @ B): the work of one rank.

Same call contract as iris/ops/matmul_all_reduce.py:147-372 of the reference (signatures, checks,
error classes and messages, workspace handling, barrier unless async_op).  The Triton kernel launch
is replaced by one call into libiris_hip.so.
"""

import logging
from typing import Optional

import torch

from .. import _lib
from ..host.logging import debug_on, log_rank
from ._common import (acc_code, current_stream, dtype_code, iris_launch, is_fp8, path_code, ptr,
                      require_gpu_tensors, stage_idle_peers)
from .config import FusedConfig
from .workspace import FusedWorkspace

_VARIANT_CODES = {"atomic": _lib.VARIANT_ATOMIC, "one_shot": _lib.VARIANT_ONE_SHOT, "two_shot": _lib.VARIANT_TWO_SHOT}


def _tile_count(M, N, config):
    num_pid_m = (M + config.block_size_m - 1) // config.block_size_m
    num_pid_n = (N + config.block_size_n - 1) // config.block_size_n
    return num_pid_m * num_pid_n


def matmul_all_reduce_preamble(
    shmem,
    C: torch.Tensor,
    A: torch.Tensor,
    B: torch.Tensor,
    config: Optional[FusedConfig] = None,
    workspace: Optional[FusedWorkspace] = None,
) -> FusedWorkspace:
    """Allocate (or reset) the flag array and the aux buffer on the symmetric heap, zero C, barrier.

    One int32 flag per block_size_m x block_size_n tile; aux has C's shape and dtype.
    """
    if config is None:
        config = FusedConfig()
    M, K = A.shape[:2]
    N = B.shape[1]
    world_size = shmem.get_num_ranks()
    config.validate(world_size=world_size)
    if workspace is None:
        workspace = FusedWorkspace()
    workspace.operation = "matmul_all_reduce"
    workspace.shape = (M, N, K)
    workspace.dtype = A.dtype
    workspace.world_size = world_size
    workspace.variant = config.all_reduce_variant
    workspace.prepared = False

    total_tiles = _tile_count(M, N, config)
    if config.all_reduce_variant in ["spinlock", "one_shot", "two_shot"]:
        if workspace.locks is None or workspace.locks.numel() != total_tiles:
            workspace.locks = shmem.zeros((total_tiles,), dtype=torch.int32)
        else:
            workspace.locks.zero_()
    else:
        workspace.locks = None
    if config.all_reduce_variant in ["one_shot", "two_shot"]:
        if workspace.aux_buffer is None or workspace.aux_buffer.shape != (M, N):
            workspace.aux_buffer = shmem.zeros((M, N), dtype=C.dtype)
        else:
            workspace.aux_buffer.zero_()
    else:
        workspace.aux_buffer = None

    C.zero_()
    stage_idle_peers(shmem, workspace)
    shmem.barrier()
    workspace.prepared = True
    return workspace


def matmul_all_reduce(
    shmem,
    C: torch.Tensor,
    A: torch.Tensor,
    B: torch.Tensor,
    async_op: bool = False,
    config: Optional[FusedConfig] = None,
    workspace: Optional[FusedWorkspace] = None,
    *,
    scale_a: Optional[float] = None,
    scale_b: Optional[float] = None,
    slot_sum: str = "fp32",
    kernel_path: str = "auto",
) -> FusedWorkspace:
    """C = all_reduce(A @ B) for this rank; returns the workspace (reusable on the next call).

    A is (M, K), different on every rank; B is (K, N), replicated; C is (M, N).  With variant
    "atomic" the rank's product is added atomically into every rank's C (which the preamble zeroed);
    with "one_shot" this rank sums every tile of its own product with the peers' tiles (read from their
    aux buffers once their flags are up) into its own C; with "two_shot" it does so only for the
    tiles t with t % world_size == rank and writes the result into every rank's C.

    Keyword-only additions to the reference signature:
        scale_a, scale_b: per-tensor dequantisation scales for float8_e4m3fn inputs (C is bfloat16
            or float16 then); the fp32 product is multiplied by scale_a * scale_b before the cast.
        slot_sum: "fp32" carries the sum over ranks in fp32 and casts once; "reference" follows the
            reference rule (fp32 only for float16 data, otherwise the data type after every add).
        kernel_path: "auto", "mfma" or "generic".
    """
    if config is None:
        config = FusedConfig()
    if A.ndim != 2 or B.ndim != 2:
        raise ValueError(f"A and B must be 2D tensors, got shapes {A.shape} and {B.shape}")
    M, K = A.shape
    K_B, N = B.shape
    if K != K_B:
        raise ValueError(
            f"Incompatible matrix dimensions: A is ({M}, {K}), B is ({K_B}, {N}). "
            f"Inner dimensions must match (K={K} != K_B={K_B})"
        )
    if C.shape != (M, N):
        raise ValueError(f"Output tensor shape {C.shape} doesn't match expected ({M}, {N})")
    if is_fp8(A.dtype):
        if A.dtype != B.dtype or C.dtype not in (torch.bfloat16, torch.float16):
            raise ValueError(f"float8 inputs need a bfloat16/float16 output, got A:{A.dtype}, B:{B.dtype}, C:{C.dtype}")
    elif A.dtype != B.dtype or A.dtype != C.dtype:
        raise ValueError(f"All tensors must have same dtype, got A:{A.dtype}, B:{B.dtype}, C:{C.dtype}")
    assert M >= config.block_size_m, f"M={M} too small for block_size_m={config.block_size_m}"
    assert K >= config.block_size_k, f"K={K} too small for block_size_k={config.block_size_k}"
    assert N >= config.block_size_n, f"N={N} too small for block_size_n={config.block_size_n}"

    stride_am, stride_ak = A.stride()
    stride_bk, stride_bn = B.stride()
    stride_cm, stride_cn = C.stride()
    rank = shmem.get_rank()
    world_size = shmem.get_num_ranks()
    if debug_on():
        log_rank(logging.DEBUG, "matmul_all_reduce: shape=(%d,%d,%d) dtype=%s variant=%s rank=%d/%d", M, N, K, A.dtype,
                 config.all_reduce_variant, rank, world_size, rank=rank, num_ranks=world_size)
    if config.all_reduce_variant not in _VARIANT_CODES:
        config.validate(world_size=world_size)
        raise NotImplementedError(
            f"all_reduce_variant {config.all_reduce_variant!r} has no HIP kernel; use 'atomic', 'one_shot' or 'two_shot'"
        )
    needs_prepare = workspace is None or not workspace.matches(
        "matmul_all_reduce", (M, N, K), A.dtype, world_size, config.all_reduce_variant
    )
    if needs_prepare:
        workspace = matmul_all_reduce_preamble(shmem, C, A, B, config=config, workspace=workspace)

    device_context = shmem.get_device_context()
    total_tiles = _tile_count(M, N, config)
    grid = (total_tiles,)
    if workspace.locks is not None and workspace.locks.numel() < total_tiles:
        raise ValueError(
            f"Lock array too small: have {workspace.locks.numel()} but need {total_tiles}. "
            f"Pre-allocate workspace with the smallest block sizes you intend to use."
        )
    if config.all_reduce_variant == "atomic":
        if not shmem.is_symmetric(C):
            raise RuntimeError("C must be allocated on the symmetric heap (every rank's copy is added to)")
    else:
        if workspace.aux_buffer is None or workspace.locks is None:
            raise ValueError("workspace has no aux buffer / locks for the one_shot / two_shot variants")
        if workspace.aux_buffer.dtype != C.dtype:
            raise ValueError(f"workspace aux buffer has dtype {workspace.aux_buffer.dtype}, C has {C.dtype}")
        # aux is addressed with C's strides, as in the reference kernel.
        if (M - 1) * stride_cm + (N - 1) * stride_cn >= workspace.aux_buffer.numel():
            raise ValueError("C's strides address beyond the aux buffer")

    scale = 1.0
    if is_fp8(A.dtype):
        scale = float(1.0 if scale_a is None else scale_a) * float(1.0 if scale_b is None else scale_b)
    elif scale_a is not None or scale_b is not None:
        raise ValueError("scale_a / scale_b only apply to float8 inputs")

    acc, path = acc_code(slot_sum), path_code(kernel_path)
    require_gpu_tensors(shmem, A=A, B=B, C=C)
    iris_launch(
        "iris_hip_matmul_all_reduce",
        grid,
        ptr(A), ptr(B), ptr(C), ptr(workspace.aux_buffer), ptr(workspace.locks),
        M, N, K,
        stride_am, stride_ak, stride_bk, stride_bn, stride_cm, stride_cn,
        ptr(device_context), rank, world_size,
        config.block_size_m, config.block_size_n, config.block_size_k,
        _VARIANT_CODES[config.all_reduce_variant],
        dtype_code(A.dtype), dtype_code(C.dtype), scale, acc,
        shmem.spin_limit, ptr(shmem._status), path, current_stream(shmem),
        algorithm="matmul_all_reduce",
        rank=rank,
        dtype=A.dtype,
    )

    if workspace is not None:
        workspace.prepared = False
    if not async_op:
        shmem.barrier()
    return workspace
