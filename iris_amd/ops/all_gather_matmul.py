"""Fused out = all_gather(A_sharded) @ B (+ bias): the work of one rank, pull pattern.

Same call contract as iris/ops/all_gather_matmul.py:162-305 of the reference: every rank holds an
(M, K_local) column block of A at the same heap offset, B is (K, N) with K = W * K_local, and the
kernel reads the A tiles straight out of the owners' heaps while it multiplies.
"""

import logging
from typing import Optional

import torch

from .. import _lib
from ..host.logging import debug_on, log_rank
from ._common import current_stream, dtype_code, iris_launch, is_fp8, path_code, ptr, require_gpu_tensors
from .config import FusedConfig
from .workspace import FusedWorkspace


def all_gather_matmul_preamble(
    shmem,
    A_sharded: torch.Tensor,
    B: torch.Tensor,
    config: Optional[FusedConfig] = None,
    *,
    gather_dim: int = 1,
) -> FusedWorkspace:
    """The pull pattern needs no buffers; this only checks shapes and returns a prepared workspace."""
    if config is None:
        config = FusedConfig()
    world_size = shmem.get_num_ranks()
    K, N = B.shape
    if gather_dim == 1:
        M, K_local = A_sharded.shape
        expected_K = world_size * K_local
        assert K == expected_K, f"K ({K}) must equal world_size ({world_size}) * K_local ({K_local})"
    else:
        M_local, K_a = A_sharded.shape
        assert K == K_a, f"K ({K}) must equal A_sharded.shape[1] ({K_a}) when gathering rows"
        M = M_local * world_size
    return FusedWorkspace(
        operation="all_gather_matmul",
        shape=(M, N, K),
        dtype=A_sharded.dtype,
        world_size=world_size,
        prepared=True,
    )


def all_gather_matmul(
    shmem,
    output_tensor: torch.Tensor,
    A_sharded: torch.Tensor,
    B: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    async_op: bool = False,
    config: Optional[FusedConfig] = None,
    workspace: Optional[FusedWorkspace] = None,
    *,
    gather_dim: int = 1,
    scale_a: Optional[float] = None,
    scale_b: Optional[float] = None,
    kernel_path: str = "auto",
) -> FusedWorkspace:
    """out = all_gather(A_sharded) @ B, plus `bias[:, None]` when a length-M bias is given.

    Keyword-only additions to the reference signature:
        gather_dim: 1 (default, the reference layout) gathers columns: A_sharded is (M, K_local) and
            the reduction runs over rank 0's columns, then rank 1's, ....  0 gathers rows:
            A_sharded is (M / W, K) and output rows [r*M/W, (r+1)*M/W) use rank r's shard.
        scale_a, scale_b, kernel_path: as for matmul_all_reduce.
    """
    if config is None:
        config = FusedConfig()
    if gather_dim not in (0, 1):
        raise ValueError(f"gather_dim must be 0 (rows) or 1 (columns), got {gather_dim}")
    world_size = shmem.get_num_ranks()
    rank = shmem.get_rank()
    K, N = B.shape
    if gather_dim == 1:
        M, K_local = A_sharded.shape
    else:
        M_local, K_local = A_sharded.shape
        M = M_local * world_size
    if debug_on():
        log_rank(logging.DEBUG, "all_gather_matmul: shape=(%d,%d,%d) dtype=%s rank=%d/%d", M, N, K, A_sharded.dtype, rank,
                 world_size, rank=rank, num_ranks=world_size)

    if gather_dim == 1:
        expected_K = world_size * K_local
        assert K == expected_K, f"K ({K}) must equal world_size ({world_size}) * K_local ({K_local})"
    else:
        assert K == K_local, f"K ({K}) must equal A_sharded.shape[1] ({K_local}) when gathering rows"
    assert output_tensor.shape == (M, N), f"Output must be ({M}, {N}), got {output_tensor.shape}"
    rows_checked = M if gather_dim == 1 else M // world_size
    assert rows_checked >= config.block_size_m, (
        f"M ({rows_checked}) must be >= block_size_m ({config.block_size_m}). Use smaller block sizes for small problems."
    )
    assert K_local >= config.block_size_k, (
        f"K_local ({K_local}) must be >= block_size_k ({config.block_size_k}). "
        f"Use smaller block sizes for small problems."
    )
    assert N >= config.block_size_n, (
        f"N ({N}) must be >= block_size_n ({config.block_size_n}). Use smaller block sizes for small problems."
    )
    if is_fp8(A_sharded.dtype):
        if B.dtype != A_sharded.dtype or output_tensor.dtype not in (torch.bfloat16, torch.float16):
            raise ValueError("float8 inputs need a float8 B and a bfloat16/float16 output")
    elif B.dtype != A_sharded.dtype or output_tensor.dtype != A_sharded.dtype:
        raise ValueError(
            f"All tensors must have same dtype, got A:{A_sharded.dtype}, B:{B.dtype}, C:{output_tensor.dtype}"
        )
    if not shmem.is_symmetric(A_sharded):
        raise RuntimeError("A_sharded must be allocated on the symmetric heap (the peers' shards are read by offset)")

    if workspace is None:
        workspace = all_gather_matmul_preamble(shmem, A_sharded, B, config, gather_dim=gather_dim)

    stride_am, stride_ak = A_sharded.stride()
    stride_bk, stride_bn = B.stride()
    stride_cm, stride_cn = output_tensor.stride()
    if bias is not None:
        assert bias.shape[0] == M
        stride_bias = bias.stride()[0] if bias.dim() > 0 else 1
        bias_code = dtype_code(bias.dtype)
    else:
        stride_bias = 1
        bias_code = _lib.FP32

    scale = 1.0
    if is_fp8(A_sharded.dtype):
        scale = float(1.0 if scale_a is None else scale_a) * float(1.0 if scale_b is None else scale_b)
    elif scale_a is not None or scale_b is not None:
        raise ValueError("scale_a / scale_b only apply to float8 inputs")

    path = path_code(kernel_path)
    require_gpu_tensors(shmem, A_sharded=A_sharded, B=B, output_tensor=output_tensor, bias=bias)
    num_sms = config.num_sms if config.num_sms is not None else shmem.get_cu_count()
    iris_launch(
        "iris_hip_all_gather_matmul",
        (num_sms,),
        ptr(A_sharded), ptr(B), ptr(output_tensor), ptr(bias),
        M, N, K, K_local,
        stride_am, stride_ak, stride_bk, stride_bn, stride_cm, stride_cn, stride_bias,
        ptr(shmem.get_device_context()), rank, world_size,
        config.block_size_m, config.block_size_n, config.block_size_k,
        _lib.GATHER_K if gather_dim == 1 else _lib.GATHER_M,
        dtype_code(A_sharded.dtype), dtype_code(output_tensor.dtype), bias_code, scale,
        path, current_stream(shmem),
        algorithm="all_gather_matmul",
        rank=rank,
        dtype=A_sharded.dtype,
    )
    if not async_op:
        shmem.barrier()
    return workspace
