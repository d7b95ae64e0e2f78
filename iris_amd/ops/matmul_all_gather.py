"""Fused out = all_gather(A @ B + bias) along rows: the work of one rank, scatter pattern.

Same call contract as iris/ops/matmul_all_gather.py:108-276 of the reference: every rank multiplies
its (M_local, K) block by the replicated B and writes the product tile into rows
[rank * M_local, (rank + 1) * M_local) of the (M, N) output of EVERY rank.
"""

import logging
from typing import Optional

import torch

from .. import _lib
from ..host.logging import debug_on, log_rank
from ._common import current_stream, dtype_code, iris_launch, is_fp8, path_code, ptr, require_gpu_tensors
from .config import FusedConfig
from .workspace import FusedWorkspace


def matmul_all_gather_preamble(
    shmem,
    A: torch.Tensor,
    B: torch.Tensor,
    config: Optional[FusedConfig] = None,
) -> FusedWorkspace:
    """No buffers are needed (tiles go straight to the destination heaps); checks shapes only."""
    if config is None:
        config = FusedConfig()
    M_local, K = A.shape
    K2, N = B.shape
    world_size = shmem.get_num_ranks()
    assert K == K2, f"Inner dimensions must match: A has K={K}, B has K={K2}"
    return FusedWorkspace(
        operation="matmul_all_gather",
        shape=(M_local * world_size, N, K),
        dtype=A.dtype,
        world_size=world_size,
        prepared=True,
    )


def matmul_all_gather(
    shmem,
    output_tensor: torch.Tensor,
    A: torch.Tensor,
    B: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    async_op: bool = False,
    config: Optional[FusedConfig] = None,
    workspace: Optional[FusedWorkspace] = None,
    *,
    scale_a: Optional[float] = None,
    scale_b: Optional[float] = None,
    kernel_path: str = "auto",
) -> FusedWorkspace:
    """output[rank*M_local:(rank+1)*M_local] = A @ B (+ bias[:, None]) on every rank's output.

    output_tensor is (M, N) with M = M_local * world_size and must live on the symmetric heap;
    bias, if given, has M_local elements.  scale_a / scale_b / kernel_path: as for matmul_all_reduce.
    """
    if config is None:
        config = FusedConfig()
    M_local, K = A.shape
    K2, N = B.shape
    world_size = shmem.get_num_ranks()
    rank = shmem.get_rank()
    if debug_on():
        log_rank(logging.DEBUG, "matmul_all_gather: shape=(%d,%d,%d) dtype=%s rank=%d/%d", M_local * world_size, N, K,
                 A.dtype, rank, world_size, rank=rank, num_ranks=world_size)
    assert K == K2, f"Inner dimensions must match: A has K={K}, B has K={K2}"
    M = M_local * world_size
    assert output_tensor.shape == (M, N), f"Output must be ({M}, {N}), got {output_tensor.shape}"
    assert M_local >= config.block_size_m, (
        f"M_local ({M_local}) must be >= block_size_m ({config.block_size_m}). "
        f"Use smaller block sizes for small problems."
    )
    assert K >= config.block_size_k, (
        f"K ({K}) must be >= block_size_k ({config.block_size_k}). Use smaller block sizes for small problems."
    )
    assert N >= config.block_size_n, (
        f"N ({N}) must be >= block_size_n ({config.block_size_n}). Use smaller block sizes for small problems."
    )
    if is_fp8(A.dtype):
        if B.dtype != A.dtype or output_tensor.dtype not in (torch.bfloat16, torch.float16):
            raise ValueError("float8 inputs need a float8 B and a bfloat16/float16 output")
    elif B.dtype != A.dtype or output_tensor.dtype != A.dtype:
        raise ValueError(f"All tensors must have same dtype, got A:{A.dtype}, B:{B.dtype}, C:{output_tensor.dtype}")
    if not shmem.is_symmetric(output_tensor):
        raise RuntimeError("output_tensor must be allocated on the symmetric heap (every rank's copy is written)")
    if workspace is None:
        workspace = matmul_all_gather_preamble(shmem, A, B, config)

    stride_am, stride_ak = A.stride()
    stride_bk, stride_bn = B.stride()
    stride_cm, stride_cn = output_tensor.stride()
    if bias is not None:
        assert bias.shape[0] == M_local
        stride_bias = bias.stride()[0] if bias.dim() > 0 else 1
        bias_code = dtype_code(bias.dtype)
    else:
        stride_bias = 1
        bias_code = _lib.FP32
    scale = 1.0
    if is_fp8(A.dtype):
        scale = float(1.0 if scale_a is None else scale_a) * float(1.0 if scale_b is None else scale_b)
    elif scale_a is not None or scale_b is not None:
        raise ValueError("scale_a / scale_b only apply to float8 inputs")
    path = path_code(kernel_path)
    require_gpu_tensors(shmem, A=A, B=B, output_tensor=output_tensor, bias=bias)
    num_sms = config.num_sms if config.num_sms is not None else shmem.get_cu_count()
    iris_launch(
        "iris_hip_matmul_all_gather",
        (num_sms,),
        ptr(A), ptr(B), ptr(output_tensor), ptr(bias),
        M_local, M, N, K,
        stride_am, stride_ak, stride_bk, stride_bn, stride_cm, stride_cn, stride_bias,
        ptr(shmem.get_device_context()), rank, world_size,
        config.block_size_m, config.block_size_n, config.block_size_k,
        dtype_code(A.dtype), dtype_code(output_tensor.dtype), bias_code, scale,
        path, current_stream(shmem),
        algorithm="matmul_all_gather",
        rank=rank,
        dtype=A.dtype,
    )
    if not async_op:
        shmem.barrier()
    return workspace
