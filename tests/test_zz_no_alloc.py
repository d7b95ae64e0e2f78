"""The entry point that allocates nothing (iris_hip_matmul_all_reduce_noalloc), through the C ABI,
against iris_hip_matmul_all_reduce with a caller-owned workspace at world size 1: same kernels, so
every output bit must agree.  Two calls in a row on the same GPU, the second with a smaller input (the
library's workspace keeps the first call's contents)."""

import ctypes

import pytest
import torch

import iris_amd as iris
from iris_amd import _lib, ops
from helpers import assert_bits_equal, heap_tensor, randn_cpu

pytestmark = pytest.mark.gpu

CODES = {torch.bfloat16: _lib.BF16, torch.float16: _lib.FP16, torch.float32: _lib.FP32}


def _reference(A, B, cfg):
    """C of the existing entry point (workspace on the symmetric heap), W = 1."""
    ctx = iris.iris(1 << 27, num_ranks=1, rank=0)
    dA, dB = heap_tensor(ctx, A), heap_tensor(ctx, B)
    dC = ctx.zeros((A.shape[0], B.shape[1]), dtype=A.dtype)
    ops.matmul_all_reduce(ctx, dC, dA, dB, config=cfg)
    return dC.cpu(), _lib.last_kernel()


def _noalloc(A, B, cfg, variant):
    lib = _lib.library()
    dA, dB = A.cuda(), B.cuda()  # ordinary device tensors: no symmetric heap is involved
    dC = torch.full((A.shape[0], B.shape[1]), 7.0, dtype=A.dtype, device="cuda")
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.iris_hip_matmul_all_reduce_noalloc(
        p(dA), p(dB), p(dC), A.shape[0], B.shape[1], A.shape[1],
        dA.stride(0), dA.stride(1), dB.stride(0), dB.stride(1), dC.stride(0), dC.stride(1),
        cfg.block_size_m, cfg.block_size_n, cfg.block_size_k, variant,
        CODES[A.dtype], CODES[A.dtype], 1.0, _lib.PATH_AUTO, stream)
    assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    return dC.cpu(), _lib.last_kernel()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16_mfma", "fp32_generic"])
def test_noalloc_matches_the_workspace_entry_point_twice(dtype):
    shapes = [(1024, 768, 256), (200, 136, 72)]  # the second call is smaller (and ragged)
    for i, (M, N, K) in enumerate(shapes):
        A, B = randn_cpu((M, K), 10 + i, dtype, K ** -0.5), randn_cpu((K, N), 20 + i, dtype, K ** -0.5)
        for variant_name, variant in (("one_shot", _lib.VARIANT_ONE_SHOT), ("two_shot", _lib.VARIANT_TWO_SHOT)):
            cfg = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32, all_reduce_variant=variant_name)
            want, k_ref = _reference(A, B, cfg)
            got, k_new = _noalloc(A, B, cfg, variant)
            assert k_new == k_ref and k_new.startswith("mfma_" if dtype == torch.bfloat16 else "generic_"), (k_new, k_ref)
            assert_bits_equal(got, want, f"call {i} ({M}x{N}x{K}, {variant_name}, {k_new})")


def test_noalloc_rejects_what_does_not_fit():
    lib = _lib.library()
    null, p = ctypes.c_void_p(0), ctypes.c_void_p(0x10000)  # rejected before anything is dereferenced

    def call(M, N, K, bm, bn, out=_lib.BF16):
        return lib.iris_hip_matmul_all_reduce_noalloc(p, p, p, M, N, K, K, 1, N, 1, N, 1, bm, bn, 32,
                                                      _lib.VARIANT_ONE_SHOT, _lib.BF16, out, 1.0, _lib.PATH_AUTO, null)

    assert call(8192, 8192, 64, 256, 64) == 1 and "beyond the 33554432 bytes" in _lib.last_error()
    assert call(4096, 2048, 64, 16, 16) == 1 and "beyond the 16384 flags" in _lib.last_error()
    assert lib.iris_hip_matmul_all_reduce_noalloc(p, p, p, 64, 64, 64, 64, 1, 64, 1, 64, 1, 64, 64, 32, _lib.VARIANT_ATOMIC,
                                                  _lib.BF16, _lib.BF16, 1.0, 0, null) == 1 and "variant" in _lib.last_error()
