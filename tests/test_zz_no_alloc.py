"""The entry point that allocates nothing (iris_hip_matmul_all_reduce_noalloc), through the C ABI,
against iris_hip_matmul_all_reduce with a caller-owned workspace at world size 1 (same kernels, so
every output bit must agree) and against the oracle's product (a mistake that both entry points share
would pass the first comparison).  Two calls in a row on the same GPU, the second with a smaller
input (the library's workspace keeps the first call's contents)."""

import ctypes

import pytest
import torch

import iris_amd as iris
from iris_amd import _lib, ops
from helpers import assert_bits_equal, heap_tensor, randint_cpu, randn_cpu
from oracle import iris_oracle as oracle  # the checker

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
            tol = 1e-2 if dtype == torch.bfloat16 else 1e-5  # relative Frobenius error against the oracle's product
            assert oracle.rel_frobenius(got, oracle.gemm(A, B)) <= tol, f"call {i} against the oracle"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16_mfma", "fp32_generic"])
def test_noalloc_is_bit_exact_against_the_oracle_twice(dtype):
    """Integer-valued inputs make every fp32 partial sum exact, so the oracle's product is the one right
    answer whatever the summation order: the no-alloc entry point must hit it bit for bit, on two
    calls in a row, the second smaller and ragged."""
    for i, (M, N, K) in enumerate([(1024, 768, 256), (200, 136, 72)]):
        A, B = randint_cpu((M, K), 30 + i, dtype), randint_cpu((K, N), 40 + i, dtype)
        for variant_name, variant in (("one_shot", _lib.VARIANT_ONE_SHOT), ("two_shot", _lib.VARIANT_TWO_SHOT)):
            cfg = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32, all_reduce_variant=variant_name)
            got, kernel = _noalloc(A, B, cfg, variant)
            assert_bits_equal(got, oracle.gemm(A, B), f"call {i} ({M}x{N}x{K}, {variant_name}, {kernel}) against the oracle")


def test_noalloc_under_graph_capture():
    """What the entry point is for: two calls captured into one HIP graph (the second smaller, so it
    meets the first call's leftovers in the library's workspace), replayed three times with eager work
    and synchronisations in between; every replay must give the oracle's bits.  One eager call comes
    first: the library resolves its workspace address and the kernels' attributes on first use, which
    belongs in front of a capture."""
    lib = _lib.library()
    dtype = torch.bfloat16
    cfg = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32, all_reduce_variant="one_shot")
    shapes = [(1024, 768, 256), (200, 136, 72)]
    host = [(randint_cpu((M, K), 50 + i, dtype), randint_cpu((K, N), 60 + i, dtype)) for i, (M, N, K) in enumerate(shapes)]
    for A, B in host:  # eager first use of both kernel builds
        _noalloc(A, B, cfg, _lib.VARIANT_ONE_SHOT)
    dev = [(A.cuda(), B.cuda(), torch.zeros((A.shape[0], B.shape[1]), dtype=dtype, device="cuda")) for A, B in host]
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        for dA, dB, dC in dev:
            rc = lib.iris_hip_matmul_all_reduce_noalloc(
                p(dA), p(dB), p(dC), dA.shape[0], dB.shape[1], dA.shape[1],
                dA.stride(0), dA.stride(1), dB.stride(0), dB.stride(1), dC.stride(0), dC.stride(1),
                cfg.block_size_m, cfg.block_size_n, cfg.block_size_k, _lib.VARIANT_ONE_SHOT,
                CODES[dtype], CODES[dtype], 1.0, _lib.PATH_AUTO, stream)
            assert rc == 0, _lib.last_error()
    want = [oracle.gemm(A, B) for A, B in host]
    for replay in range(3):
        for _, _, dC in dev:
            dC.fill_(-5.0)  # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for i, (_, _, dC) in enumerate(dev):
            assert_bits_equal(dC.cpu(), want[i], f"replay {replay}, call {i}")


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
    # rejected by the checks of the launch itself, before anything is enqueued: an unsupported type pair,
    # operands the MFMA kernel cannot take when that kernel is demanded
    assert call(64, 64, 64, 64, 64, out=_lib.FP16) == 1 and "element types" in _lib.last_error()
    assert lib.iris_hip_matmul_all_reduce_noalloc(p, p, p, 64, 64, 64, 1, 64, 64, 1, 64, 1, 64, 64, 32, _lib.VARIANT_ONE_SHOT,
                                                  _lib.BF16, _lib.BF16, 1.0, _lib.PATH_MFMA, null) == 1 and "MFMA" in _lib.last_error()
