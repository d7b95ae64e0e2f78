"""GPU parity tests: the HIP path, called through the package and the C ABI, against the CPU oracle.

Tolerances (relative Frobenius error): 1e-2 for bfloat16/float16/float32, 3e-2 for float8 inputs.
Flags, owners, destinations and - for integer-valued inputs, where the fp32 product is exact -
every output bit must match.
"""

import pytest
import torch

import iris_amd as iris
from iris_amd import _lib
from iris_amd import ops
from helpers import (assert_bits_equal, heap_tensor, oracle, randint_cpu, randn_cpu, slot_copies, stage_peers)

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 1e-2, torch.float16: 1e-2, torch.float32: 1e-2}
HEAP = 1 << 28


def _ctx(world, rank=0, heap=HEAP):
    return iris.iris(heap, num_ranks=world, rank=rank)


def _run_all_reduce(ctx, A, B, peers, cfg, mode="fp32", path="auto", out_dtype=None, **kw):
    out_dtype = out_dtype or A.dtype
    dA, dB = heap_tensor(ctx, A), heap_tensor(ctx, B)
    dC = ctx.zeros((A.shape[0], B.shape[1]), dtype=out_dtype)
    ws = ops.matmul_all_reduce_preamble(ctx, dC, dA, dB, config=cfg)
    if peers is not None:
        stage_peers(ctx, ws, peers)
    ws = ops.matmul_all_reduce(ctx, dC, dA, dB, config=cfg, workspace=ws, slot_sum=mode, kernel_path=path, **kw)
    return dC, ws, _lib.last_kernel()


# ------------------------------------------------------------------------------------------------
# W = 1: every operator is a plain GEMM (the reference's own single-rank test configuration)
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("M,N,K", [(128, 64, 32), (1024, 256, 512), (256, 256, 64), (512, 384, 1376)])
@pytest.mark.parametrize("variant", ["one_shot", "two_shot"])
def test_single_rank_is_gemm(dtype, M, N, K, variant):
    ctx = _ctx(1)
    A, B = randn_cpu((M, K), 0, dtype), randn_cpu((K, N), 1, dtype)
    small = M <= 128 or K <= 64 or N <= 128 or dtype == torch.float32
    cfg = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32, all_reduce_variant=variant) if small \
        else iris.FusedConfig(all_reduce_variant=variant)
    dC, ws, kernel = _run_all_reduce(ctx, A, B, None, cfg)
    ref = oracle.gemm(A, B)
    err = oracle.rel_frobenius(dC.cpu(), ref)
    assert err <= TOL[dtype], f"{kernel}: rel Frobenius {err}"
    # the reference's own acceptance test (tests/ops/test_matmul_all_reduce.py:18-25,89)
    atol, rtol = {torch.float16: (0.2, 0.01), torch.float32: (0.3, 0.01), torch.bfloat16: (2.5, 0.02)}[dtype]
    assert torch.allclose(dC.cpu().float(), ref.float(), atol=atol, rtol=rtol)
    assert torch.all(ws.locks.cpu() == 1)
    assert_bits_equal(ws.aux_buffer.cpu(), dC.cpu(), "aux vs C at W=1")
    if dtype != torch.float32:
        assert kernel.startswith("mfma"), kernel


@pytest.mark.parametrize("path", ["mfma", "generic"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_exact_inputs_bit_exact(path, dtype):
    """Integer-valued inputs make the fp32 product exact, so the whole output must match bit for bit."""
    ctx = _ctx(1)
    M, N, K = 384, 320, 160
    A, B = randint_cpu((M, K), 3, dtype), randint_cpu((K, N), 4, dtype)
    cfg = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32, all_reduce_variant="one_shot")
    dC, ws, kernel = _run_all_reduce(ctx, A, B, None, cfg, path=path)
    assert kernel.startswith(path)
    assert_bits_equal(dC.cpu(), oracle.gemm(A, B), f"{kernel} exact GEMM")


# ------------------------------------------------------------------------------------------------
# W = 8 all-reduce: slot sums, flags, owners, destinations
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("path", ["mfma", "generic"])
@pytest.mark.parametrize("variant", ["one_shot", "two_shot"])
@pytest.mark.parametrize("mode", ["fp32", "reference"])
@pytest.mark.parametrize("rank", [0, 5])
def test_all_reduce_bit_exact(path, variant, mode, rank):
    W, dtype = 8, torch.bfloat16
    M, N, K = 512, 384, 96
    ctx = _ctx(W, rank)
    A, B = randint_cpu((M, K), 10, dtype), randint_cpu((K, N), 11, dtype)
    peers = [randn_cpu((M, N), 100 + r, dtype) for r in range(W)]
    cfg = iris.FusedConfig(block_size_m=128, block_size_n=64, block_size_k=32, all_reduce_variant=variant)
    dC, ws, kernel = _run_all_reduce(ctx, A, B, peers, cfg, mode=mode, path=path)
    exp = oracle.matmul_all_reduce(A, B, peers, rank, W, 128, 64, variant, mode)
    assert_bits_equal(ws.aux_buffer.cpu(), exp["aux"], "aux")
    assert torch.equal(ws.locks.cpu(), torch.from_numpy(exp["locks"])), "flags"
    got = slot_copies(ctx, dC)
    for r in range(W):
        assert_bits_equal(got[r], exp["C"][r], f"{kernel} C in slot {r}")


@pytest.mark.parametrize("path", ["mfma", "generic"])
@pytest.mark.parametrize("W,rank", [(2, 1), (3, 0), (5, 4), (12, 7), (16, 15)])
def test_all_reduce_other_world_sizes(path, W, rank):
    """World sizes other than the register-cached peer counts (1, 3, 7 peers), including more than
    eight slots, take the general peer loop."""
    dtype = torch.bfloat16
    M, N, K = 256, 128, 64
    ctx = _ctx(W, rank, heap=1 << 24)
    A, B = randint_cpu((M, K), 10, dtype), randint_cpu((K, N), 11, dtype)
    peers = [randn_cpu((M, N), 100 + r, dtype) for r in range(W)]
    for variant in ("one_shot", "two_shot"):
        cfg = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32, all_reduce_variant=variant)
        dC, ws, kernel = _run_all_reduce(ctx, A, B, peers, cfg, path=path)
        exp = oracle.matmul_all_reduce(A, B, peers, rank, W, 64, 64, variant)
        for r, got in enumerate(slot_copies(ctx, dC)):
            assert_bits_equal(got, exp["C"][r], f"{kernel} {variant} W={W} slot {r}")


def test_all_reduce_closed_form():
    """Rank r contributes r + 1 everywhere: every element sums to W(W+1)/2
    (the reference's tile-collective check, tests/context/test_all_reduce.py:245-246,352-356)."""
    W, dtype = 8, torch.bfloat16
    M, N, K = 256, 256, 64
    for rank in (0, 3):
        ctx = _ctx(W, rank)
        A = torch.zeros(M, K, dtype=dtype)
        A[:, 0] = rank + 1
        B = torch.zeros(K, N, dtype=dtype)
        B[0, :] = 1
        peers = [torch.full((M, N), float(r + 1), dtype=dtype) for r in range(W)]
        cfg = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32, all_reduce_variant="one_shot")
        dC, ws, _ = _run_all_reduce(ctx, A, B, peers, cfg)
        assert torch.all(dC.cpu().float() == W * (W + 1) / 2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_all_reduce_random(dtype):
    W, rank = 4, 1
    M, N, K = 1024, 256, 512
    ctx = _ctx(W, rank)
    A, B = randn_cpu((M, K), 0, dtype, K ** -0.5), randn_cpu((K, N), 1, dtype)
    peers = [randn_cpu((M, N), 7 + r, dtype) for r in range(W)]
    cfg = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32, all_reduce_variant="two_shot")
    dC, ws, kernel = _run_all_reduce(ctx, A, B, peers, cfg)
    exp = oracle.matmul_all_reduce(A, B, peers, rank, W, 64, 64, "two_shot")
    for r, got in enumerate(slot_copies(ctx, dC)):
        assert oracle.rel_frobenius(got, exp["C"][r]) <= TOL[dtype], f"{kernel} slot {r}"
    mine = torch.from_numpy(oracle.owner_map(M, N, 64, 64, W, "two_shot") == rank)
    assert torch.all(dC.cpu()[~mine] == 0), "tiles of other owners must stay untouched"


def test_flag_tiles_larger_than_kernel_tiles():
    """Flag tiles that span several kernel tiles are raised exactly once, by the last arrival."""
    W, rank, dtype = 2, 0, torch.bfloat16
    M, N, K = 1024, 1024, 64
    ctx = _ctx(W, rank)
    A, B = randint_cpu((M, K), 1, dtype), randint_cpu((K, N), 2, dtype)
    peers = [randn_cpu((M, N), 50 + r, dtype) for r in range(W)]
    for bm, bn in [(512, 512), (384, 200), (1024, 1024)]:
        cfg = iris.FusedConfig(block_size_m=bm, block_size_n=bn, block_size_k=32, all_reduce_variant="one_shot")
        dC, ws, kernel = _run_all_reduce(ctx, A, B, peers, cfg)
        exp = oracle.matmul_all_reduce(A, B, peers, rank, W, bm, bn, "one_shot")
        assert torch.equal(ws.locks.cpu(), torch.from_numpy(exp["locks"])), f"{kernel} flags {bm}x{bn}"
        assert_bits_equal(dC.cpu(), exp["C"][rank], f"{kernel} {bm}x{bn}")


@pytest.mark.parametrize("M,N,K", [(100, 72, 50), (130, 66, 33), (257, 129, 70)])
def test_ragged_shapes_generic(M, N, K):
    W, rank, dtype = 3, 2, torch.float16
    ctx = _ctx(W, rank)
    A, B = randint_cpu((M, K), 5, dtype), randint_cpu((K, N), 6, dtype)
    peers = [randn_cpu((M, N), 20 + r, dtype) for r in range(W)]
    cfg = iris.FusedConfig(block_size_m=32, block_size_n=24, block_size_k=16, all_reduce_variant="two_shot")
    dC, ws, kernel = _run_all_reduce(ctx, A, B, peers, cfg)
    assert kernel.startswith("generic")
    exp = oracle.matmul_all_reduce(A, B, peers, rank, W, 32, 24, "two_shot")
    for r, got in enumerate(slot_copies(ctx, dC)):
        assert_bits_equal(got, exp["C"][r], f"slot {r}")
    assert torch.all(ws.locks.cpu() == 1)


@pytest.mark.parametrize("M,N,K", [(256, 384, 128), (3072, 3072, 200)])
def test_transposed_b_and_strided_views(M, N, K):
    """B handed over as the transpose of an (N, K) tensor (K-contiguous) takes the MFMA path too
    (the small-output kernel for the first shape, 256x256 tiles for the second)."""
    ctx = _ctx(1, heap=1 << 27)
    dtype = torch.bfloat16
    A, Bt = randint_cpu((M, K), 8, dtype), randint_cpu((N, K), 9, dtype)
    dA, dBt = heap_tensor(ctx, A), heap_tensor(ctx, Bt)
    dC = ctx.zeros((M, N), dtype=dtype)
    cfg = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32, all_reduce_variant="one_shot")
    ops.matmul_all_reduce(ctx, dC, dA, dBt.t(), config=cfg)
    assert _lib.last_kernel().endswith("_nt"), _lib.last_kernel()
    assert_bits_equal(dC.cpu(), oracle.gemm(A, Bt.t()), "NT GEMM")


# ------------------------------------------------------------------------------------------------
# reduce-scatter
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("path", ["mfma", "generic"])
@pytest.mark.parametrize("rank", [0, 7])
def test_reduce_scatter_bit_exact(path, rank):
    W, dtype = 8, torch.bfloat16
    M, N, K = 640, 256, 64   # 10 x 4 tiles of 64x64 = 40 tiles: 5 per rank
    ctx = _ctx(W, rank)
    A, B = randint_cpu((M, K), 12, dtype), randint_cpu((K, N), 13, dtype)
    peers = [randn_cpu((M, N), 200 + r, dtype) for r in range(W)]
    cfg = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32)
    dA, dB = heap_tensor(ctx, A), heap_tensor(ctx, B)
    dC = ctx.zeros((M, N), dtype=dtype)
    ws = ops.matmul_reduce_scatter(ctx, dC, dA, dB, config=cfg, kernel_path=path,
                                   stage=lambda w: stage_peers(ctx, w, peers))
    exp = oracle.matmul_reduce_scatter(A, B, peers, rank, W, 64, 64)
    assert_bits_equal(ws.aux_buffer.cpu(), exp["aux"], "aux")
    assert torch.all(ws.locks.cpu() == 1)
    for r, got in enumerate(slot_copies(ctx, dC)):
        assert_bits_equal(got, exp["C"][r], f"C in slot {r}")


def test_reduce_scatter_reference_acceptance():
    """The reference's own check (tests/ops/test_matmul_reduce_scatter.py:24-89) at W = 1."""
    for dtype, atol, rtol in [(torch.float16, 2e-1, 1e-2), (torch.float32, 1e-1, 1e-2)]:
        ctx = _ctx(1)
        M, N, K = 128, 128, 32
        A, B = randn_cpu((M, K), 0, dtype), randn_cpu((K, N), 1, dtype)
        dA, dB = heap_tensor(ctx, A), heap_tensor(ctx, B)
        dC = ctx.zeros((M, N), dtype=dtype)
        cfg = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32)
        ops.matmul_reduce_scatter(ctx, dC, dA, dB, config=cfg)
        assert torch.allclose(dC.cpu().float(), (A.float() @ B.float()), atol=atol, rtol=rtol)


def test_reduce_scatter_all_owners_row_blocks():
    """One launch standing in for all ranks: row block r lands in slot r at its global coordinates."""
    W, rank, dtype = 8, 0, torch.bfloat16
    M, N, K = 2048, 512, 64   # 256x64 tiles: 8 x 8 = 64 tiles, 8 per rank = one tile row = 256 rows
    ctx = _ctx(W, rank)
    A, B = randint_cpu((M, K), 14, dtype), randint_cpu((K, N), 15, dtype)
    dA, dB = heap_tensor(ctx, A), heap_tensor(ctx, B)
    dC = ctx.zeros((M, N), dtype=dtype)
    for r in range(W):
        ctx.peer_view(dC, r).zero_()
    ops.matmul_reduce_scatter(ctx, dC, dA, dB, all_owners=True, sum_peers=False)
    exp = oracle.matmul_reduce_scatter(A, B, None, rank, W, 256, 64, all_owners=True, sum_peers=False)
    full = oracle.gemm(A, B)
    for r, got in enumerate(slot_copies(ctx, dC)):
        assert_bits_equal(got, exp["C"][r], f"slot {r}")
        assert_bits_equal(got[256 * r:256 * (r + 1)], full[256 * r:256 * (r + 1)], f"row block {r}")


# ------------------------------------------------------------------------------------------------
# all-gather + matmul
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("path", ["mfma", "generic"])
@pytest.mark.parametrize("M,K_local,N", [(128, 32, 64), (256, 64, 128), (512, 96, 256)])
@pytest.mark.parametrize("W", [1, 2, 8])
def test_all_gather_matmul_columns(path, M, K_local, N, W):
    dtype, rank = torch.float16, W - 1
    ctx = _ctx(W, rank)
    shards = [randint_cpu((M, K_local), 42 + r, dtype) for r in range(W)]
    B = randint_cpu((W * K_local, N), 123, dtype)
    dA = ctx.zeros((M, K_local), dtype=dtype)
    for r in range(W):
        ctx.peer_view(dA, r).copy_(shards[r])
    dB = heap_tensor(ctx, B)
    out = ctx.zeros((M, N), dtype=dtype)
    cfg = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32)
    ops.all_gather_matmul(ctx, out, dA, dB, config=cfg, kernel_path=path)
    assert _lib.last_kernel().startswith(path)
    assert_bits_equal(out.cpu(), oracle.all_gather_matmul(shards, B), _lib.last_kernel())


# The 256x256 tile (two wave groups half a K step apart) gathering along K: the A source changes in the
# middle of the load pipeline; K_local = 80 ends every source with a partial K step, 1 with an almost
# empty one.
@pytest.mark.parametrize("K_local,W", [(96, 4), (80, 3), (32, 8), (1, 2)])
def test_all_gather_matmul_columns_big_tile(K_local, W):
    M = N = 3072
    dtype, rank = torch.bfloat16, W - 1
    ctx = _ctx(W, rank, heap=1 << 27)
    shards = [randint_cpu((M, K_local), 42 + r, dtype) for r in range(W)]
    B = randint_cpu((W * K_local, N), 123, dtype)
    ok_mfma = K_local % 8 == 0
    dA = ctx.zeros((M, K_local), dtype=dtype)
    for r in range(W):
        ctx.peer_view(dA, r).copy_(shards[r])
    dB = heap_tensor(ctx, B)
    out = ctx.zeros((M, N), dtype=dtype)
    cfg = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=1)
    ops.all_gather_matmul(ctx, out, dA, dB, config=cfg)
    kernel = _lib.last_kernel()
    assert kernel.startswith("mfma_bf16_256x256" if ok_mfma else "generic"), kernel
    assert_bits_equal(out.cpu(), oracle.all_gather_matmul(shards, B), kernel)


def test_all_gather_matmul_rows_and_bias():
    W, rank, dtype = 8, 3, torch.bfloat16
    M_local, K, N = 128, 256, 192
    ctx = _ctx(W, rank)
    shards = [randint_cpu((M_local, K), 60 + r, dtype) for r in range(W)]
    B = randint_cpu((K, N), 70, dtype)
    bias = randint_cpu((W * M_local,), 71, dtype, -8, 9)
    dA = ctx.zeros((M_local, K), dtype=dtype)
    for r in range(W):
        ctx.peer_view(dA, r).copy_(shards[r])
    dB, dbias = heap_tensor(ctx, B), heap_tensor(ctx, bias)
    out = ctx.zeros((W * M_local, N), dtype=dtype)
    cfg = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32)
    for path in ("mfma", "generic"):
        out.zero_()
        ops.all_gather_matmul(ctx, out, dA, dB, bias=dbias, config=cfg, gather_dim=0, kernel_path=path)
        assert_bits_equal(out.cpu(), oracle.all_gather_matmul(shards, B, bias=bias, gather_dim=0), path)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float8_e4m3fn], ids=["bf16", "fp8"])
@pytest.mark.parametrize("gather_dim,W,rank,M,Kl,N", [(1, 8, 5, 80, 128, 272), (1, 2, 0, 200, 384, 144), (1, 3, 2, 32, 512, 1168),
                                                        (0, 4, 1, 32, 144, 528), (0, 8, 7, 64, 1360, 80)])
def test_all_gather_matmul_small_outputs(dtype, gather_dim, W, rank, M, Kl, N):
    """Small outputs take the 32x32 kernel also when A is gathered: along K the slot changes between the
    256-byte pieces of K that the waves own (K_local a multiple of 256 bytes), along M between row
    tiles (M here is the rows per slot); with and without the row bias, integer data, every bit."""
    fp8 = dtype == torch.float8_e4m3fn
    if fp8 and gather_dim == 1:
        Kl *= 2  # 256 bytes are 256 e4m3 values
    out_dtype = torch.bfloat16 if fp8 else dtype
    ctx = _ctx(W, rank)
    shards = [randint_cpu((M, Kl), 500 + r, torch.float32, -3, 4).to(dtype) for r in range(W)]
    Kt = Kl * W if gather_dim == 1 else Kl
    rows = M if gather_dim == 1 else M * W
    B = randint_cpu((Kt, N), 520, torch.float32, -3, 4).to(dtype)
    bias = randint_cpu((rows,), 521, out_dtype, -8, 9) if (rank % 2) else None
    dA = ctx.zeros((M, Kl), dtype=dtype)
    for r in range(W):
        ctx.peer_view(dA, r).copy_(shards[r])
    dB = heap_tensor(ctx, B)
    dbias = heap_tensor(ctx, bias) if bias is not None else None
    out = ctx.zeros((rows, N), dtype=out_dtype)
    cfg = iris.FusedConfig(block_size_m=16, block_size_n=16, block_size_k=16)
    kw = dict(scale_a=0.5, scale_b=2.0) if fp8 else {}
    ops.all_gather_matmul(ctx, out, dA, dB, bias=dbias, config=cfg, gather_dim=gather_dim, **kw)
    kernel = _lib.last_kernel()
    assert "_32x32x" in kernel, kernel
    exp = oracle.all_gather_matmul(shards, B, bias=bias, gather_dim=gather_dim, out_dtype=out_dtype, scale=1.0)
    assert_bits_equal(out.cpu(), exp, f"{kernel} gather_dim={gather_dim} bias={bias is not None}")


def test_all_gather_matmul_random_via_namespace():
    W, rank, dtype = 4, 0, torch.float16
    M, K_local, N = 256, 64, 128
    ctx = _ctx(W, rank)
    shards = [randn_cpu((M, K_local), 42 + r, dtype) for r in range(W)]
    B = randn_cpu((W * K_local, N), 123, dtype)
    dA = ctx.zeros((M, K_local), dtype=dtype)
    for r in range(W):
        ctx.peer_view(dA, r).copy_(shards[r])
    dB = heap_tensor(ctx, B)
    out = ctx.zeros((M, N), dtype=dtype)
    ctx.ops.all_gather_matmul(out, dA, dB, config=iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32))
    ref = torch.cat(shards, dim=1).float() @ B.float()
    # tests/ops/test_all_gather_matmul.py:97-101: atol = rtol = 1e-2 for fp16 ... on fp16-rounded reference
    assert torch.allclose(out.cpu().float(), ref.half().float(), atol=5e-2, rtol=1e-2)
    assert oracle.rel_frobenius(out.cpu(), ref) <= 1e-2


# ------------------------------------------------------------------------------------------------
# matmul + all-gather (scatter pattern) and the atomic all-reduce variant
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("path", ["mfma", "generic"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(64, 64, 32), (512, 256, 512), (1024, 2048, 1024)])
def test_matmul_all_gather(path, dtype, M, N, K):
    """Shapes of tests/ops/test_matmul_all_gather.py:18-30 of the reference, W = 4, every rank in turn."""
    W = 4
    M_local = M // W
    if M_local < 16:
        pytest.skip("M_local too small")
    B = randint_cpu((K, N), 77, dtype, -2, 3)
    As = [randint_cpu((M_local, K), 80 + r, dtype, -2, 3) for r in range(W)]
    bias = randint_cpu((M_local,), 90, dtype, -4, 5)
    bm = 16 if M_local < 64 else 64
    cfg = iris.FusedConfig(block_size_m=bm, block_size_n=64, block_size_k=32)
    for rank in (0, W - 1):
        ctx = _ctx(W, rank)
        dA, dB, dbias = heap_tensor(ctx, As[rank]), heap_tensor(ctx, B), heap_tensor(ctx, bias)
        out = ctx.zeros((M, N), dtype=dtype)
        for r in range(W):
            ctx.peer_view(out, r).zero_()
        ctx.ops.matmul_all_gather(out, dA, dB, bias=dbias, config=cfg, kernel_path=path)
        assert _lib.last_kernel().startswith(path)
        exp = oracle.matmul_all_gather(As[rank], B, rank, W, bias=bias)
        for r, got in enumerate(slot_copies(ctx, out)):
            assert_bits_equal(got, exp[r], f"{_lib.last_kernel()} rank {rank} slot {r}")


def test_matmul_all_gather_big_tile():
    """Enough rows per rank for the 256x256 tile (16 x 9 tiles), row bias, two slots."""
    W, rank, dtype = 2, 1, torch.bfloat16
    M_local, N, K = 4096, 2304, 72
    B = randint_cpu((K, N), 77, dtype, -2, 3)
    A = randint_cpu((M_local, K), 81, dtype, -2, 3)
    bias = randint_cpu((M_local,), 90, dtype, -4, 5)
    ctx = _ctx(W, rank, heap=1 << 27)
    dA, dB, dbias = heap_tensor(ctx, A), heap_tensor(ctx, B), heap_tensor(ctx, bias)
    out = ctx.zeros((W * M_local, N), dtype=dtype)
    for r in range(W):
        ctx.peer_view(out, r).zero_()
    ctx.ops.matmul_all_gather(out, dA, dB, bias=dbias, config=iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=8))
    assert _lib.last_kernel().startswith("mfma_bf16_256x256"), _lib.last_kernel()
    exp = oracle.matmul_all_gather(A, B, rank, W, bias=bias)
    for r, got in enumerate(slot_copies(ctx, out)):
        assert_bits_equal(got, exp[r], f"slot {r}")


@pytest.mark.parametrize("path", ["mfma", "generic"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_all_reduce_atomic(path, dtype):
    if dtype == torch.float32 and path == "mfma":
        pytest.skip("fp32 data runs on the generic kernel")
    W, rank = 4, 2
    M, N, K = 256, 192, 64
    ctx = _ctx(W, rank)
    A, B = randint_cpu((M, K), 21, dtype), randint_cpu((K, N), 22, dtype)
    before = [randint_cpu((M, N), 300 + r, dtype, -50, 51) for r in range(W)]  # what C held: the peers' adds so far
    dA, dB = heap_tensor(ctx, A), heap_tensor(ctx, B)
    dC = ctx.zeros((M, N), dtype=dtype)
    cfg = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32, all_reduce_variant="atomic")
    ws = ops.matmul_all_reduce_preamble(ctx, dC, dA, dB, config=cfg)
    assert ws.locks is None and ws.aux_buffer is None
    for r in range(W):
        ctx.peer_view(dC, r).copy_(before[r])
    ops.matmul_all_reduce(ctx, dC, dA, dB, config=cfg, workspace=ws, kernel_path=path)
    exp = oracle.matmul_all_reduce(A, B, before, rank, W, 64, 64, "atomic")
    for r, got in enumerate(slot_copies(ctx, dC)):
        assert_bits_equal(got, exp["C"][r], f"{_lib.last_kernel()} slot {r}")


# ------------------------------------------------------------------------------------------------
# float8 inputs
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("path", ["mfma", "generic"])
@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (32, 512, 256), (512, 384, 192)])
def test_fp8_all_reduce(path, M, N, K):
    W, rank = 8, 0
    ctx = _ctx(W, rank)
    a, b = randn_cpu((M, K), 0, torch.float32), randn_cpu((K, N), 1, torch.float32)
    Aq, sa = oracle.quantize_e4m3(a)
    Bq, sb = oracle.quantize_e4m3(b)
    peers = [randn_cpu((M, N), 30 + r, torch.bfloat16) for r in range(W)]
    cfg = iris.FusedConfig(block_size_m=32, block_size_n=64, block_size_k=64, all_reduce_variant="one_shot")
    dC, ws, kernel = _run_all_reduce(ctx, Aq, Bq, peers, cfg, path=path, out_dtype=torch.bfloat16, scale_a=sa, scale_b=sb)
    assert kernel.startswith(path), kernel
    exp = oracle.matmul_all_reduce(Aq, Bq, peers, rank, W, 32, 64, "one_shot", out_dtype=torch.bfloat16, scale=sa * sb)
    assert oracle.rel_frobenius(ws.aux_buffer.cpu(), exp["aux"]) <= 3e-2
    assert oracle.rel_frobenius(dC.cpu(), exp["C"][rank]) <= 3e-2
    # against the unquantised product the error is the quantisation error, still within the bound
    assert oracle.rel_frobenius(ws.aux_buffer.cpu(), a @ b) <= 6e-2


# ------------------------------------------------------------------------------------------------
# protocol and error behaviour
# ------------------------------------------------------------------------------------------------
def test_unstaged_peer_flags_time_out():
    """A peer that never raises its flags: the kernel gives up after spin_limit polls and the next
    barrier reports it (the reference would spin forever, iris/mem/triton/context.py:758)."""
    W, rank, dtype = 2, 0, torch.bfloat16
    ctx = _ctx(W, rank)
    ctx.spin_limit = 64
    M, N, K = 256, 256, 64
    dA, dB = heap_tensor(ctx, randint_cpu((M, K), 1, dtype)), heap_tensor(ctx, randint_cpu((K, N), 2, dtype))
    dC = ctx.zeros((M, N), dtype=dtype)
    cfg = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32, all_reduce_variant="one_shot")
    ws = ops.matmul_all_reduce_preamble(ctx, dC, dA, dB, config=cfg)
    ctx.peer_view(ws.locks, 1).zero_()
    with pytest.raises(RuntimeError, match="peer flag"):
        ops.matmul_all_reduce(ctx, dC, dA, dB, config=cfg, workspace=ws)
    assert torch.all(ws.locks.cpu() == 1), "own flags are raised before waiting"


@pytest.mark.parametrize("M,N,K,variant", [(512, 384, 96, "one_shot"), (512, 384, 96, "two_shot"),
                                           (32, 1168, 1360, "one_shot"), (1280, 3072, 1040, "two_shot"),
                                           (640, 1024, 96, "one_shot"), (3072, 3072, 80, "two_shot")])
def test_peer_flags_raised_while_the_kernel_waits(M, N, K, variant):
    """The normal case between real ranks: the peers' flags are not up yet when the kernel looks.  The
    launch goes out with the peers' flags at zero; another stream raises them a little later.  The
    kernel must have raised its own flags first, poll (bounded), and then sum what the peers
    published - on the small-output kernel (several row tiles, and one), the 128x128, the 64x64 and the
    256x256 kernel."""
    W, rank, dtype = 4, 2, torch.bfloat16
    ctx = _ctx(W, rank)
    A, B = randint_cpu((M, K), 30, dtype), randint_cpu((K, N), 31, dtype)
    peers = [randn_cpu((M, N), 400 + r, dtype) for r in range(W)]
    fbm = 32 if M == 32 else 128
    cfg = iris.FusedConfig(block_size_m=fbm, block_size_n=64, block_size_k=32, all_reduce_variant=variant)
    dA, dB = heap_tensor(ctx, A), heap_tensor(ctx, B)
    dC = ctx.zeros((M, N), dtype=dtype)
    ws = ops.matmul_all_reduce_preamble(ctx, dC, dA, dB, config=cfg)
    for r in range(W):
        if r != rank:
            ctx.peer_view(ws.aux_buffer, r).copy_(peers[r])
            ctx.peer_view(ws.locks, r).zero_()
    torch.cuda.synchronize()
    # The side stream's work goes out BEFORE the fused launch: a spin kernel, then the stores that raise the
    # flags.  Whatever hardware queue the side stream shares, the spin kernel is already dispatched when
    # the fused launch arrives, so nothing can queue the flag stores behind the polling kernel: either
    # the two streams run side by side (the fused kernel polls until the spin kernel ends) or the fused
    # launch waits behind both (and finds the flags up).
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        torch.cuda._sleep(2_000_000)
        for r in range(W):
            if r != rank:
                ctx.peer_view(ws.locks, r).fill_(1)
    ops.matmul_all_reduce(ctx, dC, dA, dB, async_op=True, config=cfg, workspace=ws)
    torch.cuda.synchronize()
    ctx.check_status()  # no spin time-out
    exp = oracle.matmul_all_reduce(A, B, peers, rank, W, fbm, 64, variant, "fp32")
    assert torch.equal(ws.locks.cpu(), torch.from_numpy(exp["locks"])), "flags"
    got = slot_copies(ctx, dC)
    for r in range(W if variant == "two_shot" else 1):
        slot = r if variant == "two_shot" else rank
        assert_bits_equal(got[slot], exp["C"][slot], f"{_lib.last_kernel()} C in slot {slot}")


@pytest.mark.parametrize("M,N,K,variant", [(512, 384, 96, "one_shot"), (512, 384, 96, "two_shot"),
                                           (32, 1168, 1360, "one_shot"), (1280, 3072, 1040, "two_shot"),
                                           (640, 1024, 96, "one_shot"), (3072, 3072, 80, "one_shot")])
def test_unregistered_context_tensor_gives_the_same_bits(M, N, K, variant):
    """The kernels take the heap bases as kernel arguments when the host has registered the context
    tensor's contents, and load them from the tensor otherwise (a binding that never registers).
    Both routes must produce the same aux, flags and C; the sizes cover the small-output kernel and the
    128x128, 64x64 and 256x256 tiles."""
    W, rank, dtype = 4, 1, torch.bfloat16
    A, B = randint_cpu((M, K), 20, dtype), randint_cpu((K, N), 21, dtype)
    peers = [randn_cpu((M, N), 200 + r, dtype) for r in range(W)]
    fbm = 32 if M == 32 else 128
    cfg = iris.FusedConfig(block_size_m=fbm, block_size_n=64, block_size_k=32, all_reduce_variant=variant)
    exp = oracle.matmul_all_reduce(A, B, peers, rank, W, fbm, 64, variant, "fp32")
    kernels = []
    for registered in (True, False):
        ctx = _ctx(W, rank)
        if not registered:
            ctx._forget_device_context()
        assert ctx._context_registered == registered
        dC, ws, kernel = _run_all_reduce(ctx, A, B, peers, cfg)
        kernels.append(kernel)
        assert_bits_equal(ws.aux_buffer.cpu(), exp["aux"], f"aux, registered={registered}")
        assert torch.equal(ws.locks.cpu(), torch.from_numpy(exp["locks"])), "flags"
        got = slot_copies(ctx, dC)
        for r in range(W if variant == "two_shot" else 1):
            slot = r if variant == "two_shot" else rank
            assert_bits_equal(got[slot], exp["C"][slot], f"{kernel} C in slot {slot}, registered={registered}")
    assert kernels[0] == kernels[1] and kernels[0].startswith("mfma_")


def test_heap_tensors_outlive_their_context(monkeypatch):
    """The heap allocation is released with its last tensor, not with the context object."""
    from iris_amd.host import hip as hip_mod

    freed = []
    real_free = hip_mod.hip_free
    monkeypatch.setattr(hip_mod, "hip_free", lambda ptr: (freed.append(ptr), real_free(ptr)))
    ctx = _ctx(2)
    base = ctx.heap.base_address
    t = ctx.zeros((256, 256), dtype=torch.float32)
    peer = ctx.peer_view(t, 1)
    t.fill_(2.0)
    peer.fill_(5.0)
    del ctx
    import gc
    gc.collect()
    assert base not in freed
    assert float(t.sum()) == 2.0 * 256 * 256 and float(peer.sum()) == 5.0 * 256 * 256
    del t
    gc.collect()
    assert base not in freed, "a peer view still holds the heap"
    del peer
    gc.collect()
    torch.cuda.synchronize()
    assert freed.count(base) == 1


def test_c_abi_rejects_bad_arguments():
    lib = _lib.library()
    import ctypes
    ctx = _ctx(1)
    t = ctx.zeros((64, 64), dtype=torch.bfloat16)
    null = ctypes.c_void_p(0)
    p = ctypes.c_void_p(t.data_ptr())
    rc = lib.iris_hip_matmul_all_reduce(p, p, p, null, null, 64, 64, 64, 64, 1, 64, 1, 64, 1, null, 0, 1, 64, 64, 32,
                                        _lib.VARIANT_ONE_SHOT, _lib.BF16, _lib.BF16, 1.0, 0, 0, null, 0, null)
    assert rc == 1 and "aux_buffer" in _lib.last_error()
    rc = lib.iris_hip_matmul_all_reduce(p, p, p, p, p, 64, 64, 64, 64, 1, 64, 1, 64, 1, null, 0, 1, 64, 64, 32,
                                        7, _lib.BF16, _lib.BF16, 1.0, 0, 0, null, 0, null)
    assert rc == 1 and "variant" in _lib.last_error()
    cu, xcc, lds = ctypes.c_int32(), ctypes.c_int32(), ctypes.c_int32()
    assert lib.iris_hip_query(0, ctypes.byref(cu), ctypes.byref(xcc), ctypes.byref(lds)) == 0
    assert cu.value == torch.cuda.get_device_properties(0).multi_processor_count and xcc.value >= 1


# ------------------------------------------------------------------------------------------------
# HIP graphs: a launch is one kernel node, so launch-bound loops can be captured and replayed
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("M,N,K,kernel", [(1280, 3072, 1040, "128x128"), (1280, 3072, 160, "64x128"), (256, 384, 160, "32x32"),
                                          (32, 1168, 1360, "32x32"), (3072, 3072, 80, "256x256")])
@pytest.mark.parametrize("variant", ["one_shot", "two_shot"])
def test_graph_replay_matches_eager(variant, M, N, K, kernel):
    """Captured once, replayed four times with new operands: the tiled kernels and the small-output kernel
    (whose helper wave probes the peers' flags through heap bases that travel as kernel arguments), the
    latter with several row tiles and with a single one."""
    W, dtype = 4, torch.bfloat16
    ctx = _ctx(W)
    B = randint_cpu((K, N), 21, dtype)
    peers = [randn_cpu((M, N), 200 + r, dtype) for r in range(W)]
    fbm = min(64, M)
    cfg = iris.FusedConfig(block_size_m=fbm, block_size_n=64, block_size_k=32, all_reduce_variant=variant)
    dA, dB = ctx.zeros((M, K), dtype=dtype), heap_tensor(ctx, B)
    dC = ctx.zeros((M, N), dtype=dtype)
    ws = ops.matmul_all_reduce_preamble(ctx, dC, dA, dB, config=cfg)
    stage_peers(ctx, ws, peers)

    def launch():
        ws.prepared = True
        ops.matmul_all_reduce(ctx, dC, dA, dB, async_op=True, config=cfg, workspace=ws)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch()  # first call outside the capture: one-time function attributes are set here
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        launch()

    for rep in range(4):
        A = randint_cpu((M, K), 300 + rep, dtype)
        dA.copy_(A)  # eager work between the replays: new operands, outputs and own flags cleared
        for r in range(W):
            ctx.peer_view(dC, r).zero_()
        ws.locks.zero_()
        ws.aux_buffer.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        ctx.check_status()
        assert f"_{kernel}x" in _lib.last_kernel(), _lib.last_kernel()
        exp = oracle.matmul_all_reduce(A, B, peers, 0, W, fbm, 64, variant, "fp32")
        assert_bits_equal(ws.aux_buffer.cpu(), exp["aux"], f"aux, replay {rep}")
        assert torch.equal(ws.locks.cpu(), torch.from_numpy(exp["locks"])), f"flags, replay {rep}"
        got = slot_copies(ctx, dC)
        for r in range(W):
            assert_bits_equal(got[r], exp["C"][r], f"C in slot {r}, replay {rep}")


# ------------------------------------------------------------------------------------------------
# Ragged extents on the MFMA path: partial tiles in M, N and K, single-row problems
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("M,N,K", [(200, 264, 72), (1000, 520, 1376), (1, 2880, 512), (33, 136, 24), (4100, 4104, 40)])
@pytest.mark.parametrize("variant", ["one_shot", "two_shot"])
def test_ragged_shapes_mfma(M, N, K, variant):
    W, rank, dtype = 8, 6, torch.bfloat16
    ctx = _ctx(W, rank, heap=1 << 27)
    A, B = randint_cpu((M, K), 50, dtype), randint_cpu((K, N), 51, dtype)
    peers = [randn_cpu((M, N), 600 + r, dtype) for r in range(W)]
    cfg = iris.FusedConfig(block_size_m=32 if M >= 32 else 1, block_size_n=64, block_size_k=8, all_reduce_variant=variant)
    dC, ws, kernel = _run_all_reduce(ctx, A, B, peers, cfg, path="mfma")
    assert kernel.startswith("mfma_bf16"), kernel
    exp = oracle.matmul_all_reduce(A, B, peers, rank, W, cfg.block_size_m, cfg.block_size_n, variant, "fp32")
    assert_bits_equal(ws.aux_buffer.cpu(), exp["aux"], "aux")
    assert torch.equal(ws.locks.cpu(), torch.from_numpy(exp["locks"])), "flags"
    got = slot_copies(ctx, dC)
    for r in range(W):
        assert_bits_equal(got[r], exp["C"][r], f"{kernel} C in slot {r}")


# Tile counts that are not a multiple of the eight XCDs: the launch grid is rounded up and the surplus
# workgroups must find no tile (90, 180, 270 and 432 tiles of 32x32 - one and two rounds of the small-output
# kernel -, 132 and 405 of 64x64 - one and two workgroups per CU -, 257 and 368 of 64x128 - the same -, 184 of
# 128x128, 140 of 256x256).
@pytest.mark.parametrize("M,N,K,tile", [(32, 2880, 64, "32x32"), (48, 2880, 64, "32x32"), (96, 2880, 64, "32x32"),
                                        (384, 1152, 96, "32x32"), (48, 8400, 64, "64x64"), (300, 5184, 64, "64x64"), (48, 32848, 64, "64x128"), (1000, 2880, 64, "64x128"), (1000, 2880, 1032, "128x128"),
                                        (2560, 3584, 64, "256x256")])
def test_tile_counts_off_the_xcd_multiple(M, N, K, tile):
    W, rank, dtype = 2, 1, torch.float16
    ctx = _ctx(W, rank, heap=1 << 27)
    A, B = randint_cpu((M, K), 52, dtype), randint_cpu((K, N), 53, dtype)
    peers = [randn_cpu((M, N), 620 + r, dtype) for r in range(W)]
    cfg = iris.FusedConfig(block_size_m=32, block_size_n=64, block_size_k=8, all_reduce_variant="two_shot")
    dC, ws, kernel = _run_all_reduce(ctx, A, B, peers, cfg, path="mfma")
    assert kernel.startswith(f"mfma_f16_{tile}"), kernel
    exp = oracle.matmul_all_reduce(A, B, peers, rank, W, 32, 64, "two_shot", "fp32")
    assert_bits_equal(ws.aux_buffer.cpu(), exp["aux"], "aux")
    assert torch.equal(ws.locks.cpu(), torch.from_numpy(exp["locks"])), "flags"
    got = slot_copies(ctx, dC)
    for r in range(W):
        assert_bits_equal(got[r], exp["C"][r], f"{kernel} C in slot {r}")


# Seeded random draws over world size, rank, element type, shape (all four tile shapes), variant and
# flag-tile size; integer-valued operands, so every output bit is determined.
@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_shapes_bit_exact(seed):
    import random

    rng = random.Random(seed)
    for case in range(10):
        W = rng.choice([1, 2, 3, 4, 8])
        rank = rng.randrange(W)
        dtype = rng.choice([torch.bfloat16, torch.float16])
        if rng.random() < 0.3:
            M, N, K = rng.choice([2304, 2560, 4100]), rng.choice([3584, 4096, 2312]), rng.choice([8, 40, 136])
        else:
            M = rng.choice([1, 17, 32, 33, 64, 96, 130, 200, 384, 640, 1000])
            N = rng.choice([64, 72, 136, 264, 520, 1152, 2880])
            K = rng.choice([8, 24, 72, 128, 200, 520])
        variant = rng.choice(["one_shot", "two_shot"])
        bm = min(rng.choice([16, 32, 64, 128]), M) if M >= 16 else 1
        bn = min(rng.choice([32, 64, 128]), N)
        what = f"seed {seed} case {case}: W={W} rank={rank} {dtype} {M}x{N}x{K} {variant} flags {bm}x{bn}"
        ctx = _ctx(W, rank, heap=1 << 27)
        A, B = randint_cpu((M, K), 1000 + case, dtype), randint_cpu((K, N), 2000 + case, dtype)
        peers = [randn_cpu((M, N), 3000 + 10 * case + r, dtype) for r in range(W)]
        cfg = iris.FusedConfig(block_size_m=bm, block_size_n=bn, block_size_k=8, all_reduce_variant=variant)
        dC, ws, kernel = _run_all_reduce(ctx, A, B, peers, cfg)
        assert kernel.startswith("mfma_"), f"{what}: {kernel}"
        exp = oracle.matmul_all_reduce(A, B, peers, rank, W, bm, bn, variant, "fp32")
        assert_bits_equal(ws.aux_buffer.cpu(), exp["aux"], f"{what}: aux")
        assert torch.equal(ws.locks.cpu(), torch.from_numpy(exp["locks"])), f"{what}: flags"
        for r, got in enumerate(slot_copies(ctx, dC)):
            assert_bits_equal(got, exp["C"][r], f"{what}: {kernel} C in slot {r}")
        del ctx, dC, ws
        torch.cuda.empty_cache()


@pytest.mark.parametrize("M,N,K", [(200, 272, 80), (1, 1024, 256), (520, 144, 1008)])
def test_ragged_shapes_mfma_fp8(M, N, K):
    W, rank = 4, 1
    ctx = _ctx(W, rank)
    a, b = randn_cpu((M, K), 60, torch.float32), randn_cpu((K, N), 61, torch.float32)
    (Aq, sa), (Bq, sb) = oracle.quantize_e4m3(a), oracle.quantize_e4m3(b)
    peers = [randn_cpu((M, N), 700 + r, torch.bfloat16) for r in range(W)]
    cfg = iris.FusedConfig(block_size_m=32 if M >= 32 else 1, block_size_n=64, block_size_k=16, all_reduce_variant="one_shot")
    dC, ws, kernel = _run_all_reduce(ctx, Aq, Bq, peers, cfg, path="mfma", out_dtype=torch.bfloat16, scale_a=sa, scale_b=sb)
    assert kernel.startswith("mfma_fp8"), kernel
    exp = oracle.matmul_all_reduce(Aq, Bq, peers, rank, W, cfg.block_size_m, 64, "one_shot", "fp32",
                                   out_dtype=torch.bfloat16, scale=sa * sb)
    assert torch.equal(ws.locks.cpu(), torch.from_numpy(exp["locks"])), "flags"
    assert oracle.rel_frobenius(dC.cpu(), exp["C"][rank]) < 3e-2
