"""The five target configurations of this build at full size on the GPU, against the CPU oracle.

Inputs are drawn on the CPU from torch.Generator().manual_seed(seed) as the configurations state.
Full-size comparisons use the oracle directly; the largest case (fp8, 16384 x 8192) is compared in row
chunks that cover the whole output, plus size-independent properties (flags all raised, untouched slots
untouched).
"""

import pytest
import torch

import iris_amd as iris
from iris_amd import _lib, ops
from helpers import assert_bits_equal, heap_tensor, oracle, randn_cpu, slot_copies, stage_peers

pytestmark = pytest.mark.gpu


def test_config1_plumbing_fp32_one_shot():
    """fp32 256^3, uniform[-1,1] seed 0, one synthetic peer N(0,1) seed 1, W = 2, one-shot."""
    g = torch.Generator().manual_seed(0)
    A = torch.rand((256, 256), generator=g) * 2 - 1
    B = torch.rand((256, 256), generator=g) * 2 - 1
    peer = randn_cpu((256, 256), 1, torch.float32)
    ctx = iris.iris(1 << 26, num_ranks=2, rank=0)
    dA, dB = heap_tensor(ctx, A), heap_tensor(ctx, B)
    dC = ctx.zeros((256, 256), dtype=torch.float32)
    cfg = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32, all_reduce_variant="one_shot")
    ws = ops.matmul_all_reduce_preamble(ctx, dC, dA, dB, config=cfg)
    stage_peers(ctx, ws, [None, peer])
    ops.matmul_all_reduce(ctx, dC, dA, dB, config=cfg, workspace=ws)
    exp = oracle.matmul_all_reduce(A, B, [None, peer], 0, 2, 64, 64, "one_shot")
    assert oracle.rel_frobenius(dC.cpu(), exp["C"][0]) <= 1e-5
    assert torch.allclose(dC.cpu(), A @ B + peer, atol=1e-4, rtol=1e-5)


@pytest.mark.parametrize("variant", ["one_shot", "two_shot"])
def test_config2_matmul_all_reduce_bf16(variant):
    M, N, K, W = 4096, 4096, 1376, 8
    g = torch.Generator().manual_seed(0)
    A = (torch.randn((M, K), generator=g) / K ** 0.5).to(torch.bfloat16)
    B = (torch.randn((K, N), generator=g) / K ** 0.5).to(torch.bfloat16)
    peers = [None] + [randn_cpu((M, N), r, torch.bfloat16) for r in range(1, W)]
    ctx = iris.iris(1 << 28, num_ranks=W, rank=0)
    dA, dB = heap_tensor(ctx, A), heap_tensor(ctx, B)
    dC = ctx.zeros((M, N), dtype=torch.bfloat16)
    cfg = iris.FusedConfig(all_reduce_variant=variant)  # 256 x 64 flag tiles: 1024 flags
    ws = ops.matmul_all_reduce_preamble(ctx, dC, dA, dB, config=cfg)
    assert ws.locks.numel() == 1024
    stage_peers(ctx, ws, peers)
    ops.matmul_all_reduce(ctx, dC, dA, dB, config=cfg, workspace=ws)
    kernel = _lib.last_kernel()
    assert kernel.startswith("mfma_bf16_256x256"), kernel
    exp = oracle.matmul_all_reduce(A, B, peers, 0, W, 256, 64, variant)
    assert torch.all(ws.locks.cpu() == 1)
    assert oracle.rel_frobenius(ws.aux_buffer.cpu(), exp["aux"]) <= 1e-2
    got = slot_copies(ctx, dC)
    for r in range(W):
        assert oracle.rel_frobenius(got[r], exp["C"][r]) <= 1e-2, f"slot {r}"
    # The slot sum itself must be exact given the aux the kernel produced.
    again = oracle.slot_sum(ws.aux_buffer.cpu(), peers[1:])
    if variant == "one_shot":
        assert_bits_equal(got[0], again, "slot sum from the kernel's own aux")
        for r in range(1, W):
            assert torch.all(got[r] == 0)
    else:
        mine = torch.from_numpy(oracle.owner_map(M, N, 256, 64, W, "two_shot") == 0)
        for r in range(W):
            assert_bits_equal(got[r], torch.where(mine, again, torch.zeros_like(again)), f"slot {r}")


def test_config3_all_gather_matmul_bf16_rows():
    W, M_local, K, N = 8, 1024, 4096, 1792
    shards = [(randn_cpu((M_local, K), r, torch.float32) / K ** 0.5).to(torch.bfloat16) for r in range(W)]
    B = (randn_cpu((K, N), 8, torch.float32) / K ** 0.5).to(torch.bfloat16)
    ctx = iris.iris(1 << 27, num_ranks=W, rank=0)
    dA = ctx.zeros((M_local, K), dtype=torch.bfloat16)
    for r in range(W):
        ctx.peer_view(dA, r).copy_(shards[r])
    dB = heap_tensor(ctx, B)
    out = ctx.zeros((W * M_local, N), dtype=torch.bfloat16)
    ops.all_gather_matmul(ctx, out, dA, dB, gather_dim=0)
    assert _lib.last_kernel().startswith("mfma_bf16"), _lib.last_kernel()
    ref = oracle.all_gather_matmul(shards, B, gather_dim=0)
    assert oracle.rel_frobenius(out.cpu(), ref) <= 1e-2


def test_config3_shape_in_reference_layout_columns():
    """The same GEMM shape in the reference's layout: A sharded along K (K_local = 512)."""
    W, M, K_local, N = 8, 8192, 512, 1792
    K = W * K_local
    shards = [(randn_cpu((M, K_local), r, torch.float32) / K ** 0.5).to(torch.bfloat16) for r in range(W)]
    B = (randn_cpu((K, N), 8, torch.float32) / K ** 0.5).to(torch.bfloat16)
    ctx = iris.iris(1 << 27, num_ranks=W, rank=2)
    dA = ctx.zeros((M, K_local), dtype=torch.bfloat16)
    for r in range(W):
        ctx.peer_view(dA, r).copy_(shards[r])
    dB = heap_tensor(ctx, B)
    out = ctx.zeros((M, N), dtype=torch.bfloat16)
    ops.all_gather_matmul(ctx, out, dA, dB)
    assert oracle.rel_frobenius(out.cpu(), oracle.all_gather_matmul(shards, B)) <= 1e-2


def test_config4_matmul_reduce_scatter_bf16():
    M, N, K, W = 8192, 4096, 1376, 8
    g = torch.Generator().manual_seed(0)
    A = (torch.randn((M, K), generator=g) / K ** 0.5).to(torch.bfloat16)
    B = (torch.randn((K, N), generator=g) / K ** 0.5).to(torch.bfloat16)
    ctx = iris.iris(1 << 28, num_ranks=W, rank=0)
    dA, dB = heap_tensor(ctx, A), heap_tensor(ctx, B)
    dC = ctx.zeros((M, N), dtype=torch.bfloat16)
    for r in range(W):
        ctx.peer_view(dC, r).zero_()
    ws = ops.matmul_reduce_scatter(ctx, dC, dA, dB, all_owners=True, sum_peers=False)
    assert ws.locks.numel() == 2048 and torch.all(ws.locks.cpu() == 1)
    ref = oracle.gemm(A, B)
    aux = ws.aux_buffer.cpu()
    assert oracle.rel_frobenius(aux, ref) <= 1e-2
    got = slot_copies(ctx, dC)
    for r in range(W):
        rows = slice(1024 * r, 1024 * (r + 1))
        assert_bits_equal(got[r][rows], aux[rows], f"row block {r} in slot {r}")
        other = torch.ones(M, dtype=torch.bool)
        other[rows] = False
        assert torch.all(got[r][other] == 0), f"slot {r} holds rows it does not own"


@pytest.mark.parametrize("rank", [0, 7])
def test_config4_matmul_reduce_scatter_accumulate_leg(rank):
    """The reference semantics at full size (iris/mem/triton/context.py:953-997): one rank's launch,
    seven staged peer aux buffers, the rank's 1024-row block summed over the slots in fp32 and cast once."""
    M, N, K, W = 8192, 4096, 1376, 8
    g = torch.Generator().manual_seed(0)
    A = (torch.randn((M, K), generator=g) / K ** 0.5).to(torch.bfloat16)
    B = (torch.randn((K, N), generator=g) / K ** 0.5).to(torch.bfloat16)
    peers = [None if r == rank else randn_cpu((M, N), 1 + r, torch.bfloat16) for r in range(W)]
    ctx = iris.iris(1 << 28, num_ranks=W, rank=rank)
    dA, dB = heap_tensor(ctx, A), heap_tensor(ctx, B)
    dC = ctx.zeros((M, N), dtype=torch.bfloat16)
    for r in range(W):
        ctx.peer_view(dC, r).zero_()
    ws = ops.matmul_reduce_scatter(ctx, dC, dA, dB, stage=lambda w: stage_peers(ctx, w, peers))
    kernel = _lib.last_kernel()
    assert kernel.startswith("mfma_bf16_256x256"), kernel
    assert ws.locks.numel() == 2048 and torch.all(ws.locks.cpu() == 1)
    aux = ws.aux_buffer.cpu()
    assert oracle.rel_frobenius(aux, oracle.gemm(A, B)) <= 1e-2
    rows = slice(1024 * rank, 1024 * (rank + 1))
    assert torch.equal(torch.from_numpy(oracle.owner_map(M, N, 256, 64, W, "reduce_scatter") == rank).nonzero()[:, 0].unique(),
                       torch.arange(rows.start, rows.stop)), "the rank owns exactly its 1024-row block"
    got = slot_copies(ctx, dC)
    want = oracle.slot_sum(aux[rows], [p[rows] for p in peers if p is not None])
    assert_bits_equal(got[rank][rows], want, f"rank {rank}: slot sum of the owned block from the kernel's own aux")
    exp = oracle.matmul_reduce_scatter(A, B, peers, rank, W, 256, 64)
    assert oracle.rel_frobenius(got[rank], exp["C"][rank]) <= 1e-2
    other = torch.ones(M, dtype=torch.bool)
    other[rows] = False
    assert torch.all(got[rank][other] == 0), "rows of other owners are left alone"
    for r in range(W):
        if r != rank:
            assert torch.all(got[r] == 0), f"slot {r} was written"


def _fp8_case(M, N, K, W, block_m):
    a, b = randn_cpu((M, K), 0, torch.float32), randn_cpu((K, N), 1, torch.float32)
    Aq, sa = oracle.quantize_e4m3(a)
    Bq, sb = oracle.quantize_e4m3(b)
    ctx = iris.iris(1 << 30, num_ranks=W, rank=0)
    dA, dB = heap_tensor(ctx, Aq), heap_tensor(ctx, Bq)
    dC = ctx.zeros((M, N), dtype=torch.bfloat16)
    cfg = iris.FusedConfig(block_size_m=block_m, block_size_n=64, block_size_k=64, all_reduce_variant="one_shot")
    ws = ops.matmul_all_reduce_preamble(ctx, dC, dA, dB, config=cfg)
    for r in range(1, W):  # peers' partial results: bf16 N(0,1) from the CPU generator, seed r
        ctx.peer_view(ws.aux_buffer, r).copy_(randn_cpu((M, N), r, torch.bfloat16))
        ctx.peer_view(ws.locks, r).fill_(1)
    ops.matmul_all_reduce(ctx, dC, dA, dB, config=cfg, workspace=ws, scale_a=sa, scale_b=sb)
    return ctx, ws, dC, Aq, Bq, sa * sb, _lib.last_kernel()


def test_config5a_fp8_matmul_all_reduce():
    """Every row of the 16384 x 8192 output, in chunks the CPU product finishes in seconds."""
    M, N, K, W = 16384, 8192, 1024, 8
    ctx, ws, dC, Aq, Bq, scale, kernel = _fp8_case(M, N, K, W, 256)
    assert kernel.startswith("mfma_fp8_256x256"), kernel
    assert torch.all(ws.locks.cpu() == 1)
    err2 = ref2 = 0.0
    step = 2048
    for r0 in range(0, M, step):
        rows = slice(r0, r0 + step)
        own = oracle.gemm(Aq[rows], Bq, torch.bfloat16, scale)
        aux = ws.aux_buffer[rows].cpu()
        assert oracle.rel_frobenius(aux, own) <= 3e-2, f"rows {r0}"
        err2 += float(((aux.double() - own.double()) ** 2).sum())
        ref2 += float((own.double() ** 2).sum())
        peers = [ctx.peer_view(ws.aux_buffer, r)[rows].cpu() for r in range(1, W)]
        if r0 == 0:
            assert_bits_equal(peers[0], randn_cpu((M, N), 1, torch.bfloat16)[rows], "staged peer 1")
        assert_bits_equal(dC[rows].cpu(), oracle.slot_sum(aux, peers), f"rows {r0}")
        for r in range(1, W):
            assert torch.all(ctx.peer_view(dC, r)[rows] == 0), f"one-shot wrote slot {r}"
    assert (err2 / ref2) ** 0.5 <= 3e-2


def test_config5b_fp8_skinny():
    M, N, K, W = 32, 8192, 1024, 8
    ctx, ws, dC, Aq, Bq, scale, kernel = _fp8_case(M, N, K, W, 32)
    own = oracle.gemm(Aq, Bq, torch.bfloat16, scale)
    aux = ws.aux_buffer.cpu()
    assert oracle.rel_frobenius(aux, own) <= 3e-2, kernel
    peers = [ctx.peer_view(ws.aux_buffer, r).cpu() for r in range(1, W)]
    assert_bits_equal(dC.cpu(), oracle.slot_sum(aux, peers), kernel)
