"""GPU parity tests of the tail policy of the 256x256 tile: in a last round of tiles that is at most half
full, workgroups without a tile multiply the second part of the others' K ranges and pass fp32 partial
sums on.  Integer-valued inputs make every partial sum exact, so the split launch must give the oracle's
bits wherever the split point is; the shapes put it next to K tails and between the source slots of a
gathered A, after one whole round of tiles."""

import pytest
import torch

import iris_amd as iris
from iris_amd import _lib, ops
from helpers import assert_bits_equal, heap_tensor, oracle, randint_cpu, randn_cpu, slot_copies, stage_peers

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def split_whenever_possible():
    """Mode 1: split whenever the last round can be split (the default rule only splits long K loops)."""
    _lib.library().iris_hip_set_split_tiles(1)
    yield
    _lib.library().iris_hip_set_split_tiles(-1)


def _ctx(world, rank=0, heap=1 << 28):
    return iris.iris(heap, num_ranks=world, rank=rank)


# tiles of 256 x 256 on 256 CUs in 8 XCDs (32 workgroups each); every XCD first takes a whole round of 32:
#   5120 x 3840 = 20 x 15 = 300 tiles: 38 per XCD (34 in the last XCD): 6 (2) tiles left for the split round
#   5120 x 4096 = 20 x 16 = 320 tiles: 40 per XCD: 8 left
#   4352 x 4096 = 17 x 16 = 272 tiles: 34 per XCD: 2 left
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float8_e4m3fn], ids=["bf16", "f16", "fp8"])
@pytest.mark.parametrize("M,N,K", [(5120, 3840, 320), (5120, 4096, 512), (4352, 4096, 1040), (5120, 3840, 272)])
def test_plain_gemm_split(dtype, M, N, K):
    """all_gather_matmul with one rank is the plain GEMM; K = 1040 and 272 end in a partial K step."""
    fp8 = dtype == torch.float8_e4m3fn
    out_dtype = torch.bfloat16 if fp8 else dtype
    ctx = _ctx(1)
    A = randint_cpu((M, K), 1, torch.float32, -3, 4).to(dtype)
    B = randint_cpu((K, N), 2, torch.float32, -3, 4).to(dtype)
    dA, dB = heap_tensor(ctx, A), heap_tensor(ctx, B)
    out = ctx.zeros((M, N), dtype=out_dtype)
    kw = dict(scale_a=0.5, scale_b=2.0) if fp8 else {}
    ops.all_gather_matmul(ctx, out, dA, dB, **kw)
    kernel = _lib.last_kernel()
    assert "256x256" in kernel and kernel.endswith("_splitk"), kernel
    assert_bits_equal(out.cpu(), oracle.all_gather_matmul([A], B, out_dtype=out_dtype, scale=1.0), kernel)


@pytest.mark.parametrize("gather_dim,W,rank", [(1, 4, 3), (1, 3, 0), (0, 8, 5)])
def test_gathered_a_split(gather_dim, W, rank):
    """A gathered from the slots: along K the split points fall inside and between the sources' column
    blocks (K_local = 80: every source ends in a partial K step), along M every tile reads one slot."""
    dtype = torch.bfloat16
    ctx = _ctx(W, rank)
    if gather_dim == 1:
        M, N, Kl = 5120, 3840, 80
        shards = [randint_cpu((M, Kl), 10 + r, dtype) for r in range(W)]
        B = randint_cpu((W * Kl, N), 30, dtype)
        rows = M
    else:
        M_local, N, Kl = 768, 3328, 200  # 6144 x 3328 = 24 x 13 = 312 tiles: 39 per XCD, 7 left
        shards = [randint_cpu((M_local, Kl), 10 + r, dtype) for r in range(W)]
        B = randint_cpu((Kl, N), 30, dtype)
        rows = W * M_local
    bias = randint_cpu((rows,), 31, dtype, -8, 9)
    dA = ctx.zeros(tuple(shards[0].shape), dtype=dtype)
    for r in range(W):
        ctx.peer_view(dA, r).copy_(shards[r])
    dB, dbias = heap_tensor(ctx, B), heap_tensor(ctx, bias)
    out = ctx.zeros((rows, N), dtype=dtype)
    ops.all_gather_matmul(ctx, out, dA, dB, bias=dbias, gather_dim=gather_dim)
    kernel = _lib.last_kernel()
    assert kernel.endswith("_splitk"), kernel
    assert_bits_equal(out.cpu(), oracle.all_gather_matmul(shards, B, bias=bias, gather_dim=gather_dim), kernel)


@pytest.mark.parametrize("variant,W,rank,M,N,K", [("one_shot", 4, 1, 5120, 3840, 200), ("one_shot", 2, 0, 5120, 4096, 192),
                                                  ("two_shot", 1, 0, 5120, 3840, 200)])
def test_all_reduce_split(variant, W, rank, M, N, K):
    """The main of a split tile runs the whole epilogue: aux, flags, the slot sum over the peers.  (A
    two-shot launch with peers and more tiles than CUs keeps one workgroup per tile and is not split.)"""
    dtype = torch.bfloat16
    ctx = _ctx(W, rank, heap=1 << 29)
    A, B = randint_cpu((M, K), 5, dtype), randint_cpu((K, N), 6, dtype)
    peers = [randn_cpu((M, N), 40 + r, dtype) for r in range(W)]
    cfg = iris.FusedConfig(block_size_m=128, block_size_n=64, block_size_k=32, all_reduce_variant=variant)
    dA, dB = heap_tensor(ctx, A), heap_tensor(ctx, B)
    dC = ctx.zeros((M, N), dtype=dtype)
    ws = ops.matmul_all_reduce_preamble(ctx, dC, dA, dB, config=cfg)
    stage_peers(ctx, ws, peers)
    ops.matmul_all_reduce(ctx, dC, dA, dB, config=cfg, workspace=ws)
    kernel = _lib.last_kernel()
    assert kernel.endswith("_splitk"), kernel
    exp = oracle.matmul_all_reduce(A, B, peers, rank, W, 128, 64, variant, "fp32")
    assert torch.equal(ws.locks.cpu(), torch.from_numpy(exp["locks"])), "flags"
    assert_bits_equal(ws.aux_buffer.cpu(), exp["aux"], f"{kernel} aux")
    got = slot_copies(ctx, dC)
    for slot in (range(W) if variant == "two_shot" else [rank]):
        assert_bits_equal(got[slot], exp["C"][slot], f"{kernel} C in slot {slot}")


def test_split_launches_in_a_row_and_on_two_streams():
    """The flags of the workspace are never cleared: every launch uses a new flag value.  Three launches in
    a row on one stream, then one on a second stream (which gets a workspace of its own), each checked."""
    dtype, M, N, K = torch.bfloat16, 5120, 3840, 136
    ctx = _ctx(1)
    outs = []
    side = torch.cuda.Stream()
    for i in range(4):
        A, B = randint_cpu((M, K), 70 + i, dtype), randint_cpu((K, N), 80 + i, dtype)
        dA, dB = heap_tensor(ctx, A), heap_tensor(ctx, B)
        out = ctx.zeros((M, N), dtype=dtype)
        torch.cuda.synchronize()
        if i == 3:
            with torch.cuda.stream(side):
                ops.all_gather_matmul(ctx, out, dA, dB)
            side.synchronize()
        else:
            ops.all_gather_matmul(ctx, out, dA, dB)
        assert _lib.last_kernel().endswith("_splitk")
        outs.append((out, oracle.all_gather_matmul([A], B)))
    torch.cuda.synchronize()
    for i, (out, want) in enumerate(outs):
        assert_bits_equal(out.cpu(), want, f"launch {i}")


def test_captured_launches_are_not_split():
    """A launch recorded into a HIP graph keeps its tiles whole (its flag value would repeat on every
    replay); the replays give the oracle's bits, with eager split launches in between."""
    dtype, M, N, K = torch.bfloat16, 5120, 3840, 136
    ctx = _ctx(1)
    A, B = randint_cpu((M, K), 95, dtype), randint_cpu((K, N), 96, dtype)
    dA, dB = heap_tensor(ctx, A), heap_tensor(ctx, B)
    out, eager = ctx.zeros((M, N), dtype=dtype), ctx.zeros((M, N), dtype=dtype)
    want = oracle.all_gather_matmul([A], B)
    ops.all_gather_matmul(ctx, eager, dA, dB)  # the stream has a workspace by now
    assert _lib.last_kernel().endswith("_splitk")
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        ops.all_gather_matmul(ctx, out, dA, dB, async_op=True)
    assert not _lib.last_kernel().endswith("_splitk"), _lib.last_kernel()
    for replay in range(3):
        out.zero_()
        eager.zero_()
        ops.all_gather_matmul(ctx, eager, dA, dB)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert_bits_equal(out.cpu(), want, f"replay {replay}")
        assert_bits_equal(eager.cpu(), want, f"eager launch before replay {replay}")


def test_random_data_within_tolerance_and_default_rule():
    """Random data: the split launch sums K in another order, the result stays within the bf16 bound.  And
    the default rule: a short K loop is not split, a long one with a last round that is a fifth full is."""
    dtype, M, N = torch.bfloat16, 5120, 3840
    ctx = _ctx(1, heap=1 << 29)
    for K, want_split in ((256, False), (4096, True)):
        A, B = randn_cpu((M, K), 90, dtype, K ** -0.5), randn_cpu((K, N), 91, dtype, K ** -0.5)
        dA, dB = heap_tensor(ctx, A), heap_tensor(ctx, B)
        out = ctx.zeros((M, N), dtype=dtype)
        _lib.library().iris_hip_set_split_tiles(1)
        ops.all_gather_matmul(ctx, out, dA, dB)
        assert _lib.last_kernel().endswith("_splitk")
        assert oracle.rel_frobenius(out.cpu(), oracle.gemm(A, B)) <= 1e-2
        _lib.library().iris_hip_set_split_tiles(-1)
        ops.all_gather_matmul(ctx, out, dA, dB)
        assert _lib.last_kernel().endswith("_splitk") == want_split, (K, _lib.last_kernel())
        assert oracle.rel_frobenius(out.cpu(), oracle.gemm(A, B)) <= 1e-2
        _lib.library().iris_hip_set_split_tiles(0)
        ops.all_gather_matmul(ctx, out, dA, dB)
        assert not _lib.last_kernel().endswith("_splitk")
