"""GPU parity tests of the stand-alone collectives (ctx.ccl.all_reduce / reduce_scatter) against the
CPU oracle.  The kernel reproduces the reference's order of fp32 additions, so every comparison is
bit for bit, random data included.  Shapes and block sizes follow tests/ccl/test_all_reduce.py:33-41
of the reference.
"""

import ctypes

import pytest
import torch

import iris_amd as iris
from iris_amd import _lib
from iris_amd.ccl import Config
from helpers import assert_bits_equal, oracle, randn_cpu, slot_copies

pytestmark = pytest.mark.gpu

HEAP = 1 << 28
SHAPES = [(128, 64, 32, 64), (128, 128, 32, 32), (256, 128, 32, 16), (1024, 256, 32, 64)]


def _stage(ctx, inputs, out_fill=0.0, group=None):
    """Heap tensors for input/output with every slot of the group filled; returns (d_in, d_out)."""
    ranks = list(range(ctx.get_num_ranks())) if group is None else list(group)
    d_in = ctx.zeros(tuple(inputs[0].shape), dtype=inputs[0].dtype)
    d_out = ctx.zeros(tuple(inputs[0].shape), dtype=inputs[0].dtype)
    for i, r in enumerate(ranks):
        ctx.peer_view(d_in, r).copy_(inputs[i])
        ctx.peer_view(d_out, r).fill_(out_fill)
    return d_in, d_out


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,bm,bn", SHAPES)
@pytest.mark.parametrize("variant", ["one_shot", "two_shot", "atomic"])
def test_all_reduce_matches_oracle(variant, M, N, bm, bn, dtype):
    W, rank = 8, 3
    ctx = iris.iris(HEAP, num_ranks=W, rank=rank)
    inputs = [randn_cpu((M, N), 40 + r, dtype) for r in range(W)]
    d_in, d_out = _stage(ctx, inputs)
    cfg = Config(all_reduce_variant=variant, block_size_m=bm, block_size_n=bn)
    if variant == "two_shot":
        cfg.all_reduce_distribution = 0  # as the reference test does
    ws = ctx.ccl.all_reduce_preamble(d_out, d_in, config=cfg)
    ctx.ccl.all_reduce(d_out, d_in, config=cfg, workspace=ws)
    if variant == "atomic":  # one dword per thread: packed pairs of 16-bit values, or one float
        assert _lib.last_kernel().endswith("vec1" if dtype == torch.float32 else "vec2"), _lib.last_kernel()
    else:
        assert "vec" in _lib.last_kernel() and "vec1" not in _lib.last_kernel()
    exp = oracle.ccl_all_reduce(inputs, [torch.zeros((M, N), dtype=dtype)] * W, rank, variant, bm, bn,
                                cfg.swizzle_size, cfg.comm_sms, cfg.all_reduce_distribution)
    got = slot_copies(ctx, d_out)
    for r in range(W):
        assert_bits_equal(got[r], exp[r], f"{variant} output in slot {r}")


@pytest.mark.parametrize("variant", ["one_shot", "two_shot", "atomic"])
def test_all_reduce_closed_form_all_ranks(variant):
    # tests/ccl/test_all_reduce.py:55,92-97: rank r holds r+1; after every rank has run, every rank's
    # output is W(W+1)/2 everywhere.  One GPU plays the ranks one after the other on one heap.
    W, M, N = 8, 1024, 256
    ctx0 = iris.iris(HEAP, num_ranks=W, rank=0)
    d_in, d_out = _stage(ctx0, [torch.full((M, N), float(r + 1), dtype=torch.bfloat16) for r in range(W)])
    lib = _lib.library()
    cfg = Config(all_reduce_variant=variant)
    code = {"atomic": _lib.VARIANT_ATOMIC, "one_shot": _lib.VARIANT_ONE_SHOT, "two_shot": _lib.VARIANT_TWO_SHOT}[variant]
    for r in range(W):  # the launch of rank r, through the C ABI, on rank r's copies
        rc = lib.iris_hip_all_reduce(
            ctypes.c_void_p(ctx0.peer_view(d_in, r).data_ptr()), ctypes.c_void_p(ctx0.peer_view(d_out, r).data_ptr()),
            M, N, N, 1, N, 1, ctypes.c_void_p(ctx0.get_heap_bases().data_ptr()), r, r, W, 0, 1,
            cfg.block_size_m, cfg.block_size_n, cfg.swizzle_size, cfg.comm_sms, cfg.num_xcds, cfg.chunk_size,
            code, cfg.all_reduce_distribution, _lib.BF16, None)
        assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    for r, out in enumerate(slot_copies(ctx0, d_out)):
        assert torch.all(out == W * (W + 1) / 2), f"slot {r}"


@pytest.mark.parametrize("distribution", [0, 1])
@pytest.mark.parametrize("W,rank", [(1, 0), (2, 1), (3, 2), (4, 0), (8, 7), (12, 5), (16, 15)])
def test_two_shot_distributions_and_world_sizes(W, rank, distribution):
    M, N = 200, 136  # ragged against 32 x 64 tiles; 136 = 17 chunks of 8
    ctx = iris.iris(1 << 24, num_ranks=W, rank=rank)
    inputs = [randn_cpu((M, N), 60 + r, torch.bfloat16) for r in range(W)]
    d_in, d_out = _stage(ctx, inputs, out_fill=-1.0)
    cfg = Config(all_reduce_variant="two_shot", all_reduce_distribution=distribution, comm_sms=5, swizzle_size=3)
    ctx.ccl.all_reduce(d_out, d_in, config=cfg)
    exp = oracle.ccl_all_reduce(inputs, [torch.full((M, N), -1.0, dtype=torch.bfloat16)] * W, rank, "two_shot", 32, 64, 3, 5,
                                distribution)
    got = slot_copies(ctx, d_out)
    for r in range(W):
        assert_bits_equal(got[r], exp[r], f"slot {r}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("distribution", [0, 1])
def test_reduce_scatter_matches_oracle(distribution, dtype):
    W, rank, M, N = 8, 6, 512, 320
    ctx = iris.iris(HEAP, num_ranks=W, rank=rank)
    inputs = [randn_cpu((M, N), 80 + r, dtype) for r in range(W)]
    d_in, d_out = _stage(ctx, inputs, out_fill=7.0)
    cfg = Config(all_reduce_distribution=distribution)
    ctx.ccl.reduce_scatter(d_out, d_in, config=cfg)
    exp = oracle.ccl_reduce_scatter(inputs, torch.full((M, N), 7.0, dtype=dtype), rank, 32, 64, 4, 64, distribution)
    got = slot_copies(ctx, d_out)
    assert_bits_equal(got[rank], exp, "own output")
    for r in range(W):
        if r != rank:
            assert torch.all(got[r] == 7.0), f"slot {r} must not be written"


@pytest.mark.parametrize("variant", ["one_shot", "two_shot", "atomic"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_element_path_for_odd_shapes_and_strides(variant, dtype):
    # N not a multiple of 16 bytes, and column-strided views: the kernel falls back to element accesses
    W, rank, M, N = 4, 1, 70, 51
    ctx = iris.iris(1 << 24, num_ranks=W, rank=rank)
    wide = [randn_cpu((M, 2 * N), 90 + r, dtype) for r in range(W)]
    d_in_wide, d_out_wide = _stage(ctx, wide)
    d_in, d_out = d_in_wide[:, ::2], d_out_wide[:, 1::2]
    cfg = Config(all_reduce_variant=variant, block_size_m=16, block_size_n=32, swizzle_size=2, comm_sms=3)
    ctx.ccl.all_reduce(d_out, d_in, config=cfg)
    assert _lib.last_kernel().endswith("vec1")
    inputs = [w[:, ::2].contiguous() for w in wide]
    exp = oracle.ccl_all_reduce(inputs, [torch.zeros((M, N), dtype=dtype)] * W, rank, variant, 16, 32, 2, 3, 1)
    for r in range(W):
        got = ctx.peer_view(d_out_wide, r).cpu()
        assert_bits_equal(got[:, 1::2].contiguous(), exp[r], f"slot {r}")
        assert torch.all(got[:, 0::2] == 0), "columns between the output's are untouched"


def test_strided_group():
    W, rank, M, N = 8, 5, 128, 128
    group = [1, 3, 5, 7]
    ctx = iris.iris(1 << 24, num_ranks=W, rank=rank)
    inputs = [randn_cpu((M, N), 110 + i, torch.float16) for i in range(len(group))]
    d_in, d_out = _stage(ctx, inputs, group=group)
    for r in (0, 2, 4, 6):  # outsiders: poison the input, mark the output
        ctx.peer_view(d_in, r).fill_(float("nan"))
        ctx.peer_view(d_out, r).fill_(3.0)
    cfg = Config(all_reduce_variant="two_shot", all_reduce_distribution=0)
    ctx.ccl.all_reduce(d_out, d_in, group=group, config=cfg)
    exp = oracle.ccl_all_reduce(inputs, [torch.zeros((M, N), dtype=torch.float16)] * 4, 2, "two_shot", 32, 64, 4, 64, 0)
    got = slot_copies(ctx, d_out)
    for i, r in enumerate(group):
        assert_bits_equal(got[r], exp[i], f"group member {r}")
    for r in (0, 2, 4, 6):
        assert torch.all(got[r] == 3.0)


def test_large_one_shot_closed_form():
    # the reference's "Large" case, 8192 x 8192 (tests/ccl/test_all_reduce.py:40)
    W, M, N = 8, 8192, 8192
    ctx = iris.iris(2 * M * N * 2 + (1 << 20), num_ranks=W, rank=2)
    d_in = ctx.zeros((M, N), dtype=torch.bfloat16)
    d_out = ctx.zeros((M, N), dtype=torch.bfloat16)
    for r in range(W):
        ctx.peer_view(d_in, r).fill_(float(r + 1))
    ctx.ccl.all_reduce(d_out, d_in, config=Config(all_reduce_variant="one_shot"))
    assert torch.all(d_out == 36.0)
    ctx.ccl.all_reduce(d_out, d_in, config=Config(all_reduce_variant="two_shot"))
    for r in range(W):
        out = ctx.peer_view(d_out, r)
        owned = out[2 * 1024:3 * 1024] if r != 2 else out  # block distribution: rank 2 owns tile rows 64..95
        assert torch.all(owned == 36.0)


def test_ccl_errors():
    ctx = iris.iris(1 << 24, num_ranks=2, rank=0)
    a = ctx.zeros((64, 64), dtype=torch.bfloat16)
    b = ctx.zeros((64, 64), dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="Only ReduceOp.SUM"):
        ctx.ccl.all_reduce(b, a, op=iris.ccl.ReduceOp.MAX)
    with pytest.raises(ValueError, match="use_gluon"):
        ctx.ccl.all_reduce(b, a, config=Config(use_gluon=True))
    with pytest.raises(NotImplementedError, match="ring"):
        ctx.ccl.all_reduce(b, a, config=Config(all_reduce_variant="ring"))
    with pytest.raises(ValueError, match="does not match input shape"):
        ctx.ccl.reduce_scatter(ctx.zeros((32, 64), dtype=torch.bfloat16), a)
    with pytest.raises(RuntimeError, match="not part of the specified process group"):
        ctx.ccl.all_reduce(b, a, group=[1])
    lib = _lib.library()
    p, null = ctypes.c_void_p(a.data_ptr()), ctypes.c_void_p(0)
    rc = lib.iris_hip_all_reduce(p, p, 64, 64, 64, 1, 64, 1, null, 0, 0, 2, 0, 1, 32, 64, 4, 64, 8, 8,
                                 _lib.VARIANT_ONE_SHOT, 1, _lib.BF16, None)
    assert rc == 1 and "heap_bases" in _lib.last_error()
    hb = ctypes.c_void_p(ctx.get_heap_bases().data_ptr())
    rc = lib.iris_hip_all_reduce(p, p, 64, 64, 64, 1, 64, 1, hb, 0, 0, 2, 0, 1, 32, 64, 4, 64, 8, 8, 1, 1, _lib.BF16, None)
    assert rc == 1 and "variant" in _lib.last_error()
    rc = lib.iris_hip_reduce_scatter(p, p, 64, 64, 64, 1, 64, 1, hb, 0, 0, 2, 0, 1, 32, 64, 4, 64, 8, 8, 2, _lib.BF16, None)
    assert rc == 1 and "distribution" in _lib.last_error()


def test_collectives_replay_in_a_hip_graph():
    """all_reduce and reduce_scatter launches are single kernel nodes: captured once, replayed with new
    inputs, every replay bit-identical to the oracle."""
    W, rank, M, N = 4, 1, 256, 192
    ctx = iris.iris(1 << 24, num_ranks=W, rank=rank)
    d_in = ctx.zeros((M, N), dtype=torch.bfloat16)
    d_ar = ctx.zeros((M, N), dtype=torch.bfloat16)
    d_rs = ctx.zeros((M, N), dtype=torch.bfloat16)
    cfg = Config(all_reduce_variant="two_shot", all_reduce_distribution=0)
    ws = ctx.ccl.all_reduce_preamble(d_ar, d_in, config=cfg)

    def launch():
        ws.prepared = True
        ctx.ccl.all_reduce(d_ar, d_in, config=cfg, workspace=ws, async_op=True)
        ctx.ccl.reduce_scatter(d_rs, d_in, config=cfg, async_op=True)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        launch()
    for rep in range(3):
        inputs = [randn_cpu((M, N), 900 + 10 * rep + r, torch.bfloat16) for r in range(W)]
        for r in range(W):
            ctx.peer_view(d_in, r).copy_(inputs[r])
            ctx.peer_view(d_ar, r).fill_(-2.0)
        d_rs.fill_(-2.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        blank = torch.full((M, N), -2.0, dtype=torch.bfloat16)
        exp_ar = oracle.ccl_all_reduce(inputs, [blank] * W, rank, "two_shot", 32, 64, 4, 64, 0)
        exp_rs = oracle.ccl_reduce_scatter(inputs, blank, rank, 32, 64, 4, 64, 0)
        for r, got in enumerate(slot_copies(ctx, d_ar)):
            assert_bits_equal(got, exp_ar[r], f"all_reduce slot {r}, replay {rep}")
        assert_bits_equal(d_rs.cpu(), exp_rs, f"reduce_scatter, replay {rep}")
