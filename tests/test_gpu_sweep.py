"""Bit-exact coverage of every compiled build of the MFMA kernel, and a seeded sweep over all five
operators.

Operands are small integers (exact in bfloat16, float16 and e4m3, with exact fp32 products and sums),
scales are powers of two, peers' partial results are arbitrary values of the output type: every bit
of aux, flags and C in every slot is then determined and is compared with the CPU oracle.
"""

import random

import pytest
import torch

import iris_amd as iris
from iris_amd import _lib, ops
from helpers import assert_bits_equal, heap_tensor, oracle, randint_cpu, randn_cpu, slot_copies, stage_peers

pytestmark = pytest.mark.gpu

FP8 = torch.float8_e4m3fn
NAMES = {torch.bfloat16: "bf16", torch.float16: "f16", FP8: "fp8"}

# Shapes that make the host pick each tile shape on a 256-CU part: >= 136 tiles of 256x256 (big), at
# most 256 tiles of 128x128 but more than 256 of 64x128 (small), more than 256 of 128x128 (small2, two
# workgroups per CU), M <= 64 or at most 512 tiles of 64x128 with a short K (skinny), at most 512 tiles of 64x64;
# outputs of at most 512 tiles of 32x32 take the small-output kernel
# (one row tile, six of them, and more tiles than CUs: two workgroups per CU, K in chunks of half the size).
TILE_SHAPES = {
    "256x256": (3072, 3072, 80),
    "128x128s": (1280, 3072, 2064),  # 128-byte K steps
    "64x128m": (1280, 3072, 208),    # 480 tiles of 64x128 and a short K
    "128x128d": (2304, 2048, 80),    # 64-byte K steps, two workgroups per CU
    "64x128": (48, 32832, 336),      # at most 64 rows: 513 tiles of 64x64, 257 of 64x128
    "64x64": (48, 8320, 336),        # 130 tiles of 64x64
    "32x32": (32, 1168, 1360),       # at most 32 rows: K in 1024-byte chunks (2 or 3 here)
    "32x32m": (176, 400, 1360),      # 6 x 13 tiles, the last row tile half empty
    "32x32h": (96, 2768, 1360),      # 3 x 87 tiles: 512-byte chunks, the last one ragged across the waves
    "64x64l": (192, 2864, 4112),     # 135 tiles of 64x64 (540 of 32x32: past the small-output kernel), long K
}


def _operand(shape, seed, dtype, lo=-3, hi=4):
    return randint_cpu(shape, seed, torch.float32, lo, hi).to(dtype)


def _device_b(ctx, B, layout):
    """B on the heap, N-contiguous ("nn") or as the transpose of an (N, K) tensor ("nt")."""
    if layout == "nn":
        return heap_tensor(ctx, B)
    return heap_tensor(ctx, B.t().contiguous()).t()


def _scales(dtype):
    return dict(scale_a=0.25, scale_b=2.0) if dtype == FP8 else {}


@pytest.mark.parametrize("layout", ["nn", "nt"])
@pytest.mark.parametrize("tile", sorted(TILE_SHAPES))
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, FP8], ids=lambda d: NAMES[d])
def test_every_build_bit_exact(dtype, tile, layout):
    """3 input types x 7 kernels (the small-output one at three shapes, the 64x64 tile at two) x 2 layouts of B through
    matmul_all_reduce with three peers."""
    M, N, K = TILE_SHAPES[tile]
    W, rank = 4, 2
    out_dtype = torch.bfloat16 if dtype == FP8 else dtype
    variant = "two_shot" if layout == "nt" else "one_shot"
    ctx = iris.iris(1 << 27, num_ranks=W, rank=rank)
    A, B = _operand((M, K), 7, dtype), _operand((K, N), 8, dtype)
    peers = [randn_cpu((M, N), 40 + r, out_dtype) for r in range(W)]
    bm = 16 if M < 64 else 64
    cfg = iris.FusedConfig(block_size_m=bm, block_size_n=64, block_size_k=16, all_reduce_variant=variant)
    dA, dB = heap_tensor(ctx, A), _device_b(ctx, B, layout)
    dC = ctx.zeros((M, N), dtype=out_dtype)
    ws = ops.matmul_all_reduce_preamble(ctx, dC, dA, dB, config=cfg)
    stage_peers(ctx, ws, peers)
    ops.matmul_all_reduce(ctx, dC, dA, dB, config=cfg, workspace=ws, kernel_path="mfma", **_scales(dtype))
    kernel = _lib.last_kernel()
    assert kernel.startswith(f"mfma_{NAMES[dtype]}_{tile[:7].rstrip('sdmhl')}") and kernel.endswith("_" + layout), kernel
    kstep = int(kernel.split("x")[2].split("_")[0]) * (1 if dtype == FP8 else 2)  # bytes per K step
    assert kstep == {"256x256": 64, "128x128s": 128, "128x128d": 64, "64x128": 128, "64x128m": 128, "64x64": 128, "32x32": 1024, "32x32m": 1024, "32x32h": 512, "64x64l": 128}[tile], kernel
    scale = 0.5 if dtype == FP8 else 1.0
    exp = oracle.matmul_all_reduce(A, B, peers, rank, W, bm, 64, variant, out_dtype=out_dtype, scale=scale)
    assert_bits_equal(ws.aux_buffer.cpu(), exp["aux"], f"{kernel}: aux")
    assert torch.equal(ws.locks.cpu(), torch.from_numpy(exp["locks"])), f"{kernel}: flags"
    for r, got in enumerate(slot_copies(ctx, dC)):
        assert_bits_equal(got, exp["C"][r], f"{kernel}: C in slot {r}")


@pytest.mark.parametrize("tile,shape", [("256x256", (3000, 3088, 48)), ("128x128", (1300, 3088, 80)), ("128x128", (2300, 2064, 48)),
                                        ("64x128", (48, 32848, 96)), ("64x64", (48, 8336, 96)), ("64x64", (300, 5136, 80)), ("32x32", (600, 400, 80)), ("32x32", (48, 1168, 96))])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, FP8], ids=lambda d: NAMES[d])
def test_atomic_variant_on_every_tile(dtype, tile, shape):
    """The atomic epilogue deals the dwords of a tile out to the threads in its own order (one wave
    instruction = 256 contiguous bytes); ragged edges in both directions, every tiled kernel and the
    small-output kernel."""
    M, N, K = shape
    W, rank = 3, 1
    out_dtype = torch.bfloat16 if dtype == FP8 else dtype
    ctx = iris.iris(1 << 27, num_ranks=W, rank=rank)
    A, B = _operand((M, K), 17, dtype), _operand((K, N), 18, dtype)
    before = [_operand((M, N), 60 + r, out_dtype, -40, 41) for r in range(W)]
    dA, dB = heap_tensor(ctx, A), heap_tensor(ctx, B)
    dC = ctx.zeros((M, N), dtype=out_dtype)
    cfg = iris.FusedConfig(block_size_m=16, block_size_n=64, block_size_k=16, all_reduce_variant="atomic")
    ws = ops.matmul_all_reduce_preamble(ctx, dC, dA, dB, config=cfg)
    for r in range(W):
        ctx.peer_view(dC, r).copy_(before[r])
    ops.matmul_all_reduce(ctx, dC, dA, dB, config=cfg, workspace=ws, kernel_path="mfma", **_scales(dtype))
    kernel = _lib.last_kernel()
    assert kernel.startswith(f"mfma_{NAMES[dtype]}_{tile}"), kernel
    scale = 0.5 if dtype == FP8 else 1.0
    exp = oracle.matmul_all_reduce(A, B, before, rank, W, 16, 64, "atomic", out_dtype=out_dtype, scale=scale)
    for r, got in enumerate(slot_copies(ctx, dC)):
        assert_bits_equal(got, exp["C"][r], f"{kernel}: C in slot {r}")


def _draw_shape(rng, dtype):
    ce = 16 if dtype == FP8 else 8  # elements per 16 bytes: K and N stay MFMA-eligible
    if rng.random() < 0.15:  # enough tiles for the 256x256 or the two-per-CU builds
        return rng.choice([2304, 2560, 3080]), rng.choice([2048, 3072, 2320]), ce * rng.choice([1, 3, 9])
    M = rng.choice([16, 17, 32, 48, 64, 96, 130, 200, 384, 640, 1000])
    N = rng.choice([64, 80, 144, 272, 528, 1152, 2880])
    K = ce * rng.choice([1, 2, 5, 8, 13, 32, 150])
    return M, N, K


def _sweep_case(rng, case, what):
    op = rng.choice(["all_reduce", "all_reduce", "reduce_scatter", "all_gather_matmul", "matmul_all_gather"])
    dtype = rng.choice([torch.bfloat16, torch.float16, FP8])
    out_dtype = rng.choice([torch.bfloat16, torch.float16]) if dtype == FP8 else dtype
    layout = rng.choice(["nn", "nt"])
    W = rng.choice([1, 2, 3, 4, 8])
    rank = rng.randrange(W)
    M, N, K = _draw_shape(rng, dtype)
    bm = rng.choice([16, 32, 64, 128])
    bn = rng.choice([32, 64, 128])
    bm, bn = min(bm, M), min(bn, N)
    scale = 0.5 if dtype == FP8 else 1.0
    kw = _scales(dtype)
    # the MFMA builds pair e4m3 inputs with a bfloat16 output; e4m3 -> float16 takes the generic kernel
    family = "generic_" if (dtype == FP8 and out_dtype == torch.float16) else "mfma_"
    what = f"{what}: {op} {NAMES[dtype]}->{out_dtype} {layout} W={W} rank={rank} {M}x{N}x{K} flags {bm}x{bn}"
    print(what, flush=True)
    ctx = iris.iris(1 << 27, num_ranks=W, rank=rank)
    seed = 10000 + 50 * case

    if op in ("all_reduce", "reduce_scatter"):
        A, B = _operand((M, K), seed, dtype), _operand((K, N), seed + 1, dtype)
        peers = [randn_cpu((M, N), seed + 2 + r, out_dtype) for r in range(W)]
        dA, dB = heap_tensor(ctx, A), _device_b(ctx, B, layout)
        dC = ctx.zeros((M, N), dtype=out_dtype)
        if op == "all_reduce":
            variant = rng.choice(["one_shot", "two_shot", "atomic"])
            mode = rng.choice(["fp32", "reference"])
            cfg = iris.FusedConfig(block_size_m=bm, block_size_n=bn, block_size_k=1, all_reduce_variant=variant)
            ws = ops.matmul_all_reduce_preamble(ctx, dC, dA, dB, config=cfg)
            if variant == "atomic":
                before = [_operand((M, N), seed + 20 + r, out_dtype, -40, 41) for r in range(W)]
                for r in range(W):
                    ctx.peer_view(dC, r).copy_(before[r])
                ops.matmul_all_reduce(ctx, dC, dA, dB, config=cfg, workspace=ws, **kw)
                exp = oracle.matmul_all_reduce(A, B, before, rank, W, bm, bn, "atomic", out_dtype=out_dtype, scale=scale)
            else:
                stage_peers(ctx, ws, peers)
                ops.matmul_all_reduce(ctx, dC, dA, dB, config=cfg, workspace=ws, slot_sum=mode, **kw)
                exp = oracle.matmul_all_reduce(A, B, peers, rank, W, bm, bn, variant, mode, out_dtype=out_dtype, scale=scale)
            what += f" {variant} {mode}"
        else:
            all_owners = rng.random() < 0.3
            cfg = iris.FusedConfig(block_size_m=bm, block_size_n=bn, block_size_k=1)
            for r in range(W):
                ctx.peer_view(dC, r).zero_()
            ws = ops.matmul_reduce_scatter(ctx, dC, dA, dB, config=cfg, all_owners=all_owners,
                                           stage=lambda w: stage_peers(ctx, w, peers), **kw)
            exp = oracle.matmul_reduce_scatter(A, B, peers, rank, W, bm, bn, out_dtype=out_dtype, scale=scale,
                                               all_owners=all_owners)
            what += f" all_owners={all_owners}"
        kernel = _lib.last_kernel()
        assert kernel.startswith(family), f"{what}: {kernel}"
        if exp["aux"] is not None:
            assert_bits_equal(ws.aux_buffer.cpu(), exp["aux"], f"{what}: {kernel} aux")
            assert torch.equal(ws.locks.cpu(), torch.from_numpy(exp["locks"])), f"{what}: flags"
        for r, got in enumerate(slot_copies(ctx, dC)):
            assert_bits_equal(got, exp["C"][r], f"{what}: {kernel} C in slot {r}")
        return kernel

    if op == "all_gather_matmul":
        gather_dim = rng.choice([0, 1])
        if gather_dim == 1:
            K_local = K
            shards = [_operand((M, K_local), seed + r, dtype) for r in range(W)]
            rows = M
        else:
            M_local = rng.choice([128, 256, 512])  # row gathering: whole kernel tiles per source slot
            shards = [_operand((M_local, K), seed + r, dtype) for r in range(W)]
            rows = M_local * W
            bm = min(bm, M_local)
        Kt = K * W if gather_dim == 1 else K
        B = _operand((Kt, N), seed + 30, dtype)
        bias = _operand((rows,), seed + 31, out_dtype, -8, 9) if rng.random() < 0.5 else None
        dA = ctx.zeros(tuple(shards[0].shape), dtype=dtype)
        for r in range(W):
            ctx.peer_view(dA, r).copy_(shards[r])
        dB = _device_b(ctx, B, layout)
        dbias = heap_tensor(ctx, bias) if bias is not None else None
        out = ctx.zeros((rows, N), dtype=out_dtype)
        cfg = iris.FusedConfig(block_size_m=bm, block_size_n=bn, block_size_k=1)
        ops.all_gather_matmul(ctx, out, dA, dB, bias=dbias, config=cfg, gather_dim=gather_dim, **kw)
        kernel = _lib.last_kernel()
        assert kernel.startswith(family), f"{what}: {kernel}"
        exp = oracle.all_gather_matmul(shards, B, bias=bias, gather_dim=gather_dim, out_dtype=out_dtype, scale=scale)
        assert_bits_equal(out.cpu(), exp, f"{what}: gather_dim={gather_dim} bias={bias is not None} {kernel}")
        return kernel

    # matmul_all_gather
    if M * W * N * 2 > (1 << 26):  # the gathered output must fit the heap slot
        W = 2
        rank = rank % W
        ctx = iris.iris(1 << 27, num_ranks=W, rank=rank)
    A, B = _operand((M, K), seed, dtype), _operand((K, N), seed + 1, dtype)
    bias = _operand((M,), seed + 2, out_dtype, -8, 9) if rng.random() < 0.5 else None
    dA, dB = heap_tensor(ctx, A), _device_b(ctx, B, layout)
    dbias = heap_tensor(ctx, bias) if bias is not None else None
    out = ctx.zeros((M * W, N), dtype=out_dtype)
    for r in range(W):
        ctx.peer_view(out, r).zero_()
    cfg = iris.FusedConfig(block_size_m=bm, block_size_n=bn, block_size_k=1)
    ops.matmul_all_gather(ctx, out, dA, dB, bias=dbias, config=cfg, **kw)
    kernel = _lib.last_kernel()
    assert kernel.startswith(family), f"{what}: {kernel}"
    exp = oracle.matmul_all_gather(A, B, rank, W, bias=bias, out_dtype=out_dtype, scale=scale)
    for r, got in enumerate(slot_copies(ctx, out)):
        assert_bits_equal(got, exp[r], f"{what}: bias={bias is not None} {kernel} slot {r}")
    return kernel


@pytest.mark.parametrize("seed", [101, 102, 103, 104, 105, 106])
def test_seeded_sweep_over_all_operators(seed):
    """50 draws per seed (300 in all) over operator, element type (fp8 included), layout of B, world
    size, rank, shape, flag-tile size, variant, sum rule, bias and gather direction."""
    rng = random.Random(seed)
    kernels = set()
    for case in range(50):
        kernels.add(_sweep_case(rng, case, f"seed {seed} case {case}"))
        torch.cuda.empty_cache()
    assert len(kernels) >= 6, kernels  # several element types, tile shapes and layouts were met
