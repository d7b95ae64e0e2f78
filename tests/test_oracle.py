"""The CPU oracle against everything that pins it without the GPU: the golden index-math vectors,
closed forms from the reference's tests, brute force on tiny inputs, and torch library routines.
A mistake in the oracle (a dropped term, a swapped index, a wrong rounding point) fails one of these.
"""

import json
import os

import numpy as np
import pytest
import torch

from helpers import oracle, randint_cpu, randn_cpu

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "index_math.json")))


# -- index math against the golden vectors ---------------------------------------------------------
@pytest.mark.parametrize("case", GOLDEN["ownership_reduce_scatter"], ids=lambda c: f"{c['M']}x{c['N']}_W{c['world']}")
def test_reduce_scatter_ownership_matches_reference_tests(case):
    M, N, bm, bn, W = case["M"], case["N"], case["block_m"], case["block_n"], case["world"]
    tiles_m, tiles_n = oracle.tile_grid(M, N, bm, bn)
    total = tiles_m * tiles_n
    assert total == case["total_tiles"]
    owners = [oracle.owner_reduce_scatter(t, total, W) for t in range(total)]
    omap = oracle.owner_map(M, N, bm, bn, W, "reduce_scatter")
    for rank_s, tiles in case["owned"].items():
        rank = int(rank_s)
        mine = [t for t in range(total) if owners[t] == rank]
        if isinstance(tiles, dict):
            assert len(mine) == tiles["count"]
            assert mine[0] == tiles["first"][0] and mine[-1] == tiles["last"][0]
            rows = np.where((omap == rank).any(axis=1))[0]
            assert [int(rows.min()), int(rows.max()) + 1] == tiles["rows"]
            checks = [tiles["first"], tiles["last"]]
        else:
            assert mine == [t[0] for t in tiles]
            checks = tiles
        for tile_id, r0, r1, c0, c1 in checks:
            assert oracle.tile_bounds(tile_id, M, N, bm, bn) == (r0, r1, c0, c1)
            assert (omap[r0:r1, c0:c1] == rank).all()
    assert sorted(set(owners)) == sorted({o for o in owners})  # every tile has exactly one owner


def test_config4_row_blocks():
    """8192 x 4096 with 256 x 64 tiles and W = 8: rank r owns exactly rows [1024 r, 1024 (r + 1))."""
    omap = oracle.owner_map(8192, 4096, 256, 64, 8, "reduce_scatter")
    for r in range(8):
        assert (omap[1024 * r:1024 * (r + 1)] == r).all()


@pytest.mark.parametrize("case", GOLDEN["ownership_two_shot"], ids=lambda c: f"{c['M']}x{c['N']}_W{c['world']}")
def test_two_shot_ownership(case):
    total, W = case["total_tiles"], case["world"]
    assert oracle.tile_grid(case["M"], case["N"], case["block_m"], case["block_n"]) == (
        oracle.cdiv(case["M"], case["block_m"]), oracle.cdiv(case["N"], case["block_n"]))
    for rank_s, tiles in case["owned"].items():
        mine = [t for t in range(total) if oracle.owner_two_shot(t, W) == int(rank_s)]
        assert mine[:24] == tiles and len(mine) == case["owned_count"][rank_s]


def test_tile_id_is_row_major():
    assert oracle.tile_id(0, 0, 7) == 0 and oracle.tile_id(0, 6, 7) == 6 and oracle.tile_id(1, 0, 7) == 7
    assert oracle.tile_id(3, 2, 64) == 194
    assert oracle.tile_bounds(194, 4096, 4096, 256, 64) == (768, 1024, 128, 192)
    assert oracle.tile_bounds(11, 100, 72, 32, 24) == (96, 100, 48, 72)  # ragged last row of tiles


def test_bump_allocator_offsets():
    g = GOLDEN["bump_allocator"]
    offsets, end = oracle.bump_offsets([tuple(r) for r in g["requests"]], g["alignment"])
    assert offsets == g["offsets"] and end == g["end"]


def test_context_tensor_and_translate():
    g = GOLDEN["context_tensor"]
    assert oracle.context_tensor(g["rank"], g["world"], g["heap_bases"]).tolist() == g["expected"]
    for t in GOLDEN["translate"]:
        assert oracle.translate(t["ptr"], t["from"], t["to"], t["heap_bases"]) == t["expected"]
    # translation is its own inverse and the identity within a rank
    bases = [1 << 40, 3 << 40, 2 << 40]
    p = (1 << 40) + 12345
    assert oracle.translate(oracle.translate(p, 0, 2, bases), 2, 0, bases) == p
    assert oracle.translate(p, 0, 0, bases) == p


# -- arithmetic --------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_gemm_against_brute_force(dtype):
    A, B = randint_cpu((9, 7), 1, dtype), randint_cpu((7, 5), 2, dtype)
    assert torch.equal(oracle.gemm(A, B).double(), oracle.gemm_bruteforce(A, B))
    # an asymmetric case catches a transposed operand: A (2x3) @ B (3x4)
    A = torch.tensor([[1., 2., 3.], [4., 5., 6.]], dtype=dtype)
    B = torch.tensor([[1., 0., 2., 1.], [0., 1., 1., 0.], [3., 0., 0., 1.]], dtype=dtype)
    assert oracle.gemm(A, B).tolist() == [[10., 2., 4., 4.], [22., 5., 13., 10.]]


def test_gemm_rounds_once_from_fp32():
    """The product is accumulated in fp32 and cast once: summing 512 copies of 1 + 2^-7 gives 516,
    while a bf16 accumulator gets stuck at 512."""
    K = 512
    A = torch.full((1, K), 1.0 + 2 ** -7, dtype=torch.bfloat16)
    B = torch.full((K, 1), 1.0, dtype=torch.bfloat16)
    assert float(oracle.gemm(A, B)) == float(torch.tensor(K * (1.0 + 2 ** -7)).to(torch.bfloat16))
    acc = torch.zeros((), dtype=torch.bfloat16)
    for _ in range(K):
        acc = (acc + A[0, 0]).to(torch.bfloat16)
    assert float(acc) != float(oracle.gemm(A, B))  # the wrong (bf16-accumulated) answer differs
    A32, B32 = randn_cpu((33, 65), 5, torch.float32), randn_cpu((65, 17), 6, torch.float32)
    assert torch.allclose(oracle.gemm(A32, B32), torch.matmul(A32, B32), rtol=1e-5, atol=1e-5)


def test_gemm_bias_is_per_row_and_scale_applies_before_cast():
    A, B = randint_cpu((4, 6), 3, torch.float32), randint_cpu((6, 3), 4, torch.float32)
    bias = torch.tensor([10., 20., 30., 40.])
    assert torch.equal(oracle.gemm(A, B, bias=bias), A @ B + bias[:, None])
    assert torch.equal(oracle.gemm(A, B, scale=0.5), (A @ B) * 0.5)


@pytest.mark.parametrize("W", [c["world"] for c in GOLDEN["closed_form_all_reduce"]])
@pytest.mark.parametrize("mode", ["fp32", "reference"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_slot_sum_closed_form(W, mode, dtype):
    expected = {c["world"]: c["value"] for c in GOLDEN["closed_form_all_reduce"]}[W]
    for rank in range(W):
        own = torch.full((8, 8), float(rank + 1), dtype=dtype)
        peers = [torch.full((8, 8), float(r + 1), dtype=dtype) for r in range(W) if r != rank]
        assert torch.all(oracle.slot_sum(own, peers, mode) == expected)


def test_slot_sum_modes_differ_where_they_should():
    """1 + 2^-8 + 2^-8: exact in fp32 (-> 1 + 2^-7 in bf16) but each bf16 add ties back to 1."""
    own = torch.tensor([1.0], dtype=torch.bfloat16)
    peers = [torch.tensor([2.0 ** -8], dtype=torch.bfloat16)] * 2
    assert float(oracle.slot_sum(own, peers, "fp32")) == 1.0 + 2 ** -7
    assert float(oracle.slot_sum(own, peers, "reference")) == 1.0
    # fp16 data is summed in fp32 under both rules (acc_dtype = fp32 iff fp16)
    own16 = torch.tensor([1.0], dtype=torch.float16)
    peers16 = [torch.tensor([2.0 ** -12], dtype=torch.float16)] * 2
    assert float(oracle.slot_sum(own16, peers16, "reference")) == float(oracle.slot_sum(own16, peers16, "fp32"))
    # order: own first, then peers ascending (fp32 addition is not associative)
    a, b, c = torch.tensor([1e8]), torch.tensor([-1e8]), torch.tensor([1.0])
    assert float(oracle.slot_sum(a, [b, c])) == 1.0 and float(oracle.slot_sum(a, [c, b])) == 0.0


def test_quantize_e4m3():
    x = torch.tensor([448.0, -224.0, 1.0, 0.0, 0.4])
    q, s = oracle.quantize_e4m3(x)
    assert s == 1.0 and q.dtype == torch.float8_e4m3fn
    assert q.float().tolist()[:4] == [448.0, -224.0, 1.0, 0.0]
    assert abs(float(q[4].float()) - 0.4) <= 0.4 * 2 ** -4  # 3 mantissa bits
    q2, s2 = oracle.quantize_e4m3(x * 3)
    assert s2 == 3.0 and torch.equal(q2.float(), q.float())


# -- operators ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("variant", ["one_shot", "two_shot"])
def test_all_reduce_world_of_one_is_gemm(variant):
    A, B = randn_cpu((64, 32), 0, torch.float16), randn_cpu((32, 48), 1, torch.float16)
    out = oracle.matmul_all_reduce(A, B, [None], 0, 1, 32, 16, variant)
    assert torch.equal(out["C"][0], oracle.gemm(A, B)) and torch.equal(out["aux"], out["C"][0])
    assert out["locks"].tolist() == [1] * 6


def test_all_reduce_matches_torch_sum_over_ranks():
    """The reference's acceptance check: torch.matmul + all_reduce(SUM) (tests/ops/test_matmul_all_reduce.py:57-62)."""
    W, M, N, K = 4, 64, 48, 32
    As = [randn_cpu((M, K), 10 + r, torch.float32) for r in range(W)]
    B = randn_cpu((K, N), 99, torch.float32)
    partials = [a @ B for a in As]
    total = sum(partials)
    for rank in range(W):
        out = oracle.matmul_all_reduce(As[rank], B, partials, rank, W, 32, 16, "one_shot")
        assert torch.allclose(out["C"][rank], total, rtol=1e-5, atol=1e-5)
        two = oracle.matmul_all_reduce(As[rank], B, partials, rank, W, 32, 16, "two_shot")
        mine = torch.from_numpy(oracle.owner_map(M, N, 32, 16, W, "two_shot") == rank)
        for r in range(W):
            assert torch.allclose(two["C"][r][mine], total[mine], rtol=1e-5, atol=1e-5)
            assert torch.all(two["C"][r][~mine] == 0)
    # the union over ranks of what two-shot writes covers C exactly once
    cover = sum((torch.from_numpy(oracle.owner_map(M, N, 32, 16, W, "two_shot") == r)).int() for r in range(W))
    assert torch.all(cover == 1)


def test_reduce_scatter_matches_reference_acceptance():
    """tests/ops/test_matmul_reduce_scatter.py:73-89: each owned tile equals the all-reduced product."""
    W, M, N, K, bm, bn = 4, 128, 128, 32, 64, 64
    A, B = randn_cpu((M, K), 0, torch.float32), randn_cpu((K, N), 1, torch.float32)
    partial = A @ B
    case = [c for c in GOLDEN["ownership_reduce_scatter"] if (c["M"], c["world"]) == (128, 4)][0]
    for rank in range(W):
        out = oracle.matmul_reduce_scatter(A, B, [partial] * W, rank, W, bm, bn)
        for tile_id, r0, r1, c0, c1 in case["owned"][str(rank)]:
            assert torch.allclose(out["C"][rank][r0:r1, c0:c1], W * partial[r0:r1, c0:c1], rtol=1e-5, atol=1e-5)
        other = torch.from_numpy(oracle.owner_map(M, N, bm, bn, W, "reduce_scatter") != rank)
        assert torch.all(out["C"][rank][other] == 0)
        for r in range(W):
            if r != rank:
                assert torch.all(out["C"][r] == 0)
    allo = oracle.matmul_reduce_scatter(A, B, None, 0, W, bm, bn, all_owners=True, sum_peers=False)
    assert torch.equal(sum(allo["C"]), oracle.gemm(A, B))  # the slots partition the product


def test_all_gather_matmul_both_layouts():
    W = 4
    shards = [randint_cpu((6, 5), 42 + r, torch.float16) for r in range(W)]
    B = randint_cpu((20, 7), 123, torch.float16)
    assert torch.equal(oracle.all_gather_matmul(shards, B), (torch.cat(shards, 1).float() @ B.float()).half())
    # K order: shard r multiplies rows [5r, 5r+5) of B
    manual = sum(shards[r].float() @ B[5 * r:5 * r + 5].float() for r in range(W)).half()
    assert torch.equal(oracle.all_gather_matmul(shards, B), manual)
    B2 = randint_cpu((5, 7), 124, torch.float16)
    rows = oracle.all_gather_matmul(shards, B2, gather_dim=0)
    for r in range(W):
        assert torch.equal(rows[6 * r:6 * r + 6], (shards[r].float() @ B2.float()).half())


def test_matmul_all_gather_rows():
    """torch.cat(all_gather(A_r @ B), dim=0) (tests/ops/test_matmul_all_gather.py:59-66 of the reference)."""
    W, M_local, K, N = 4, 6, 5, 7
    As = [randint_cpu((M_local, K), 30 + r, torch.float16) for r in range(W)]
    B = randint_cpu((K, N), 40, torch.float16)
    expected = torch.cat([(a.float() @ B.float()).half() for a in As], dim=0)
    total = [torch.zeros(W * M_local, N, dtype=torch.float16) for _ in range(W)]
    for rank in range(W):
        written = oracle.matmul_all_gather(As[rank], B, rank, W)
        for r in range(W):
            total[r] += written[r]  # every rank writes a disjoint row block into every rank's output
    for r in range(W):
        assert torch.equal(total[r], expected)
    bias = torch.arange(M_local, dtype=torch.float16)
    with_bias = oracle.matmul_all_gather(As[2], B, 2, W, bias=bias)[0]
    assert torch.equal(with_bias[12:18], ((As[2].float() @ B.float()) + bias.float()[:, None]).half())
    assert torch.all(with_bias[:12] == 0) and torch.all(with_bias[18:] == 0)


def test_all_reduce_atomic_variant():
    """Every rank adds its product into every rank's C: after all ranks, C = sum of the products."""
    W, M, N, K = 4, 8, 8, 8
    As = [randint_cpu((M, K), 50 + r, torch.float32) for r in range(W)]
    B = randint_cpu((K, N), 60, torch.float32)
    C = [torch.zeros(M, N) for _ in range(W)]
    for rank in range(W):
        C = oracle.matmul_all_reduce(As[rank], B, C, rank, W, 4, 4, "atomic")["C"]
    for r in range(W):
        assert torch.equal(C[r], sum(a @ B for a in As))


# ------------------------------------------------------------------------------------------------
# Stand-alone collectives
# ------------------------------------------------------------------------------------------------
def test_ccl_grouped_order_hand_worked():
    # 3 x 2 tiles, groups of 2 tile-rows: the first group is walked column by column (two rows per
    # column), the last group has a single row.
    got = [oracle.ccl_tile_coords(t, 3, 2, 2) for t in range(6)]
    assert got == [(0, 0), (1, 0), (0, 1), (1, 1), (2, 0), (2, 1)]
    # one tile-row per group is plain row-major order
    assert [oracle.ccl_tile_coords(t, 2, 3, 1) for t in range(6)] == [(0, 0), (0, 1), (0, 2), (1, 0), (1, 1), (1, 2)]


@pytest.mark.parametrize("tiles_m,tiles_n,group_m", [(1, 1, 4), (5, 3, 4), (8, 8, 4), (7, 2, 3), (4, 9, 6)])
def test_ccl_grouped_order_is_a_bijection(tiles_m, tiles_n, group_m):
    seen = {oracle.ccl_tile_coords(t, tiles_m, tiles_n, group_m) for t in range(tiles_m * tiles_n)}
    assert seen == {(m, n) for m in range(tiles_m) for n in range(tiles_n)}


@pytest.mark.parametrize("distribution", [0, 1])
@pytest.mark.parametrize("total,world", [(1, 4), (7, 4), (8, 8), (33, 8), (64, 3), (5, 16)])
def test_ccl_ownership_partitions_the_tiles(total, world, distribution):
    owned = [oracle.ccl_owned_tiles(total, r, world, distribution) for r in range(world)]
    flat = sorted(t for tiles in owned for t in tiles)
    assert flat == list(range(total)), "every tile reduced by exactly one rank"
    if distribution == 0:
        assert all(t % world == r for r, tiles in enumerate(owned) for t in tiles)
    else:
        per = -(-total // world)
        assert all(t // per == r for r, tiles in enumerate(owned) for t in tiles)


@pytest.mark.parametrize("variant", ["one_shot", "two_shot", "atomic"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_ccl_all_reduce_closed_form(variant, dtype):
    # tests/ccl/test_all_reduce.py:55: rank r holds r+1 everywhere, so every element is W(W+1)/2
    W, M, N = 8, 128, 128
    inputs = [torch.full((M, N), float(r + 1), dtype=dtype) for r in range(W)]
    outs = [torch.zeros((M, N), dtype=dtype) for _ in range(W)]
    for r in range(W):  # every rank runs its launch
        outs = oracle.ccl_all_reduce(inputs, outs, r, variant, block_m=32, block_n=32, distribution=r % 2 if variant != "two_shot" else 0)
    for r in range(W):
        assert torch.all(outs[r] == W * (W + 1) / 2)


@pytest.mark.parametrize("distribution", [0, 1])
def test_ccl_two_shot_over_all_ranks_is_the_plain_sum(distribution):
    W, M, N = 4, 100, 72  # ragged against 32 x 64 tiles
    g = torch.Generator().manual_seed(5)
    inputs = [torch.randint(-8, 9, (M, N), generator=g).to(torch.bfloat16) for _ in range(W)]
    outs = [torch.full((M, N), -1.0, dtype=torch.bfloat16) for _ in range(W)]
    for r in range(W):
        outs = oracle.ccl_all_reduce(inputs, outs, r, "two_shot", distribution=distribution)
    want = sum(x.float() for x in inputs).to(torch.bfloat16)  # small integers: exact in any order
    for r in range(W):
        assert torch.equal(outs[r], want)
    # reduce-scatter: each rank's owned tiles agree with the sum, the rest is untouched
    covered = torch.zeros((M, N), dtype=torch.int32)
    for r in range(W):
        own = oracle.ccl_reduce_scatter(inputs, torch.full((M, N), -1.0, dtype=torch.bfloat16), r, distribution=distribution)
        touched = own != -1.0
        assert torch.equal(own[touched], want[touched])
        covered += touched.int()
    assert torch.all(covered[want != -1.0] == 1)


def test_ccl_one_shot_adds_in_group_order_from_zero():
    # fp32 values whose sum depends on the order: 2^24 + 1 + 1 - 2^24
    vals = [2.0 ** 24, 1.0, 1.0, -(2.0 ** 24)]
    inputs = [torch.full((4, 8), v, dtype=torch.float32) for v in vals]
    outs = [torch.zeros((4, 8)) for _ in vals]
    got = oracle.ccl_all_reduce(inputs, outs, 2, "one_shot")[2]
    acc = np.float32(0.0)
    for v in vals:
        acc = np.float32(acc + np.float32(v))
    assert acc == 0.0 and torch.all(got == float(acc))  # the two ones are absorbed one at a time
    # -0.0 in every slot comes out as +0.0 because the accumulator starts from +0.0
    neg = [torch.full((2, 8), -0.0, dtype=torch.bfloat16) for _ in range(4)]
    out = oracle.ccl_all_reduce(neg, [torch.ones((2, 8), dtype=torch.bfloat16)] * 4, 0, "one_shot")[0]
    assert torch.all(out.view(torch.int16) == 0)


def test_ccl_two_shot_with_one_workgroup_starts_every_tile_at_rank_zero():
    # comm_sms = 1 makes (j mod comm_sms) mod W zero for every tile: the order is the ascending one
    vals = [2.0 ** 24, 1.0, 1.0, -(2.0 ** 24)]
    inputs = [torch.full((64, 64), v, dtype=torch.float32) for v in vals]
    outs = [torch.zeros((64, 64)) for _ in vals]
    for r in range(4):
        outs = oracle.ccl_all_reduce(inputs, outs, r, "two_shot", block_m=32, block_n=32, comm_sms=1, distribution=0)
    assert all(torch.all(o == 0.0) for o in outs)


def _two_shot_program_replay(inputs, group_rank, block_m, block_n, group_m, comm_sms, distribution):
    """The reference kernel's loop written out program by program
    (iris/ccl/triton/all_reduce.py:602-669): programs pid = 0..COMM_SMS-1, each walking
    range(pid, max_tile_offset, COMM_SMS), every tile summed from start = pid % W going round the
    ranks, element by element in numpy float32.  Shares no code with oracle.ccl_*."""
    W = len(inputs)
    M, N = inputs[0].shape
    x = [t.to(torch.float32).numpy() for t in inputs]
    num_pid_m, num_pid_n = -(-M // block_m), -(-N // block_n)
    total_tiles = num_pid_m * num_pid_n
    tiles_per_rank = -(-total_tiles // W)
    if distribution == 0:
        start_tile, stride = group_rank, W
        max_tile_offset = -(-max(total_tiles - start_tile, 0) // stride)
    else:
        start_tile, stride = group_rank * tiles_per_rank, 1
        max_tile_offset = min(tiles_per_rank, max(total_tiles - start_tile, 0))
    out = np.full((M, N), np.nan, dtype=np.float32)
    for pid in range(comm_sms):
        for tile_offset in range(pid, max_tile_offset, comm_sms):
            tile_id = start_tile + tile_offset * stride
            num_pid_in_group = group_m * num_pid_n
            group_id = tile_id // num_pid_in_group
            first_pid_m = group_id * group_m
            group_size_m = min(num_pid_m - first_pid_m, group_m)
            pid_m = first_pid_m + ((tile_id % num_pid_in_group) % group_size_m)
            pid_n = (tile_id % num_pid_in_group) // group_size_m
            start_rank_idx = pid % W
            for m in range(pid_m * block_m, min((pid_m + 1) * block_m, M)):
                for n in range(pid_n * block_n, min((pid_n + 1) * block_n, N)):
                    acc = np.float32(x[start_rank_idx][m, n])
                    for i in range(1, W):
                        acc = np.float32(acc + x[(start_rank_idx + i) % W][m, n])
                    assert np.isnan(out[m, n]), "an element is reduced by one program only"
                    out[m, n] = acc
    return out


def test_ccl_two_shot_rotation_known_answers():
    # 2^24, -2^24, 0.5, 1 summed cyclically in fp32 gives a different value from every start rank:
    #   start 0: (2^24 - 2^24) + 0.5 + 1               = 1.5
    #   start 1: (-2^24 + 0.5 -> -2^24) + 1 -> -2^24+1 exactly; + 2^24 = 1
    #   start 2: 0.5 + 1 = 1.5; + 2^24 -> 2^24 + 2 (nearest); - 2^24 = 2
    #   start 3: 1 + 2^24 -> 2^24 (tie to even); - 2^24 = 0; + 0.5 = 0.5
    vals = [2.0 ** 24, -(2.0 ** 24), 0.5, 1.0]
    by_start = {0: 1.5, 1: 1.0, 2: 2.0, 3: 0.5}
    W, bm, bn = 4, 2, 4
    M, N = 2, 4 * 24  # one tile-row of 24 tiles, rank 0 owns tiles 0, 4, 8, ... (strided)
    inputs = [torch.full((M, N), v, dtype=torch.float32) for v in vals]
    outs = [torch.zeros((M, N)) for _ in vals]
    for comm_sms in (3, 5):
        got = oracle.ccl_all_reduce(inputs, outs, 0, "two_shot", block_m=bm, block_n=bn, group_m=1,
                                    comm_sms=comm_sms, distribution=0)
        # the j-th owned tile (tile id 4j) is handled by program j mod comm_sms
        for j in range(6):
            want = by_start[(j % comm_sms) % W]
            for r in range(W):  # the owner stores the tile into every rank's output
                assert torch.all(got[r][:, 16 * j:16 * j + 4] == want), (comm_sms, j, r)


@pytest.mark.parametrize("distribution", [0, 1])
@pytest.mark.parametrize("comm_sms", [3, 5])
def test_ccl_two_shot_matches_the_program_loop(comm_sms, distribution):
    W, M, N, bm, bn, gm = 4, 22, 40, 4, 8, 2  # ragged tiles, a short last group
    g = torch.Generator().manual_seed(17)
    # magnitudes spread over 2^0 .. 2^26 with both signs: almost every element's fp32 sum depends on the order
    inputs = [(torch.randn((M, N), generator=g) * 2.0 ** torch.randint(0, 27, (M, N), generator=g).float())
              for _ in range(W)]
    covered = np.zeros((M, N), dtype=np.int32)
    differs = 0
    for rank in range(W):
        want = _two_shot_program_replay(inputs, rank, bm, bn, gm, comm_sms, distribution)
        own = ~np.isnan(want)
        covered += own
        before = torch.full((M, N), -7.0)
        got = oracle.ccl_reduce_scatter(inputs, before, rank, bm, bn, gm, comm_sms, distribution).numpy()
        assert np.array_equal(got[own].view(np.int32), want[own].view(np.int32))
        assert np.all(got[~own] == -7.0)
        outs = oracle.ccl_all_reduce(inputs, [before.clone() for _ in range(W)], rank, "two_shot", bm, bn, gm,
                                     comm_sms, distribution)
        for r in range(W):
            assert np.array_equal(outs[r].numpy()[own].view(np.int32), want[own].view(np.int32))
            assert np.all(outs[r].numpy()[~own] == -7.0)
        ascending = sum(x.numpy().astype(np.float32) for x in inputs)  # fixed start at rank 0
        differs += int(np.sum(ascending[own] != want[own]))
    assert np.all(covered == 1)
    assert differs > 50, "the data must tell the rotated order from the ascending one"


def test_rel_frobenius_known_answers():
    """The yardstick of every tolerance test: ||x - ref||_F / ||ref||_F, worked by hand.
    ref = [[3, 4]] has norm 5; x = ref + [[0.3, -0.4]] is off by a vector of norm 0.5: 0.1.  The measure
    is relative to the SECOND argument (swapping the arguments gives 0.5 / ||x||, another number), is 0
    for equal inputs, sees every element (a single wrong entry of a 2x2 identity: 1 / sqrt(2)), works
    across dtypes in float64, and falls back to the absolute error for a zero reference."""
    ref = torch.tensor([[3.0, 4.0]])
    x = torch.tensor([[3.3, 3.6]])
    assert oracle.rel_frobenius(x, ref) == pytest.approx(0.1, rel=1e-6)
    assert oracle.rel_frobenius(ref, x) == pytest.approx(0.5 / (3.3 ** 2 + 3.6 ** 2) ** 0.5, rel=1e-6)
    assert oracle.rel_frobenius(ref, ref) == 0.0
    eye, bad = torch.eye(2), torch.tensor([[1.0, 0.0], [1.0, 1.0]])
    assert oracle.rel_frobenius(bad, eye) == pytest.approx(2 ** -0.5, rel=1e-12)
    assert oracle.rel_frobenius(torch.tensor([2.5], dtype=torch.bfloat16), torch.tensor([2.0])) == pytest.approx(0.25)
    assert oracle.rel_frobenius(torch.tensor([0.0, 2.0]), torch.zeros(2)) == pytest.approx(2.0)
