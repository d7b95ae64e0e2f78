"""CPU restatement of the rank-local semantics of Iris's fused GEMM+collective operators.

THIS IS TEST INFRASTRUCTURE.  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg
may import it, and only as the checker or the reported CPU baseline.  Nothing under iris_amd/ uses it.

It restates, with torch on the CPU (numpy for the integer index math), what one rank of a W-rank job
computes and where it puts it.  Every function cites the reference code it follows
(paths relative to the reference repository root).

Parity status of each function (what pins it, see tests/test_oracle.py):
  bump_offsets, context_tensor, translate      pinned: closed-form KATs from the reference allocator
                                                 arithmetic (allocators/torch_allocator.py:102-132) and
                                                 tests/unittests/test_device_context.py:478-492
  tile_id, owner_two_shot, owner_reduce_scatter pinned: the ownership loops the reference's own tests
                                                 restate (tests/ops/test_matmul_reduce_scatter.py:48-54,
                                                 73-81; tests/context/test_reduce_scatter.py:94-100)
  gemm                                          pinned: brute-force triple loop on small integers and
                                                 torch.matmul; the reference tests pin the GEMM only to
                                                 "allclose to torch.matmul" (tests/ops/*.py) because the
                                                 arithmetic lives in tritonblas (pyproject.toml:24), which
                                                 is not in the reference tree.  Bit-exact fp32 summation
                                                 order of the reference GEMM: parity unpinned.
  slot_sum                                      pinned: closed form "rank r contributes r+1 => W(W+1)/2"
                                                 (tests/context/test_all_reduce.py:245-246,352-356) and
                                                 a KAT that separates the fp32 rule from the reference's
                                                 data-type rule
  matmul_all_reduce / matmul_reduce_scatter /
  all_gather_matmul / matmul_all_gather         pinned: W=1 reduces to gemm; closed-form peers; the
                                                 reference tests' checks (torch.cat(shards, 1) @ B,
                                                 tests/ops/test_all_gather_matmul.py:61-66)
  flag contents                                 source-pinned only (no reference test asserts them):
                                                 parity unpinned by tests
  ccl_owned_tiles, ccl_tile_coords              pinned: partition property (every tile owned exactly once
                                                 over the ranks, both distributions), bijection of the
                                                 grouped order, and hand-worked small grids
  ccl_all_reduce / ccl_reduce_scatter           pinned: closed form "rank r holds r+1 => W(W+1)/2"
                                                 (tests/ccl/test_all_reduce.py:55,92-97), equality with a
                                                 plain fp32 sum for exactly representable data, and the
                                                 one-shot order against a sequential Python sum.  The
                                                 rotated start rank of two-shot is pinned by a literal
                                                 replay of the reference's program loop (pid over
                                                 COMM_SMS, start = pid % W) on order-sensitive fp32 data
                                                 and by hand-worked known answers per start rank
  quantize_e4m3 / fp8 products                  no reference counterpart (the reference has no fp8
                                                 path): defined by the target configuration itself (e4m3fn inputs with
                                                 per-tensor scales amax/448, fp32 accumulation), parity unpinned
"""

import math

import numpy as np
import torch

# ----------------------------------------------------------------------------------------------
# Heap and addressing
# ----------------------------------------------------------------------------------------------


def bump_offsets(requests, alignment=1024):
    """Offsets handed out by the bump allocator for a sequence of (num_elements, element_size).

    iris/host/memory/allocators/torch_allocator.py:102-132:
        aligned = ceil(nbytes / alignment) * alignment; start = heap_offset; heap_offset += aligned
    """
    offsets, cursor = [], 0
    for num_elements, element_size in requests:
        nbytes = num_elements * element_size
        offsets.append(cursor)
        cursor += math.ceil(nbytes / alignment) * alignment
    return offsets, cursor


def context_tensor(rank, world, heap_bases):
    """int64 [rank, W, base_0..base_{W-1}, 17 zeros]  (iris/host/iris.py:916-958, tracing off)."""
    return np.array([rank, world] + [int(b) for b in heap_bases] + [0] * 17, dtype=np.int64)


def translate(ptr, from_rank, to_rank, heap_bases):
    """Address of `ptr` (inside from_rank's heap) in to_rank's heap, uint64 arithmetic.

    iris/mem/triton/context.py:16-27:  to_base + (ptr - from_base)
    """
    mask = (1 << 64) - 1
    offset = (int(ptr) - int(heap_bases[from_rank])) & mask
    return (int(heap_bases[to_rank]) + offset) & mask


# ----------------------------------------------------------------------------------------------
# Tiles, flags, owners
# ----------------------------------------------------------------------------------------------


def cdiv(a, b):
    return (a + b - 1) // b


def tile_grid(M, N, block_m, block_n):
    """(tiles_m, tiles_n) of the flag-tile grid (iris/ops/matmul_all_reduce.py:318-320)."""
    return cdiv(M, block_m), cdiv(N, block_n)


def tile_id(pid_m, pid_n, tiles_n):
    """Row-major tile number (iris/ops/matmul_all_reduce.py:87-90,134)."""
    return pid_m * tiles_n + pid_n


def tile_bounds(t, M, N, block_m, block_n):
    """Row and column range of tile t, clipped to the matrix (iris/mem/triton/types.py:21-55)."""
    tiles_n = cdiv(N, block_n)
    pm, pn = divmod(t, tiles_n)
    return pm * block_m, min((pm + 1) * block_m, M), pn * block_n, min((pn + 1) * block_n, N)


def owner_two_shot(t, world):
    """iris/mem/triton/context.py:817:  tile_id % world_size."""
    return t % world


def owner_reduce_scatter(t, total_tiles, world):
    """iris/mem/triton/context.py:972-979: rank r owns [r*tpr, (r+1)*tpr), the last rank also the
    remainder, with tpr = total_tiles // world."""
    tpr = total_tiles // world
    for r in range(world):
        start = r * tpr
        end = total_tiles if r == world - 1 else start + tpr
        if start <= t < end:
            return r
    raise AssertionError("unreachable")


def owner_map(M, N, block_m, block_n, world, kind):
    """int32 [M, N]: which rank reduces each element.  kind: "one_shot" (-1: every rank),
    "two_shot", "reduce_scatter"."""
    tiles_m, tiles_n = tile_grid(M, N, block_m, block_n)
    total = tiles_m * tiles_n
    out = np.full((M, N), -1, dtype=np.int32)
    if kind == "one_shot":
        return out
    for t in range(total):
        r0, r1, c0, c1 = tile_bounds(t, M, N, block_m, block_n)
        out[r0:r1, c0:c1] = owner_two_shot(t, world) if kind == "two_shot" else owner_reduce_scatter(t, total, world)
    return out


# ----------------------------------------------------------------------------------------------
# Arithmetic
# ----------------------------------------------------------------------------------------------


def gemm(A, B, out_dtype=None, scale=1.0, bias=None):
    """fp32-accumulated product, cast once: `acc.to(C.dtype)`
    (iris/ops/matmul_all_reduce.py:105-111; bias as in iris/ops/all_gather_matmul.py:147-153)."""
    out_dtype = out_dtype or A.dtype
    acc = A.to(torch.float32) @ B.to(torch.float32)
    if scale != 1.0:
        acc = acc * scale
    if bias is not None:
        acc = acc + bias.to(torch.float32)[:, None]
    return acc.to(out_dtype)


def gemm_bruteforce(A, B):
    """Triple loop in Python floats (float64), for tiny matrices only."""
    M, K = A.shape
    _, N = B.shape
    a, b = A.to(torch.float64).tolist(), B.to(torch.float64).tolist()
    return torch.tensor([[sum(a[i][k] * b[k][j] for k in range(K)) for j in range(N)] for i in range(M)],
                        dtype=torch.float64)


def slot_sum(own, peers, mode="fp32"):
    """Sum of the own tile and the peers' tiles, in ascending peer order.

    iris/mem/triton/context.py:752-763:
        acc_dtype = fp32 if data is fp16 else the data dtype
        acc = own.to(acc_dtype); for each peer: acc += peer.to(acc_dtype); result = acc.to(dtype)
    mode "reference" follows that rule (bf16 data is re-rounded to bf16 after every add);
    mode "fp32" always carries the sum in fp32 and casts once.
    """
    dtype = own.dtype
    if mode == "fp32" or dtype in (torch.float16, torch.float32):
        acc = own.to(torch.float32)
        for p in peers:
            acc = acc + p.to(torch.float32)
        return acc.to(dtype)
    if mode != "reference":
        raise ValueError(mode)
    acc = own.clone()
    for p in peers:
        acc = (acc.to(torch.float32) + p.to(torch.float32)).to(dtype)
    return acc


def quantize_e4m3(x):
    """Per-tensor quantisation to OCP e4m3fn: scale = amax / 448, q = (x / scale) rounded to e4m3."""
    scale = float(x.abs().max()) / 448.0
    if scale == 0.0:
        scale = 1.0
    q = (x.to(torch.float32) / scale).to(torch.float8_e4m3fn)
    return q, scale


# ----------------------------------------------------------------------------------------------
# The three operators, as seen by one rank
# ----------------------------------------------------------------------------------------------


def matmul_all_reduce(A, B, peer_aux, rank, world, block_m, block_n, variant, mode="fp32", out_dtype=None,
                      scale=1.0):
    """What rank `rank` leaves behind after matmul_all_reduce.

    peer_aux: list of W tensors [M, N] (entry `rank` ignored): the peers' aux buffers.
    Returns dict(aux=own aux, locks=int32 flags, C=list of W tensors or None):
        C[r] is what this rank wrote into rank r's C (zeros where it wrote nothing; the preamble
        zeroes C, iris/ops/matmul_all_reduce.py:215).
    iris/ops/matmul_all_reduce.py:86-144; iris/mem/triton/context.py:733-764 (one_shot), 801-839 (two_shot).
    """
    out_dtype = out_dtype or A.dtype
    M, N = A.shape[0], B.shape[1]
    own = gemm(A, B, out_dtype, scale)
    if variant == "atomic":
        # iris/mem/triton/context.py:689-702: the own tile is atomically added to C on every rank
        # (one add in the data type per element).  peer_aux[r], if given, is what C of rank r held before.
        C = []
        for r in range(world):
            before = peer_aux[r] if peer_aux is not None and peer_aux[r] is not None else torch.zeros(M, N, dtype=out_dtype)
            C.append((before.to(torch.float32) + own.to(torch.float32)).to(out_dtype))
        return dict(aux=None, locks=None, C=C)
    tiles_m, tiles_n = tile_grid(M, N, block_m, block_n)
    locks = np.ones(tiles_m * tiles_n, dtype=np.int32)
    peers = [peer_aux[r] for r in range(world) if r != rank]
    reduced = slot_sum(own, peers, mode)
    C = [torch.zeros(M, N, dtype=out_dtype) for _ in range(world)]
    if variant == "one_shot":
        C[rank] = reduced
    elif variant == "two_shot":
        mine = torch.from_numpy(owner_map(M, N, block_m, block_n, world, "two_shot") == rank)
        for r in range(world):
            C[r] = torch.where(mine, reduced, C[r])
    else:
        raise ValueError(variant)
    return dict(aux=own, locks=locks, C=C)


def matmul_reduce_scatter(A, B, peer_aux, rank, world, block_m, block_n, mode="fp32", out_dtype=None, scale=1.0,
                          all_owners=False, sum_peers=True):
    """What rank `rank` leaves behind after matmul_reduce_scatter.

    iris/ops/matmul_reduce_scatter.py:74-118; iris/mem/triton/context.py:953-997: the tiles this rank
    owns are summed over all ranks and stored into its own C at their global coordinates.
    all_owners / sum_peers: the single-GPU switches of the HIP library (every tile reduced, tile t
    stored into C of slot owner(t); peers skipped).
    """
    out_dtype = out_dtype or A.dtype
    M, N = A.shape[0], B.shape[1]
    own = gemm(A, B, out_dtype, scale)
    tiles_m, tiles_n = tile_grid(M, N, block_m, block_n)
    locks = np.ones(tiles_m * tiles_n, dtype=np.int32)
    peers = [peer_aux[r] for r in range(world) if r != rank] if sum_peers else []
    reduced = slot_sum(own, peers, mode)
    owners = torch.from_numpy(owner_map(M, N, block_m, block_n, world, "reduce_scatter"))
    C = [torch.zeros(M, N, dtype=out_dtype) for _ in range(world)]
    if all_owners:
        for r in range(world):
            C[r] = torch.where(owners == r, reduced, C[r])
    else:
        C[rank] = torch.where(owners == rank, reduced, C[rank])
    return dict(aux=own, locks=locks, C=C)


def all_gather_matmul(shards, B, bias=None, gather_dim=1, out_dtype=None, scale=1.0):
    """out = all_gather(shards) @ B (+ bias[:, None]).

    iris/ops/all_gather_matmul.py:94-159: the reduction runs over rank 0's K_local columns, then
    rank 1's, ...; this equals torch.cat(shards, dim=1) @ B, the check of
    tests/ops/test_all_gather_matmul.py:61-66.  gather_dim=0 concatenates rows instead.
    """
    A = torch.cat(list(shards), dim=1 if gather_dim == 1 else 0)
    return gemm(A, B, out_dtype or A.dtype, scale, bias)


def matmul_all_gather(A, B, rank, world, bias=None, out_dtype=None, scale=1.0):
    """What rank `rank` writes: its product block into rows [rank*M_local, (rank+1)*M_local) of the
    gathered (M, N) output of every rank; rows of other ranks are left alone (returned as zeros).

    iris/ops/matmul_all_gather.py:77-105; iris/mem/triton/context.py:841-864 (dim = 0).  The
    reference test compares with torch.cat(all_gather(A_r @ B), dim=0)
    (tests/ops/test_matmul_all_gather.py:59-66).
    """
    out_dtype = out_dtype or A.dtype
    M_local, N = A.shape[0], B.shape[1]
    block = gemm(A, B, out_dtype, scale, bias)
    out = []
    for _ in range(world):
        full = torch.zeros(M_local * world, N, dtype=out_dtype)
        full[rank * M_local:(rank + 1) * M_local] = block
        out.append(full)
    return out


# ----------------------------------------------------------------------------------------------
# Error measure used by the parity tests
# ----------------------------------------------------------------------------------------------


# ----------------------------------------------------------------------------------------------
# Stand-alone collectives (iris.ccl)
# ----------------------------------------------------------------------------------------------


def ccl_tile_coords(tile, tiles_m, tiles_n, group_m):
    """(pid_m, pid_n) of tile id `tile` in the grouped order.

    iris/ccl/triton/all_reduce.py:639-644:
        num_pid_in_group = GROUP_SIZE_M * num_pid_n; group_id = tile_id // num_pid_in_group
        first_pid_m = group_id * GROUP_SIZE_M; group_size_m = min(num_pid_m - first_pid_m, GROUP_SIZE_M)
        pid_m = first_pid_m + ((tile_id % num_pid_in_group) % group_size_m)
        pid_n = (tile_id % num_pid_in_group) // group_size_m
    """
    per_group = group_m * tiles_n
    group = tile // per_group
    first = group * group_m
    size = min(tiles_m - first, group_m)
    return first + (tile % per_group) % size, (tile % per_group) // size


def ccl_owned_tiles(total_tiles, group_rank, world, distribution):
    """Tile ids rank `group_rank` reduces, in the order j = 0, 1, ... the kernel's loop meets them.

    iris/ccl/triton/all_reduce.py:620-633 (the same lines in iris/ccl/triton/reduce_scatter.py:58-70):
    distribution 0 strides (rank, rank+W, ...), distribution 1 takes ceil(T/W) consecutive tiles.
    """
    per_rank = cdiv(total_tiles, world)
    if distribution == 0:
        return list(range(group_rank, total_tiles, world))
    start = group_rank * per_rank
    return list(range(start, min(start + per_rank, total_tiles)))


def _ccl_cast_sum(slices, order, from_zero):
    acc = torch.zeros_like(slices[0], dtype=torch.float32) if from_zero else None
    for r in order:
        x = slices[r].to(torch.float32)
        acc = x.clone() if acc is None else acc + x
    return acc


def ccl_all_reduce(inputs, outputs, group_rank, variant, block_m=32, block_n=64, group_m=4, comm_sms=64,
                   distribution=1):
    """What the launch of rank `group_rank` leaves in every rank's output.

    inputs / outputs: lists (one entry per rank of the group, group order) of (M, N) tensors; outputs
    are the contents before the launch and are not modified.  Returns the new list of outputs.

    one_shot (iris/ccl/triton/all_reduce.py:401-422): acc = zeros fp32; acc += input of rank i for
        i = 0..W-1; own output = cast(acc).
    two_shot (:646-684): for the j-th owned tile, start = pid % W where the loop gives
        j = pid (mod COMM_SMS); acc = fp32(input[start]); acc += input[(start+i) % W], i = 1..W-1;
        cast once; stored to the output of every rank.
    atomic (:210-233): the own input is added into every rank's output (in the output's type).
    """
    world = len(inputs)
    M, N = inputs[0].shape
    dtype = inputs[0].dtype
    outs = [o.clone() for o in outputs]
    if variant == "atomic":
        for r in range(world):
            outs[r] = (outs[r].to(torch.float32) + inputs[group_rank].to(torch.float32)).to(dtype)
        return outs
    if variant == "one_shot":
        outs[group_rank] = _ccl_cast_sum(inputs, range(world), True).to(dtype)
        return outs
    if variant != "two_shot":
        raise ValueError(variant)
    reduced = ccl_reduce_scatter(inputs, outputs[group_rank], group_rank, block_m, block_n, group_m, comm_sms,
                                 distribution, _mask_out=True)
    tile, mask = reduced
    for r in range(world):
        outs[r] = torch.where(mask, tile, outs[r])
    return outs


def ccl_reduce_scatter(inputs, output, group_rank, block_m=32, block_n=64, group_m=4, comm_sms=64, distribution=1,
                       _mask_out=False):
    """The own output after the launch of rank `group_rank`: owned tiles hold the cast fp32 sum, the
    rest keeps `output` (iris/ccl/triton/reduce_scatter.py:72-118; same reduction as two-shot
    all-reduce, stored to the own rank only)."""
    world = len(inputs)
    M, N = inputs[0].shape
    dtype = inputs[0].dtype
    tiles_m, tiles_n = cdiv(M, block_m), cdiv(N, block_n)
    out = output.clone()
    mask = torch.zeros((M, N), dtype=torch.bool)
    for j, tile in enumerate(ccl_owned_tiles(tiles_m * tiles_n, group_rank, world, distribution)):
        pid_m, pid_n = ccl_tile_coords(tile, tiles_m, tiles_n, group_m)
        rows = slice(pid_m * block_m, min((pid_m + 1) * block_m, M))
        cols = slice(pid_n * block_n, min((pid_n + 1) * block_n, N))
        start = (j % comm_sms) % world
        order = [(start + i) % world for i in range(world)]
        acc = _ccl_cast_sum([x[rows, cols] for x in inputs], order, False)
        out[rows, cols] = acc.to(dtype)
        mask[rows, cols] = True
    return (out, mask) if _mask_out else out


def rel_frobenius(x, ref):
    x, ref = x.to(torch.float64), ref.to(torch.float64)
    denom = float(torch.linalg.norm(ref))
    return float(torch.linalg.norm(x - ref)) / (denom if denom > 0 else 1.0)
