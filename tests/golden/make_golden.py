#!/usr/bin/env python3
"""Writes tests/golden/*.json: small known-answer vectors for the index math of the fused operators.

Every expected value below is computed here from the formulas as the reference's own *tests* state
them (not from the oracle under test), so that the oracle can be checked against them:

  ownership_reduce_scatter   the loop in tests/ops/test_matmul_reduce_scatter.py:48-54,73-81 of the
                             reference (tiles_per_rank = total // W; start = rank * tiles_per_rank; the
                             last rank takes what is left), evaluated for every rank
  ownership_two_shot         tile_id % world_size == rank (iris/mem/triton/context.py:817), enumerated
  bump_allocator             sizes rounded up to 1024 bytes, cumulative
                             (iris/host/memory/allocators/torch_allocator.py:102-132), worked by hand
  closed_form_all_reduce     rank r contributes r + 1 -> W (W + 1) / 2
                             (tests/context/test_all_reduce.py:245-246,352-356)

Run from the repository root:  python tests/golden/make_golden.py
"""

import json
import os

HERE = os.path.dirname(os.path.abspath(__file__))


def reduce_scatter_owned_tiles(M, N, bm, bn, world):
    num_pid_m = (M + bm - 1) // bm
    num_pid_n = (N + bn - 1) // bn
    total_tiles = num_pid_m * num_pid_n
    owned = {}
    for rank in range(world):
        tiles_per_rank = total_tiles // world
        start_tile = rank * tiles_per_rank
        if rank == world - 1:
            tiles_per_rank = total_tiles - start_tile
        tiles = []
        for local_tile_idx in range(tiles_per_rank):
            tile_id = start_tile + local_tile_idx
            pid_m, pid_n = tile_id // num_pid_n, tile_id % num_pid_n
            m_start, n_start = pid_m * bm, pid_n * bn
            tiles.append([tile_id, m_start, min(m_start + bm, M), n_start, min(n_start + bn, N)])
        if len(tiles) > 16:  # keep the fixture small: first and last tile plus the rows covered
            tiles = {"first": tiles[0], "last": tiles[-1], "count": len(tiles),
                     "rows": [min(t[1] for t in tiles), max(t[2] for t in tiles)]}
        owned[str(rank)] = tiles
    return {"M": M, "N": N, "block_m": bm, "block_n": bn, "world": world, "total_tiles": total_tiles, "owned": owned}


def two_shot_owned_tiles(M, N, bm, bn, world):
    total = ((M + bm - 1) // bm) * ((N + bn - 1) // bn)
    return {"M": M, "N": N, "block_m": bm, "block_n": bn, "world": world, "total_tiles": total,
            "owned": {str(r): [t for t in range(total) if t % world == r][:24] for r in range(world)},
            "owned_count": {str(r): len([t for t in range(total) if t % world == r]) for r in range(world)}}


def main():
    cases = {
        "ownership_reduce_scatter": [
            reduce_scatter_owned_tiles(128, 128, 64, 64, w) for w in (1, 2, 4, 8)
        ] + [reduce_scatter_owned_tiles(8192, 4096, 256, 64, 8), reduce_scatter_owned_tiles(640, 256, 64, 64, 8),
             reduce_scatter_owned_tiles(100, 72, 32, 24, 3), reduce_scatter_owned_tiles(64, 64, 64, 64, 4)],
        "ownership_two_shot": [two_shot_owned_tiles(4096, 4096, 256, 64, 8), two_shot_owned_tiles(512, 384, 128, 64, 8),
                               two_shot_owned_tiles(100, 72, 32, 24, 3)],
        # (num_elements, element_size) requests -> offsets; worked by hand: 10 floats = 40 B -> 1024;
        # 300 bf16 = 600 B -> 1024; 1024 int32 = 4096 -> 4096; 1 byte -> 1024; 0 bytes -> 0; 1025 B -> 2048
        "bump_allocator": {
            "alignment": 1024,
            "requests": [[10, 4], [300, 2], [1024, 4], [1, 1], [0, 4], [1025, 1], [7, 8]],
            "offsets": [0, 1024, 2048, 6144, 7168, 7168, 9216],
            "end": 10240,
        },
        "closed_form_all_reduce": [{"world": w, "value": w * (w + 1) // 2} for w in (1, 2, 4, 8)],
        # context tensor: [rank, W, bases..., 17 zeros] (iris/host/iris.py:916-958)
        "context_tensor": {"rank": 3, "world": 4, "heap_bases": [4096, 1052672, 2101248, 3149824],
                           "expected": [3, 4, 4096, 1052672, 2101248, 3149824] + [0] * 17},
        # pointer translation (iris/mem/triton/context.py:16-27): to_base + (ptr - from_base)
        "translate": [
            {"heap_bases": [4096, 1052672, 2101248, 3149824], "ptr": 1052672 + 777, "from": 1, "to": 3, "expected": 3149824 + 777},
            {"heap_bases": [0x7F0000000000, 0x7E0000000000], "ptr": 0x7F0000000400, "from": 0, "to": 1, "expected": 0x7E0000000400},
        ],
    }
    with open(os.path.join(HERE, "index_math.json"), "w") as f:
        json.dump(cases, f, indent=1, sort_keys=True)
    print("wrote", os.path.join(HERE, "index_math.json"))


if __name__ == "__main__":
    main()
