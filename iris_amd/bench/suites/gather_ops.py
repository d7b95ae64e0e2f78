"""all_gather_matmul and matmul_all_gather on the grids of benchmark/ops/bench_all_gather_matmul.py
and benchmark/ops/bench_matmul_all_gather.py of the reference (float16, N = 3584, K = 8192)."""

import torch

import iris_amd.bench as bench
from iris_amd.ops import FusedConfig, all_gather_matmul_preamble


@bench.register
@bench.axis("num_ranks", [2, 4, 8])
@bench.axis("M", [1024, 4096, 16384])
@bench.axis("N", [3584])
@bench.axis("K", [8192])
@bench.axis("dtype", [torch.float16])
def all_gather_matmul(state, ctx):
    M, N, K, dtype = state["M"], state["N"], state["K"], state["dtype"]
    world = ctx.get_num_ranks()
    shard = ctx.zeros((M, K // world), dtype=dtype)
    for r in range(world):  # every rank's shard holds ones, as every process of the reference fills its own
        ctx.peer_view(shard, r).fill_(1.0)
    B = torch.randn((K, N), device="cuda", dtype=dtype)
    C = torch.zeros((M, N), device="cuda", dtype=dtype)
    config = FusedConfig()
    workspace = all_gather_matmul_preamble(ctx, shard, B, config)
    state.set_flops(2 * M * N * K)
    state.set_bytes((world - 1) * shard.numel() * shard.element_size())
    state.exec(lambda: ctx.ops.all_gather_matmul(C, shard, B, config=config, workspace=workspace))


@bench.register
@bench.axis("num_ranks", [2, 4, 8])
@bench.axis("M_local", [1024, 4096, 16384])
@bench.axis("N", [3584])
@bench.axis("K", [8192])
@bench.axis("dtype", [torch.float16])
def matmul_all_gather(state, ctx):
    M_local, N, K, dtype = state["M_local"], state["N"], state["K"], state["dtype"]
    world = ctx.get_num_ranks()
    A = ctx.zeros((M_local, K), dtype=dtype)
    A.fill_(1.0)
    B = torch.randn((K, N), device="cuda", dtype=dtype)
    C = ctx.zeros((M_local * world, N), dtype=dtype)
    config = FusedConfig()
    state.set_flops(2 * M_local * N * K)
    state.set_bytes((world - 1) * M_local * N * A.element_size())
    state.exec(lambda: ctx.ops.matmul_all_gather(C, A, B, config=config), preamble_fn=C.zero_)


if __name__ == "__main__":
    bench.main()
