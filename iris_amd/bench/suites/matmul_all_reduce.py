"""Fused GEMM + all-reduce on the grid of benchmark/ops/bench_matmul_all_reduce.py:12-47 of the
reference: M in {1024, 4096, 16384}, N = 3584, K = 8192, float16, variants atomic and two_shot, plus
one_shot.  One rank's launch is timed; the other ranks are marked finished."""

import torch

import iris_amd.bench as bench
from iris_amd.ops import FusedConfig, matmul_all_reduce_preamble

from ._common import reset_workspace


@bench.register
@bench.axis("num_ranks", [2, 4, 8])
@bench.axis("M", [1024, 4096, 16384])
@bench.axis("N", [3584])
@bench.axis("K", [8192])
@bench.axis("dtype", [torch.float16])
@bench.axis("variant", ["atomic", "two_shot", "one_shot"])
def matmul_all_reduce(state, ctx):
    M, N, K, dtype = state["M"], state["N"], state["K"], state["dtype"]
    A = ctx.zeros((M, K), dtype=dtype)
    A.fill_(0.01 * (ctx.get_rank() + 1))
    B = torch.randn((K, N), device="cuda", dtype=dtype)
    C = ctx.zeros((M, N), dtype=dtype)
    config = FusedConfig(all_reduce_variant=state["variant"])
    workspace = matmul_all_reduce_preamble(ctx, C, A, B, config=config)
    state.set_flops(2 * M * N * K)

    def run():
        ctx.ops.matmul_all_reduce(C, A, B, config=config, workspace=workspace)

    state.exec(run, preamble_fn=reset_workspace(C, workspace))


if __name__ == "__main__":
    bench.main()
