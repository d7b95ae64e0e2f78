"""Decode / hybrid / prefill shapes of benchmark/ops/bench_matmul_all_reduce_stages.py:50-103 of the
reference: M in {32, 896, 2048}, N = 2880, K = 4096 split over the ranks, float16; the fused operator
over variant x flag-tile sizes, and the unfused pair (torch.mm, then the stand-alone all-reduce over
the heap in place of the reference's RCCL call, which needs the other GPUs)."""

import torch

import iris_amd.bench as bench
from iris_amd.ccl import Config
from iris_amd.ops import FusedConfig, matmul_all_reduce_preamble

from ._common import reset_workspace


@bench.register
@bench.axis("num_ranks", [2, 4, 8])
@bench.axis("M", [32, 896, 2048])
@bench.axis("N", [2880])
@bench.axis("K", [4096])
@bench.axis("dtype", [torch.float16])
def unfused_mm_allreduce(state, ctx):
    M, N, dtype = state["M"], state["N"], state["dtype"]
    K_local = state["K"] // ctx.get_num_ranks()
    A = torch.randn((M, K_local), device="cuda", dtype=dtype)
    B = torch.randn((K_local, N), device="cuda", dtype=dtype)
    partial = ctx.zeros((M, N), dtype=dtype)
    C = ctx.zeros((M, N), dtype=dtype)
    config = Config(all_reduce_variant="one_shot")
    workspace = ctx.ccl.all_reduce_preamble(C, partial, config=config)
    state.set_flops(2 * M * N * K_local)

    def run():
        torch.mm(A, B, out=partial)
        workspace.prepared = True
        ctx.ccl.all_reduce(C, partial, config=config, workspace=workspace, async_op=True)

    state.exec(run)


@bench.register
@bench.axis("num_ranks", [2, 4, 8])
@bench.axis("M", [32, 896, 2048])
@bench.axis("N", [2880])
@bench.axis("K", [4096])
@bench.axis("dtype", [torch.float16])
@bench.axis("variant", ["atomic", "two_shot", "one_shot"])
@bench.axis("bm", [32, 64, 128])
@bench.axis("bn", [64, 128])
def fused_gemm_allreduce(state, ctx):
    M, N, dtype, bm, bn = state["M"], state["N"], state["dtype"], state["bm"], state["bn"]
    K_local = state["K"] // ctx.get_num_ranks()
    if bm > M:
        state.skip(f"bm={bm} > M={M}")
    if bn > N:
        state.skip(f"bn={bn} > N={N}")
    A = ctx.zeros((M, K_local), dtype=dtype)
    A.fill_(0.01 * (ctx.get_rank() + 1))
    B = torch.randn((K_local, N), device="cuda", dtype=dtype)
    C = ctx.zeros((M, N), dtype=dtype)
    config = FusedConfig(block_size_m=bm, block_size_n=bn, block_size_k=64, group_size_m=4, num_xcds=8,
                         all_reduce_variant=state["variant"])
    workspace = matmul_all_reduce_preamble(ctx, C, A, B, config=config)
    state.set_flops(2 * M * N * K_local)
    state.exec(lambda: ctx.ops.matmul_all_reduce(C, A, B, config=config, workspace=workspace),
               preamble_fn=reset_workspace(C, workspace))


if __name__ == "__main__":
    bench.main()
