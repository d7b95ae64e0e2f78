"""Stand-alone collectives on the grids of benchmark/ccl/bench_all_reduce.py, bench_reduce_scatter.py
and bench_all_reduce_vllm.py of the reference.  `set_bytes` keeps the reference's bus-bandwidth
convention (2(W-1)/W x size for all-reduce, (W-1)/W x size for reduce-scatter) so that the BW column
compares with the reference's; the bytes one rank's launch moves in HBM are a different number."""

import torch

import iris_amd.bench as bench
from iris_amd.ccl import Config

DECODE_MS = [1, 32, 64, 128, 512]
PREFILL_MS = [2048, 4096, 8192]


def _all_reduce_case(state, ctx):
    M, N, dtype = state["M"], state["N"], state["dtype"]
    world = ctx.get_num_ranks()
    inp = ctx.zeros((M, N), dtype=dtype)
    out = ctx.zeros((M, N), dtype=dtype)
    for r in range(world):  # rank r contributes r + 1 everywhere
        ctx.peer_view(inp, r).fill_(float(r + 1))
    state.set_bytes(int(inp.numel() * inp.element_size() * 2 * (world - 1) / world))
    config = Config(all_reduce_variant=state["variant"])
    workspace = ctx.ccl.all_reduce_preamble(out, inp, config=config)

    def reset():
        out.zero_()
        ctx.ccl.all_reduce_preamble(out, inp, config=config, workspace=workspace)

    state.exec(lambda: ctx.ccl.all_reduce(out, inp, config=config, workspace=workspace), preamble_fn=reset)


@bench.register
@bench.axis("num_ranks", [2, 4, 8])
@bench.axis("M", bench.power_of_two(10, 14))
@bench.axis("N", bench.power_of_two(10, 14))
@bench.axis("dtype", [torch.float16, torch.bfloat16])
@bench.axis("variant", ["two_shot"])
def all_reduce(state, ctx):
    _all_reduce_case(state, ctx)


@bench.register
@bench.axis("num_ranks", [8])
@bench.axis("M", DECODE_MS + PREFILL_MS)
@bench.axis("N", [2880])
@bench.axis("dtype", [torch.bfloat16])
@bench.axis("variant", ["two_shot", "one_shot"])
def iris_all_reduce(state, ctx):
    _all_reduce_case(state, ctx)


@bench.register
@bench.axis("num_ranks", [2, 4, 8])
@bench.axis("M", bench.power_of_two(10, 14))
@bench.axis("N", bench.power_of_two(10, 14))
@bench.axis("dtype", [torch.float16, torch.bfloat16])
def reduce_scatter(state, ctx):
    M, N, dtype = state["M"], state["N"], state["dtype"]
    world = ctx.get_num_ranks()
    inp = ctx.zeros((M, N), dtype=dtype)
    out = ctx.zeros((M, N), dtype=dtype)
    for r in range(world):
        ctx.peer_view(inp, r).fill_(0.1 * (r + 1))
    state.set_bytes(int(inp.numel() * inp.element_size() * (world - 1) / world))
    config = Config()
    state.exec(lambda: ctx.ccl.reduce_scatter(out, inp, config=config), preamble_fn=out.zero_)


if __name__ == "__main__":
    bench.main()
