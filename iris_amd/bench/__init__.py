"""Declarative benchmark harness with the surface of the reference's iris.bench
(iris/bench/__init__.py, _core.py, _runner.py): benchmark files written for it run unchanged with

    import iris_amd.bench as bench

    @bench.register
    @bench.axis("num_ranks", [2, 4, 8])
    @bench.axis("M", bench.power_of_two(8, 13))
    def my_benchmark(state, ctx):
        ...                         # set-up, untimed
        state.set_flops(2 * M * N * K)
        state.exec(lambda: ctx.ops.matmul_all_reduce(C, A, B), preamble_fn=reset)

    if __name__ == "__main__":
        bench.main()

The difference is the execution model: the reference spawns `num_ranks` processes, one per GPU; here
one process times the launch of ONE rank (`--rank`, default 0) on one MI355X whose heap has
`num_ranks` slots, with the other ranks marked as finished (see Iris.stand_in_peers).  Timing,
command-line flags, axis overrides and the console / JSON / CSV output formats are the reference's.
"""

from .harness import (AxisDef, BenchmarkDef, Result, State, axis, linear_range, main, power_of_two, register,
                      run_registered)

__all__ = ["AxisDef", "BenchmarkDef", "Result", "State", "axis", "linear_range", "main", "power_of_two", "register",
           "run_registered"]
