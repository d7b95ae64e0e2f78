"""The benchmark harness without a GPU: sweep order, overrides, skips, metrics and the three output
formats, with the context and the timer injected.  Formats and flags are those of the reference's
iris.bench (iris/bench/_runner.py:170-312, 399-520)."""

import csv
import io
import json

import pytest
import torch

import iris_amd.bench as bench
from iris_amd.bench import harness


class FakeContext:
    def __init__(self, heap_size, world_size, rank):
        self.heap_size, self.world_size, self.rank = heap_size, world_size, rank
        self.barriers = 0

    def get_num_ranks(self):
        return self.world_size

    def get_rank(self):
        return self.rank

    def barrier(self):
        self.barriers += 1


def fake_timer(fn, barrier_fn, preamble_fn, n_warmup, n_repeat, return_mode):
    assert return_mode == "all"
    for _ in range(1 + n_warmup + n_repeat):
        preamble_fn()
        fn()
    return [2.0] * n_repeat  # milliseconds


def _defs():
    calls = []

    @bench.axis("num_ranks", [2, 8])
    @bench.axis("M", [128, 256])
    @bench.axis("dtype", [torch.float16, torch.bfloat16])
    def gemm_like(state, ctx):
        M = state["M"]
        if M == 256 and state["dtype"] == torch.bfloat16:
            state.skip("too big")
        state.set_flops(4e9 * M)
        state.set_bytes(1e6 * ctx.get_num_ranks())
        state.add_counter("tiles", M / 128)
        state.set_repeat(3)
        state.exec(lambda: calls.append(("run", M)), preamble_fn=lambda: calls.append(("pre", M)))

    @bench.axis("N", [1, 2])
    def no_rank_axis(state, ctx):
        state.exec(lambda: None)

    defs = [harness.BenchmarkDef("gemm_like", gemm_like, gemm_like._bench_axes),
            harness.BenchmarkDef("no_rank_axis", no_rank_axis, no_rank_axis._bench_axes)]
    return defs, calls


def _run(**kw):
    defs, calls = _defs()
    kw.setdefault("n_warmup", 1)
    kw.setdefault("n_repeat", 5)
    return bench.run_registered(defs, make_context=FakeContext, time_fn=fake_timer, **kw), calls


def test_sweep_order_metrics_and_skip():
    results, calls = _run()
    rows = [r for r in results if r.benchmark_name == "gemm_like"]
    # worlds ascending, then the outermost declared axis slowest
    assert [(r.world_size, r.params["M"], r.params["dtype"]) for r in rows] == [
        (w, m, d) for w in (2, 8) for m in (128, 256) for d in (torch.float16, torch.bfloat16)]
    assert list(rows[0].params) == ["num_ranks", "M", "dtype"]
    first = rows[0]
    assert first.gpu_time_ms == 2.0 and len(first.all_times_ms) == 3  # set_repeat(3) wins over n_repeat
    assert first.tflops == pytest.approx(4e9 * 128 / 1e12 / 2e-3)
    assert first.bandwidth_gbps == pytest.approx(1e6 * 2 / 1e9 / 2e-3)
    assert first.counters == {"tiles": 1.0}
    skipped = [r for r in rows if r.skipped]
    assert len(skipped) == 2 and skipped[0].skip_reason == "too big" and skipped[0].all_times_ms == []
    # 1 cold + 1 warm-up + 3 timed calls, each preceded by the preamble
    assert calls[:10] == [("pre", 128), ("run", 128)] * 5
    # a benchmark without a num_ranks axis runs at the default world of 8 only, without that column
    plain = [r for r in results if r.benchmark_name == "no_rank_axis"]
    assert [r.world_size for r in plain] == [8, 8] and list(plain[0].params) == ["N"]


def test_overrides_skips_and_filter():
    results, _ = _run(axis_overrides={"M": [512], "num_ranks": [4]}, skip_overrides={"dtype": [torch.bfloat16]},
                      benchmark_filter="gemm")
    assert [(r.world_size, r.params["M"], r.params["dtype"]) for r in results] == [(4, 512, torch.float16)]
    results, _ = _run(axis_overrides={"num_ranks": [2]}, benchmark_filter="no_rank")
    assert [r.params for r in results] == [{"num_ranks": 2, "N": 1}, {"num_ranks": 2, "N": 2}]
    results, _ = _run(skip_overrides={"M": [128, 256]}, benchmark_filter="gemm")
    assert results == []
    results, _ = _run(rank=3, benchmark_filter="gemm")  # rank 3 does not exist in a world of 2
    assert {r.world_size for r in results} == {8}


def test_parse_axis_values():
    p = harness.parse_axis_values
    assert p("1024,2048", "M") == [1024, 2048]
    assert p("pow2:8:12", "M") == [256, 512, 1024, 2048, 4096]
    assert p("lin:64:256:64", "M") == [64, 128, 192, 256]
    assert p("fp16,bf16", "dtype") == [torch.float16, torch.bfloat16]
    assert p("float32", "x") == [torch.float32]
    assert p("0.5,1", "alpha") == [0.5, 1.0]
    assert p("two_shot,one_shot", "variant") == ["two_shot", "one_shot"]
    with pytest.raises(ValueError, match="expected format 'pow2:start:stop'"):
        p("pow2:8", "M")
    with pytest.raises(ValueError, match="Non-integer values"):
        p("lin:a:b:c", "M")
    with pytest.raises(ValueError, match="Unknown dtype"):
        p("fp12", "dtype")


def test_console_json_csv_formats():
    results, _ = _run(benchmark_filter="gemm", axis_overrides={"num_ranks": [2]})
    text = harness.format_console(results)
    lines = text.splitlines()
    assert lines[0] == "" and lines[1] == "gemm_like"
    assert lines[2].split() == ["num_ranks", "M", "dtype", "GPU", "Time", "(ms)", "BW", "(GB/s)", "TFLOPS", "tiles"]
    assert lines[3].split() == ["2", "128", "float16", "2.000", "1.0", "256.0", "1.000"]
    assert "(skipped) too big" in lines[6]
    assert len({len(l) for l in lines[2:6]}) == 1, "columns are right-aligned to a common width"

    records = json.loads(harness.format_json(results))
    assert set(records[0]) == {"benchmark", "world_size", "params", "gpu_time_ms", "all_times_ms", "bandwidth_gbps",
                               "tflops", "counters"}
    assert records[0]["params"] == {"num_ranks": "2", "M": "128", "dtype": "float16"}
    assert records[3]["skipped"] is True and records[3]["skip_reason"] == "too big"

    table = list(csv.DictReader(io.StringIO(harness.format_csv(results))))
    assert list(table[0]) == ["benchmark", "world_size", "num_ranks", "M", "dtype", "gpu_time_ms", "bandwidth_gbps",
                              "tflops", "tiles", "skipped", "skip_reason"]
    assert table[0]["gpu_time_ms"] == "2.0000" and table[0]["tflops"] == "256.00" and table[3]["gpu_time_ms"] == ""


def test_missing_exec_is_an_error():
    def forgot(state, ctx):
        pass

    with pytest.raises(RuntimeError, match="did not call state.exec"):
        bench.run_registered([harness.BenchmarkDef("forgot", forgot, [])], make_context=FakeContext, time_fn=fake_timer)


def test_range_helpers_and_registration():
    assert bench.power_of_two(3, 5) == [8, 16, 32] and bench.linear_range(2, 8, 3) == [2, 5, 8]
    before = len(harness._registry)

    @bench.register
    @bench.axis("a", [1])
    @bench.axis("b", [2])
    def sample(state, ctx):
        pass

    assert len(harness._registry) == before + 1
    assert [ax.name for ax in harness._registry[-1].axes] == ["a", "b"]  # declaration order = sweep order
    harness._registry.pop()


def test_a_benchmarks_tensors_are_gone_before_the_next_context_is_made():
    """Every benchmark gets a heap of its own, and a heap lives as long as its last tensor: what one
    benchmark allocated - also what the callables it registered hold on to - must be released before
    the next benchmark's context is created, or the heaps pile up (3 x 128 GiB does not fit a GPU)."""
    import weakref

    import iris_amd as iris

    allocated, alive_at_creation = [], []

    def make_context(heap_size, world_size, rank):
        alive_at_creation.append(sum(ref() is not None for ref in allocated))
        return iris.iris(1 << 20, num_ranks=world_size, rank=rank, device="cpu")

    def make_benchmark(name):
        @bench.axis("num_ranks", [2])
        @bench.axis("M", [64, 128])
        def fn(state, ctx):
            x = ctx.zeros((state["M"], 32), dtype=torch.float32)
            y = ctx.zeros((state["M"], 32), dtype=torch.float32)
            allocated.extend([weakref.ref(x), weakref.ref(y)])
            state.exec(lambda: y.copy_(x), preamble_fn=y.zero_)
        return harness.BenchmarkDef(name, fn, fn._bench_axes)

    results = harness.run_registered([make_benchmark("first"), make_benchmark("second"), make_benchmark("third")],
                                     make_context=make_context, time_fn=fake_timer, n_warmup=1, n_repeat=2)
    assert len(results) == 6
    assert alive_at_creation == [0, 0, 0]
    assert all(ref() is None for ref in allocated)
