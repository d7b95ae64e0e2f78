"""The benchmark suites end to end on the GPU, at toy sizes through the command-line entry point."""

import json

import pytest

import iris_amd.bench as bench
from iris_amd.bench import harness

pytestmark = pytest.mark.gpu


def test_suites_run_through_main(capsys):
    before = len(harness._registry)
    from iris_amd.bench.suites import ccl, gather_ops, matmul_all_reduce, matmul_all_reduce_stages  # noqa: F401

    try:
        bench.main(["--benchmark_format=json", "--n_warmup=1", "--n_repeat=3", f"--heap_size={1 << 27}",
                    "--axis_num_ranks=4", "--axis_M=256", "--axis_M_local=256", "--axis_N=256", "--axis_K=512"])
    finally:
        del harness._registry[before:]
    records = json.loads(capsys.readouterr().out)
    names = {r["benchmark"] for r in records}
    assert names == {"matmul_all_reduce", "unfused_mm_allreduce", "fused_gemm_allreduce", "all_gather_matmul",
                     "matmul_all_gather", "all_reduce", "iris_all_reduce", "reduce_scatter"}
    for r in records:
        assert r["world_size"] == 4 and r["params"]["num_ranks"] == "4"
        assert not r.get("skipped"), r
        assert len(r["all_times_ms"]) == 3 and r["gpu_time_ms"] > 0
        assert ("tflops" in r) or ("bandwidth_gbps" in r)
    fused = [r for r in records if r["benchmark"] == "fused_gemm_allreduce"]
    assert len(fused) == 3 * 3 * 2  # variant x bm x bn
