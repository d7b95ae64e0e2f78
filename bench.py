#!/usr/bin/env python3
"""Benchmark of the rank-local fused GEMM+collective path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--protocol both|flushed|back_to_back]

Prints ONE JSON line.  A step is one launch of the fused operator on synthetic inputs that already
sit in HBM (peers' partial results and flags staged before the timed region).

Two timing passes:
  * back to back: W untimed steps, then K timed steps between two device synchronisations; `value` is
    the whole-job throughput of those K steps in TFLOP/s (2*M*N*K flop per step, wall clock).  K more
    steps follow with a GPU event pair around every launch (`launch_ms_back_to_back`).
  * flushed, the protocol of the reference's iris.do_bench (iris/host/platform/utils.py:137-201):
    before every launch the device is synchronised, a 256 MB buffer is zeroed to push the previous
    launch's lines out of L2 / last-level cache, the device is synchronised again, and the launch is
    bracketed by GPU events on the launch stream; 25 warm-up and 100 timed launches, mean and median.
A third pass, `launch_ms_flushed_queued`, repeats the flushed launches without the synchronisation
between flush and launch: the launch is queued while the flush kernel still runs, so its event pair
holds the kernel and next to nothing of the host's launch path (5-8 us through Python, ctypes and the
HIP runtime on an idle queue) and agrees with a profiler's kernel duration for the same command.
`roofline` prices those launches (`priced_on`) against the roof that bounds the fused kernel (HBM for
the slot-sum workloads, MFMA for the others); `frac_reference_protocol` (also at the top level of the line,
next to `priced_on`) is the same fraction priced on the literal do_bench launches, host path included; the back-to-back per-launch figures are carried as well;
`gemm_phase` repeats the measurement with the peers switched off (W = 1), which isolates the MFMA
phase; `cpu_baseline` times torch's CPU matmul plus the slot reduction on the same workload.

Default workload: the headline configuration, matmul_all_reduce bf16 M=N=4096, K=1376, W=8.
"""

import argparse
import json
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK = {"hbm": (8000.0, "GB/s"), "bf16": (2500.0, "TFLOP/s"), "fp16": (2500.0, "TFLOP/s"), "fp8": (5000.0, "TFLOP/s")}


def _randn(shape, seed, dtype, scale=1.0, device="cpu"):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * scale).to(dtype)


def _time_cpu(fn, flops, budget_s, sample):
    """Median wall time of fn over 3..10 repetitions within budget_s seconds, as a cpu_baseline record."""
    fn()
    times, t_end = [], time.perf_counter() + budget_s
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 10):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    t = statistics.median(times)
    return {"value": flops / t / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{sample}; {len(times)} reps, median; os.cpu_count={os.cpu_count()}"}


class Workload:
    """One configuration: builds the heap tensors, launches a step, knows its flop and byte counts."""

    name = ""
    dtype = "bf16"

    def setup(self, iris, world):
        raise NotImplementedError

    def step(self):
        raise NotImplementedError


class MatmulAllReduce(Workload):
    def __init__(self, name, M, N, K, fp8=False, block_m=256, variant="one_shot", fp16=False):
        self.name, self.M, self.N, self.K, self.fp8 = name, M, N, K, fp8
        self.block_m, self.variant = block_m, variant
        self.dtype = "fp8" if fp8 else ("fp16" if fp16 else "bf16")
        self.elem = torch.float16 if fp16 else torch.bfloat16  # type of C, aux and the peers' partials
        self.flops = 2 * M * N * K

    def algorithmic_bytes(self, world):
        """Compulsory HBM traffic of one launch: A, B, the peers' tiles this rank reduces, the stores
        of the reduced tiles.  one_shot reduces every tile into the own C; a two_shot rank reduces the
        1/W of the tiles it owns and stores each of them into all W slots.  The aux round trip and the
        flags are not counted."""
        es = 1 if self.fp8 else 2
        mn = self.M * self.N * 2
        ab = self.M * self.K * es + self.K * self.N * es
        if self.variant == "two_shot":
            return ab + (world - 1) * mn // world + world * (mn // world)
        return ab + (world - 1) * mn + mn

    def describe(self, world):
        return {"workload": self.name, "op": "matmul_all_reduce", "variant": self.variant, "M": self.M, "N": self.N,
                "K": self.K, "W": world, "flag_tile": [self.block_m, 64]}

    def setup(self, iris, world):
        from iris_amd import ops
        M, N, K = self.M, self.N, self.K
        heap = 4 * M * N + 2 * (M * K + K * N) + (64 << 20)
        self.ctx = ctx = iris.iris(heap, num_ranks=world, rank=0)
        self.scale = {}
        if self.fp8:
            a, b = _randn((M, K), 0, torch.float32), _randn((K, N), 1, torch.float32)
            sa, sb = float(a.abs().max()) / 448.0, float(b.abs().max()) / 448.0
            A, B = (a / sa).to(torch.float8_e4m3fn), (b / sb).to(torch.float8_e4m3fn)
            self.scale = dict(scale_a=sa, scale_b=sb)
        else:
            g = torch.Generator().manual_seed(0)
            A = (torch.randn((M, K), generator=g) / K ** 0.5).to(self.elem)
            B = (torch.randn((K, N), generator=g) / K ** 0.5).to(self.elem)
        self.A_cpu, self.B_cpu = A, B
        self.A = ctx.zeros((M, K), dtype=A.dtype)
        self.A.copy_(A)
        self.B = ctx.zeros((K, N), dtype=B.dtype)
        self.B.copy_(B)
        self.C = ctx.zeros((M, N), dtype=self.elem)
        self.cfg = iris.FusedConfig(block_size_m=self.block_m, block_size_n=64, block_size_k=64,
                                    all_reduce_variant=self.variant)
        self.ws = ops.matmul_all_reduce_preamble(ctx, self.C, self.A, self.B, config=self.cfg)
        for r in range(1, world):  # synthetic peer partials: N(0,1) from the CPU generator, seed r; flags raised
            ctx.peer_view(self.ws.aux_buffer, r).copy_(_randn((M, N), r, self.elem))
            ctx.peer_view(self.ws.locks, r).fill_(1)
        self._op = ops.matmul_all_reduce
        torch.cuda.synchronize()

    def step(self):
        # The flags and aux written by the previous step are simply overwritten: no reset is needed.
        self.ws.prepared = True
        self._op(self.ctx, self.C, self.A, self.B, async_op=True, config=self.cfg, workspace=self.ws, **self.scale)

    def cpu_baseline(self, world, budget_s=20.0):
        """torch CPU matmul (bf16 in, as the GPU path; fp8 dequantised to fp32) + slot reduction with
        the same seeded peers, on the whole workload when one pass costs well under a second of CPU
        time, else on its first 2048 rows."""
        rows = self.M if self.flops <= 1e11 else min(self.M, 2048)
        A = self.A_cpu[:rows]
        A = A.float() if self.fp8 else A
        B = self.B_cpu.float() if self.fp8 else self.B_cpu
        peers = [_randn((self.M, self.N), r, self.elem)[:rows].contiguous() for r in range(1, world)]

        def once():
            C = torch.matmul(A, B).to(self.elem)
            acc = C.float()
            for p in peers:
                acc += p.float()
            return acc.to(self.elem)

        which = "all" if rows == self.M else "first"
        return _time_cpu(once, 2 * rows * self.N * self.K, budget_s,
                         f"{which} {rows} of {self.M} rows; torch.matmul + fp32 sum of {world} slots")


class AllGatherMatmul(Workload):

    def __init__(self, name, M, N, K, b_transposed=False):
        self.name, self.M, self.N, self.K = name, M, N, K
        self.flops = 2 * M * N * K
        self.b_transposed = b_transposed  # B handed over as the transpose of an (N, K) tensor

    def algorithmic_bytes(self, world):
        return 2 * (self.M * self.K + self.K * self.N + self.M * self.N)

    def describe(self, world):
        return {"workload": self.name, "op": "all_gather_matmul", "gather": "rows", "M": self.M, "N": self.N,
                "K": self.K, "W": world, "B_layout": "K-contiguous" if self.b_transposed else "N-contiguous"}

    def setup(self, iris, world):
        from iris_amd import ops
        M, N, K = self.M, self.N, self.K
        self.ctx = ctx = iris.iris(2 * (M // world * K + K * N + M * N) + (64 << 20), num_ranks=world, rank=0)
        self.A = ctx.zeros((M // world, K), dtype=torch.bfloat16)
        for r in range(world):
            ctx.peer_view(self.A, r).copy_(_randn((M // world, K), r, torch.bfloat16, K ** -0.5))
        if self.b_transposed:
            self.B = ctx.zeros((N, K), dtype=torch.bfloat16)
            self.B.copy_(_randn((K, N), 8, torch.bfloat16, K ** -0.5).t())
            self.B = self.B.t()
        else:
            self.B = ctx.zeros((K, N), dtype=torch.bfloat16)
            self.B.copy_(_randn((K, N), 8, torch.bfloat16, K ** -0.5))
        self.C = ctx.zeros((M, N), dtype=torch.bfloat16)
        self._op = ops.all_gather_matmul
        torch.cuda.synchronize()

    def step(self):
        self._op(self.ctx, self.C, self.A, self.B, async_op=True, gather_dim=0)

    def cpu_baseline(self, world, budget_s=20.0):
        """torch CPU matmul of the first gathered row block (slot 0's rows) with B, bf16 in and out."""
        rows = min(self.M // world, 1024)
        A = _randn((rows, self.K), 0, torch.bfloat16, self.K ** -0.5)
        B = _randn((self.K, self.N), 8, torch.bfloat16, self.K ** -0.5)
        return _time_cpu(lambda: torch.matmul(A, B), 2 * rows * self.N * self.K, budget_s,
                         f"first {rows} of {self.M} rows; torch.matmul bf16")


class MatmulReduceScatter(Workload):
    """accumulate=False: one launch stands in for every rank's reduce step (row block r lands in slot r,
    peers contribute nothing).  accumulate=True: the reference semantics for rank 0 - seven staged peer
    aux buffers, the rank's own row block summed over the slots in fp32 and stored to its C."""


    def __init__(self, name, M, N, K, accumulate=False):
        self.name, self.M, self.N, self.K, self.accumulate = name, M, N, K, accumulate
        self.flops = 2 * M * N * K

    def algorithmic_bytes(self, world):
        ab = 2 * (self.M * self.K + self.K * self.N)
        mn = 2 * self.M * self.N
        if self.accumulate:  # the owned 1/W of the output: W-1 peer blocks read, one block written
            return ab + (world - 1) * (mn // world) + mn // world
        return ab + mn

    def describe(self, world):
        return {"workload": self.name, "op": "matmul_reduce_scatter", "M": self.M, "N": self.N, "K": self.K,
                "W": world, "all_owners": not self.accumulate, "sum_peers": self.accumulate}

    def setup(self, iris, world):
        from iris_amd import _lib
        from iris_amd.ops import FusedConfig, matmul_reduce_scatter_preamble
        from iris_amd.ops._common import current_stream, iris_launch, ptr
        M, N, K = self.M, self.N, self.K
        self.ctx = ctx = iris.iris(2 * (M * K + K * N + 2 * M * N) + (64 << 20), num_ranks=world, rank=0)
        g = torch.Generator().manual_seed(0)
        self.A = ctx.zeros((M, K), dtype=torch.bfloat16)
        self.A.copy_((torch.randn((M, K), generator=g) / K ** 0.5).to(torch.bfloat16))
        self.B = ctx.zeros((K, N), dtype=torch.bfloat16)
        self.B.copy_((torch.randn((K, N), generator=g) / K ** 0.5).to(torch.bfloat16))
        self.C = ctx.zeros((M, N), dtype=torch.bfloat16)
        cfg = FusedConfig()
        ws = matmul_reduce_scatter_preamble(ctx, self.C, self.A, self.B, cfg)
        if self.accumulate:
            for r in range(1, world):  # peers' partial products: bf16 N(0,1), CPU generator, seed r
                ctx.peer_view(ws.aux_buffer, r).copy_(_randn((M, N), r, torch.bfloat16))
                ctx.peer_view(ws.locks, r).fill_(1)
        A, B, C = self.A, self.B, self.C
        all_owners, sum_peers = (0, 1) if self.accumulate else (1, 0)
        # The operator wrapper re-runs its preamble (two barriers, three memsets) on every call, as
        # the reference does; the step times the launch alone, through the same C entry point.
        self._launch = lambda: iris_launch(
            "iris_hip_matmul_reduce_scatter", (ws.locks.numel(),),
            ptr(A), ptr(B), ptr(C), ptr(ws.aux_buffer), ptr(ws.locks), M, N, K,
            A.stride(0), A.stride(1), B.stride(0), B.stride(1), C.stride(0), C.stride(1),
            ptr(ctx.get_device_context()), 0, world, cfg.block_size_m, cfg.block_size_n, cfg.block_size_k,
            all_owners, sum_peers, _lib.BF16, _lib.BF16, 1.0, _lib.ACC_FP32, ctx.spin_limit, ptr(ctx._status),
            _lib.PATH_AUTO, current_stream(ctx), algorithm="matmul_reduce_scatter", rank=0)
        torch.cuda.synchronize()

    def step(self):
        self._launch()

    def cpu_baseline(self, world, budget_s=20.0):
        """torch CPU matmul of the first 1024-row block plus its copy into the owner's output."""
        rows = min(self.M, 1024)
        g = torch.Generator().manual_seed(0)
        A = (torch.randn((rows, self.K), generator=g) / self.K ** 0.5).to(torch.bfloat16)
        B = (torch.randn((self.K, self.N), generator=g) / self.K ** 0.5).to(torch.bfloat16)
        out = torch.empty((rows, self.N), dtype=torch.bfloat16)
        return _time_cpu(lambda: out.copy_(torch.matmul(A, B)), 2 * rows * self.N * self.K, budget_s,
                         f"first {rows} of {self.M} rows; torch.matmul bf16 + row-block copy")


class CopyCalibration(Workload):
    """A plain device-to-device copy of known size: what the HBM byte counters read for it scales the
    counters of the real kernels (profiles/ states the factors)."""

    dtype = "u8"

    def __init__(self, name, nbytes):
        self.name, self.nbytes, self.flops = name, nbytes, 0

    def algorithmic_bytes(self, world):
        return 2 * self.nbytes

    def describe(self, world):
        return {"workload": self.name, "op": "copy", "bytes": self.nbytes}

    def setup(self, iris, world):
        self.ctx = iris.iris(1 << 20, num_ranks=1, rank=0)
        self.src = torch.empty(self.nbytes // 4, dtype=torch.int32, device="cuda").fill_(1)
        self.dst = torch.empty_like(self.src)
        torch.cuda.synchronize()

    def step(self):
        self.dst.copy_(self.src)

    def cpu_baseline(self, world, budget_s=20.0):
        return None


class CclCollective(Workload):
    """Stand-alone all-reduce / reduce-scatter over the heap slots: one rank's launch, no GEMM.  The
    value is reported in TFLOP/s like every other line (one fp32 add per input element), the roofline
    in GB/s of the bytes the launch has to move."""


    def __init__(self, name, op, variant, M, N):
        self.name, self.op, self.variant, self.M, self.N = name, op, variant, M, N

    def _share(self, world):
        return 1.0 if self.variant == "one_shot" else 1.0 / world  # fraction of the tiles the rank reduces

    def algorithmic_bytes(self, world):
        tile_bytes = self.M * self.N * 2 * self._share(world)
        stores = world if (self.op == "all_reduce" and self.variant == "two_shot") else 1
        return int(tile_bytes * (world + stores))

    def describe(self, world):
        return {"workload": self.name, "op": "ccl." + self.op, "variant": self.variant, "M": self.M, "N": self.N,
                "W": world, "tile": [32, 64], "distribution": "block"}

    def setup(self, iris, world):
        from iris_amd.ccl import Config
        M, N = self.M, self.N
        self.flops = int(M * N * world * self._share(world))
        self.ctx = ctx = iris.iris(4 * M * N + (16 << 20), num_ranks=world, rank=0)
        self.x = ctx.zeros((M, N), dtype=torch.bfloat16)
        self.y = ctx.zeros((M, N), dtype=torch.bfloat16)
        gen = torch.Generator(device="cuda").manual_seed(3)
        for r in range(world):
            ctx.peer_view(self.x, r).copy_(torch.randn((M, N), generator=gen, device="cuda").to(torch.bfloat16))
        self.cfg = Config(all_reduce_variant=self.variant)
        self.ws = ctx.ccl.all_reduce_preamble(self.y, self.x, config=self.cfg) if self.op == "all_reduce" else None
        torch.cuda.synchronize()

    def step(self):
        if self.op == "all_reduce":
            self.ws.prepared = True  # the timed step is the launch; zeroing is the preamble's job
            self.ctx.ccl.all_reduce(self.y, self.x, async_op=True, config=self.cfg, workspace=self.ws)
        else:
            self.ctx.ccl.reduce_scatter(self.y, self.x, async_op=True, config=self.cfg)

    def cpu_baseline(self, world, budget_s=20.0):
        return None


WORKLOADS = {
    "copy_calibration_1GiB": lambda: CopyCalibration("copy_calibration_1GiB", 1 << 30),
    "matmul_all_reduce_bf16_4096x4096x1376": lambda: MatmulAllReduce("matmul_all_reduce_bf16_4096x4096x1376", 4096, 4096, 1376),
    "matmul_all_reduce_two_shot_bf16_4096x4096x1376": lambda: MatmulAllReduce(
        "matmul_all_reduce_two_shot_bf16_4096x4096x1376", 4096, 4096, 1376, variant="two_shot"),
    "all_gather_matmul_bf16_8192x1792x4096": lambda: AllGatherMatmul("all_gather_matmul_bf16_8192x1792x4096", 8192, 1792, 4096),
    "all_gather_matmul_bf16_8192x1792x4096_nt": lambda: AllGatherMatmul("all_gather_matmul_bf16_8192x1792x4096_nt", 8192, 1792, 4096, b_transposed=True),
    # 32 x 12 = 384 tiles of 256 x 256: one and a half rounds on 256 CUs (the tail policy's case)
    "all_gather_matmul_bf16_8192x2880x4096": lambda: AllGatherMatmul("all_gather_matmul_bf16_8192x2880x4096", 8192, 2880, 4096),
    "matmul_reduce_scatter_bf16_8192x4096x1376": lambda: MatmulReduceScatter("matmul_reduce_scatter_bf16_8192x4096x1376", 8192, 4096, 1376),
    "matmul_reduce_scatter_accumulate_bf16_8192x4096x1376": lambda: MatmulReduceScatter(
        "matmul_reduce_scatter_accumulate_bf16_8192x4096x1376", 8192, 4096, 1376, accumulate=True),
    "matmul_all_reduce_fp8_16384x8192x1024": lambda: MatmulAllReduce("matmul_all_reduce_fp8_16384x8192x1024", 16384, 8192, 1024, fp8=True),
    "matmul_all_reduce_fp8_skinny_32x8192x1024": lambda: MatmulAllReduce(
        "matmul_all_reduce_fp8_skinny_32x8192x1024", 32, 8192, 1024, fp8=True, block_m=32),
}
for _v in ("one_shot", "two_shot"):
    WORKLOADS[f"ccl_all_reduce_{_v}_bf16_8192x8192"] = (
        lambda v=_v: CclCollective(f"ccl_all_reduce_{v}_bf16_8192x8192", "all_reduce", v, 8192, 8192))
WORKLOADS["ccl_reduce_scatter_bf16_8192x8192"] = (
    lambda: CclCollective("ccl_reduce_scatter_bf16_8192x8192", "reduce_scatter", "two_shot", 8192, 8192))
WORKLOADS["ccl_all_reduce_one_shot_bf16_128x8192"] = (
    lambda: CclCollective("ccl_all_reduce_one_shot_bf16_128x8192", "all_reduce", "one_shot", 128, 8192))
# Shapes of the reference's own benchmark definitions (no published results): fused vs unfused stages
# at decode/prefill sizes (benchmark/ops/bench_matmul_all_reduce_stages.py:50-69: M in {32, 896, 2048},
# N = 2880, K = 4096 / 8 ranks, fp16) and the large grid (benchmark/ops/bench_matmul_all_reduce.py:12-47).
for _m in (32, 896, 2048):
    WORKLOADS[f"matmul_all_reduce_fp16_{_m}x2880x512"] = (
        lambda m=_m: MatmulAllReduce(f"matmul_all_reduce_fp16_{m}x2880x512", m, 2880, 512, fp16=True, block_m=32, variant="two_shot"))
for _m in (1024, 4096, 16384):
    WORKLOADS[f"matmul_all_reduce_fp16_{_m}x3584x8192"] = (
        lambda m=_m: MatmulAllReduce(f"matmul_all_reduce_fp16_{m}x3584x8192", m, 3584, 8192, fp16=True, variant="two_shot"))
DEFAULT = "matmul_all_reduce_bf16_4096x4096x1376"


def bounding_roof(wl, world):
    """"hbm" or "mfma": whichever roof takes longer for this workload at this world size - the
    algorithmic bytes at the HBM peak or the flops at the MFMA peak of the input type.  Workloads without
    matrix products (copies, stand-alone collectives) are HBM-bound."""
    if not getattr(wl, "flops", 0) or wl.dtype not in PEAK:
        return "hbm"
    t_hbm = wl.algorithmic_bytes(world) / (PEAK["hbm"][0] * 1e9)
    t_mfma = wl.flops / (PEAK[wl.dtype][0] * 1e12)
    return "hbm" if t_hbm >= t_mfma else "mfma"


def measured_traffic(workload, world):
    """HBM bytes per launch from the rocprofv3 FETCH_SIZE / WRITE_SIZE runs recorded under profiles/
    (taken with the default W = 8); None when no profile covers this workload."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    if world != 8 or not os.path.exists(path):
        return None
    entry = json.load(open(path)).get("workloads", {}).get(workload)
    return entry["traffic_bytes"] if entry else None


def timed_steps(wl, steps, warmup, graph=False):
    """W untimed steps, then K timed ones between device synchronisations (the wall-clock figure), then K
    more with every launch bracketed by GPU events on the launch stream (the per-launch figures).  With graph=True the K steps are captured into one
    HIP graph after the warm-up and the timed region is one replay of it (no host work between the
    launches; the per-launch time is then the replay time divided by K)."""
    for _ in range(warmup):
        wl.step()
    torch.cuda.synchronize()
    if graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        captured = torch.cuda.CUDAGraph()
        with torch.cuda.graph(captured, stream=side):
            for _ in range(steps):
                wl.step()
        captured.replay()
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        start.record()
        captured.replay()
        end.record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        wl.ctx.check_status()
        return wall, [start.elapsed_time(end) / steps] * steps
    t0 = time.perf_counter()
    for i in range(steps):
        wl.step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    wl.ctx.check_status()
    # The per-launch figures come from a second run of K steps: an event pair around every launch puts
    # two more packets per step on the queue (about 5 us of gaps per step), which the timed region above
    # should not pay for.
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    for i in range(steps):
        starts[i].record()
        wl.step()
        ends[i].record()
    torch.cuda.synchronize()
    wl.ctx.check_status()
    per_launch_ms = [s.elapsed_time(e) for s, e in zip(starts, ends)]
    return wall, per_launch_ms


FLUSH_BYTES = int(256e6)


def flushed_launches(wl, n_warmup=25, n_repeat=100, queued=False):
    """Per-launch GPU-event times in ms under the protocol of the reference's do_bench
    (iris/host/platform/utils.py:137-201): synchronise, zero a 256 MB buffer, synchronise, then the
    launch alone between two events.  Warm-up launches go through the same sequence.

    queued=True leaves out the synchronisation between the flush and the launch: the host then queues
    the events and the launch while the flush kernel still runs, so the event pair holds the kernel and
    next to nothing of the host's launch path - the figure to compare with a profiler's kernel duration."""
    cache = torch.empty(FLUSH_BYTES // 4, dtype=torch.int, device="cuda")
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    for i in range(-n_warmup, n_repeat):
        torch.cuda.synchronize()
        cache.zero_()
        if not queued:
            torch.cuda.synchronize()
        if i < 0:
            wl.step()
            continue
        starts[i].record()
        wl.step()
        ends[i].record()
    torch.cuda.synchronize()
    wl.ctx.check_status()
    del cache
    return [s.elapsed_time(e) for s, e in zip(starts, ends)]


def measure(wl, args):
    """The timing passes for one prepared workload.  Returns (wall seconds of the K back-to-back steps or
    None, back-to-back per-launch ms or None, flushed per-launch ms or None, the same with the launch
    queued behind the flush or None)."""
    wall = b2b = flushed = queued = None
    if args.protocol in ("both", "back_to_back"):
        wall, b2b = timed_steps(wl, args.steps, args.warmup, args.graph)
    if args.protocol in ("both", "flushed"):
        flushed = flushed_launches(wl)
        queued = flushed_launches(wl, n_warmup=5, queued=True)
    return wall, b2b, flushed, queued


def _stats(ms):
    return None if ms is None else {"mean": round(statistics.mean(ms), 5), "median": round(statistics.median(ms), 5),
                                    "min": round(min(ms), 5), "n": len(ms)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=25)
    ap.add_argument("--workload", default=DEFAULT, choices=sorted(WORKLOADS))
    ap.add_argument("--world", type=int, default=8, help="number of heap slots W")
    ap.add_argument("--protocol", default="both", choices=["both", "flushed", "back_to_back"],
                    help="timing passes to run: K back-to-back steps (value), cache-flushed launches (roofline), or both")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-gemm-phase", action="store_true", help="skip the W=1 measurement")
    ap.add_argument("--graph", action="store_true", help="capture the K steps into one HIP graph and time its replay")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build runs the rank-local path of one MI355X "
                 "(the W ranks are heap slots in its HBM); --gpus must be 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")

    import iris_amd as iris
    from iris_amd import _lib

    wl = WORKLOADS[args.workload]()
    wl.setup(iris, args.world)
    wall, b2b, flushed, queued = measure(wl, args)
    kernel = _lib.last_kernel() if not isinstance(wl, CopyCalibration) else "torch copy kernel"
    # The roofline prices the kernel's duration after a cache flush: the flushed launches whose event
    # pairs hold the kernel alone (queued behind the flush), which is what a profiler's kernel average
    # of the same command reads.  The literal do_bench sequence (a host synchronisation between flush
    # and launch, so that the pair also holds the host's launch path) is reported beside it as
    # launch_ms_flushed / frac_do_bench.  Back-to-back launches are priced when only those were run.
    priced = queued if queued is not None else (flushed if flushed is not None else b2b)
    priced_on = "launch_ms_flushed_queued" if queued is not None else ("launch_ms_flushed" if flushed is not None else "launch_ms_back_to_back")
    launch_ms = statistics.mean(priced)
    if wall is not None:
        ms_per_step = wall * 1e3 / args.steps
        tflops = wl.flops * args.steps / wall / 1e12
    else:  # flushed launches only: no back-to-back region, the value is per launch
        ms_per_step = launch_ms
        tflops = wl.flops / (launch_ms * 1e-3) / 1e12

    bytes_alg = wl.algorithmic_bytes(args.world)
    bound = bounding_roof(wl, args.world)
    if bound == "hbm":
        peak, unit = PEAK["hbm"]
        per_ms = bytes_alg / 1e6  # achieved = per_ms / launch_ms, in GB/s
    else:
        peak, unit = PEAK[wl.dtype]
        per_ms = wl.flops / 1e9   # ... or in TFLOP/s
    achieved = per_ms / launch_ms
    frac_reference = round(per_ms / statistics.mean(flushed) / peak, 4) if flushed is not None else None
    roofline = {"bound": bound, "achieved": round(achieved, 2), "peak": peak,
                "unit": unit, "frac": round(achieved / peak, 4), "traffic": measured_traffic(args.workload, args.world),
                "kernel": kernel, "flushed": flushed is not None, "priced_on": priced_on,
                # the same fraction under the reference's literal do_bench sequence (host launch path inside the event pair)
                "frac_reference_protocol": frac_reference, "frac_do_bench": frac_reference,
                "roof_us": {"hbm": round(bytes_alg / PEAK["hbm"][0] / 1e3, 2),
                            "mfma": round(wl.flops / PEAK[wl.dtype][0] / 1e6, 2) if wl.dtype in PEAK else None},
                "launch_ms_mean": round(launch_ms, 5), "launch_ms_median": round(statistics.median(priced), 5),
                "launch_ms_flushed": _stats(flushed), "launch_ms_flushed_queued": _stats(queued),
                "launch_ms_back_to_back": _stats(b2b),
                "algorithmic_bytes": bytes_alg, "algorithmic_flops": wl.flops}

    out = {
        "metric": "TFLOP/s and % of MI355X MFMA peak, rank-local fused GEMM+epilogue, 1 GPU",
        "value": round(tflops, 3),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": wl.dtype,
        "data": "synthetic",
        "launch_mode": ("hip graph replay" if args.graph else "eager") if wall is not None else "flushed launches only",
        "config": wl.describe(args.world),
        "pct_of_mfma_peak": round(100 * tflops / PEAK[wl.dtype][0], 2) if wl.dtype in PEAK else None,
        "roofline": roofline,
        # which launches roofline.frac is priced on, and the same fraction under the reference's literal protocol
        "priced_on": priced_on,
        "frac_reference_protocol": frac_reference,
    }

    if isinstance(wl, MatmulAllReduce) and not args.no_gemm_phase:
        del wl.ctx, wl
        torch.cuda.empty_cache()
        solo = WORKLOADS[args.workload]()
        solo.setup(iris, 1)  # W = 1: same kernel and shape (aux, flags and C still written), no peers to sum
        wall1, b2b1, flushed1, queued1 = measure(solo, args)
        priced1 = queued1 if queued1 is not None else (flushed1 if flushed1 is not None else b2b1)
        t1 = solo.flops / (statistics.mean(priced1) * 1e-3) / 1e12  # per launch, like the roofline
        gp = {"world": 1, "tflops": round(t1, 3), "frac_of_mfma_peak": round(t1 / PEAK[solo.dtype][0], 4),
              "frac_of_mfma_peak_do_bench": (round(solo.flops / (statistics.mean(flushed1) * 1e-3) / 1e12 / PEAK[solo.dtype][0], 4)
                                             if flushed1 is not None else None),
              "flushed": flushed1 is not None, "launch_ms_flushed": _stats(flushed1),
              "launch_ms_flushed_queued": _stats(queued1),
              "launch_ms_back_to_back": _stats(b2b1), "kernel": _lib.last_kernel()}
        if wall1 is not None:
            gp["ms_per_step"] = round(wall1 * 1e3 / args.steps, 5)
            gp["tflops_per_step_wall"] = round(solo.flops * args.steps / wall1 / 1e12, 3)
        out["gemm_phase"] = gp
        wl = solo

    if not args.no_cpu:
        base = wl.cpu_baseline(args.world)
        if base is not None:
            base["value"] = round(base["value"], 4)
            out["cpu_baseline"] = base
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
