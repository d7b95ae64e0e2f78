"""Registry, per-combination state, sweep execution and output formats of the benchmark harness.

Behaviour follows iris/bench/_core.py (State, axis, register, range helpers) and
iris/bench/_runner.py (axis overrides :61-146, formatters :170-312, timing through do_bench :357-385,
command line :399-520) of the reference.
"""

import argparse
import csv
import io
import gc
import itertools
import json
import re
import statistics
import sys
from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional

import torch

RANKS_AXIS = "num_ranks"  # the axis that sizes the world instead of being swept inside it
DEFAULT_NUM_RANKS = 8

_DTYPE_WORDS = {"fp16": torch.float16, "float16": torch.float16, "fp32": torch.float32, "float32": torch.float32,
                "bf16": torch.bfloat16, "bfloat16": torch.bfloat16}


@dataclass
class AxisDef:
    name: str
    values: List[Any]


@dataclass
class BenchmarkDef:
    name: str
    fn: Callable
    axes: List[AxisDef]


@dataclass
class Result:
    """One row: a benchmark at one parameter combination."""

    benchmark_name: str
    params: Dict[str, Any]
    gpu_time_ms: float
    all_times_ms: List[float]
    bandwidth_gbps: Optional[float] = None
    tflops: Optional[float] = None
    counters: Dict[str, float] = field(default_factory=dict)
    skipped: bool = False
    skip_reason: str = ""
    world_size: int = 1


_registry: List[BenchmarkDef] = []


class _Skip(Exception):
    def __init__(self, reason=""):
        super().__init__(reason)
        self.reason = reason


class State:
    """Handed to the benchmark function as its first argument: axis values in, metrics and the
    callable to time out."""

    def __init__(self, params, n_warmup, n_repeat):
        self._params = params
        self._bytes = None
        self._flops = None
        self._counters = {}
        self._exec_fn = None
        self._preamble_fn = lambda: None
        self._n_warmup = n_warmup
        self._n_repeat = n_repeat

    def __getitem__(self, key):
        return self._params[key]

    def get(self, key, default=None):
        return self._params.get(key, default)

    def set_bytes(self, n):
        """Bytes moved per call: adds the BW (GB/s) column."""
        self._bytes = n

    def set_flops(self, n):
        """Flop per call: adds the TFLOPS column."""
        self._flops = n

    def add_counter(self, name, value):
        self._counters[name] = value

    def set_warmup(self, n):
        self._n_warmup = n

    def set_repeat(self, n):
        self._n_repeat = n

    def exec(self, fn, *, preamble_fn=None):
        """Register (not run) the callable to time; preamble_fn runs untimed before every call."""
        self._exec_fn = fn
        if preamble_fn is not None:
            self._preamble_fn = preamble_fn

    def skip(self, reason=""):
        raise _Skip(reason)


def power_of_two(start_exp, end_exp):
    """[2**start_exp, ..., 2**end_exp], both ends included."""
    return [1 << e for e in range(start_exp, end_exp + 1)]


def linear_range(start, end, step):
    """[start, start+step, ..., end], end included."""
    return list(range(start, end + 1, step))


def axis(name, values):
    """Decorator: add a sweep axis.  The outermost axis varies slowest."""

    def wrap(fn):
        axes = fn.__dict__.setdefault("_bench_axes", [])
        axes.insert(0, AxisDef(name, list(values)))
        return fn

    return wrap


def register(fn):
    """Decorator (outermost): make fn(state, ctx) a benchmark."""
    _registry.append(BenchmarkDef(fn.__name__, fn, getattr(fn, "_bench_axes", [])))
    return fn


# -- command-line axis values ------------------------------------------------------------------
def show(value):
    """Axis values as they appear in tables: torch dtypes by their short name."""
    return str(value).replace("torch.", "") if isinstance(value, torch.dtype) else str(value)


def parse_axis_values(raw, axis_name):
    """`1024,2048` | `pow2:8:13` | `lin:64:256:64` | dtype names (fp16, bf16, float32, ...)."""
    raw = raw.strip()
    for prefix, count, build, shape in (("pow2:", 2, power_of_two, "pow2:start:stop"),
                                        ("lin:", 3, linear_range, "lin:start:stop:step")):
        if raw.startswith(prefix):
            parts = raw.split(":")[1:]
            if len(parts) != count:
                kind = "pow2" if prefix == "pow2:" else "linear"
                raise ValueError(f"Invalid {kind} specification {raw!r} for axis {axis_name!r}; expected format '{shape}'.")
            try:
                return build(*[int(x) for x in parts])
            except ValueError:
                ints = ":".join(["<int>"] * count)
                raise ValueError(
                    f"Non-integer values in {raw!r} for axis {axis_name!r}; expected format '{prefix}{ints}'.") from None
    words = [w.strip() for w in raw.split(",")]
    if axis_name == "dtype":
        unknown = [w for w in words if w.lower() not in _DTYPE_WORDS]
        if unknown:
            raise ValueError(f"Unknown dtype(s) for axis {axis_name!r}: {', '.join(unknown)}. "
                             f"Allowed: {', '.join(sorted(_DTYPE_WORDS))}")
    if all(w.lower() in _DTYPE_WORDS for w in words):
        return [_DTYPE_WORDS[w.lower()] for w in words]
    for convert in (int, float):
        try:
            return [convert(w) for w in words]
        except ValueError:
            continue
    return words


def _values(ax, overrides, skips):
    values = list(overrides.get(ax.name, ax.values))
    return [v for v in values if v not in set(skips.get(ax.name, []))]


def _world_sizes(bdef, overrides, skips):
    for ax in bdef.axes:
        if ax.name == RANKS_AXIS:
            return _values(ax, overrides, skips)
    if RANKS_AXIS in overrides:
        return _values(AxisDef(RANKS_AXIS, overrides[RANKS_AXIS]), {}, skips)
    return [DEFAULT_NUM_RANKS]


# -- output ----------------------------------------------------------------------------------------
def _counter_names(results):
    names = []
    for r in results:
        names += [c for c in r.counters if c not in names]
    return names


def format_console(results):
    """One right-aligned table per benchmark: parameters, GPU Time (ms), BW (GB/s), TFLOPS, counters."""
    blocks = []
    for name in dict.fromkeys(r.benchmark_name for r in results):
        rows = [r for r in results if r.benchmark_name == name]
        params = list(rows[0].params)
        columns = [(p, lambda r, p=p: show(r.params[p])) for p in params]
        columns.append(("GPU Time (ms)", lambda r: f"{r.gpu_time_ms:.3f}"))
        if any(r.bandwidth_gbps is not None for r in rows):
            columns.append(("BW (GB/s)", lambda r: "" if r.bandwidth_gbps is None else f"{r.bandwidth_gbps:.1f}"))
        if any(r.tflops is not None for r in rows):
            columns.append(("TFLOPS", lambda r: "" if r.tflops is None else f"{r.tflops:.1f}"))
        for c in _counter_names(rows):
            columns.append((c, lambda r, c=c: f"{r.counters[c]:.3f}" if c in r.counters else ""))
        table = [[title for title, _ in columns]]
        for r in rows:
            if r.skipped:
                note = "(skipped)" + (f" {r.skip_reason}" if r.skip_reason else "")
                cells = ([columns[0][1](r), note] if params else [note])
            else:
                cells = [cell(r) for _, cell in columns]
            table.append(cells + [""] * (len(columns) - len(cells)))
        widths = [max(len(row[i]) for row in table) for i in range(len(columns))]
        lines = ["  ".join(cell.rjust(w) for cell, w in zip(row, widths)) for row in table]
        blocks.append("\n" + name + "\n" + "\n".join(lines))
    return "\n".join(blocks) + "\n" if blocks else ""


def format_json(results):
    records = []
    for r in results:
        rec = {"benchmark": r.benchmark_name, "world_size": r.world_size,
               "params": {k: show(v) for k, v in r.params.items()},
               "gpu_time_ms": r.gpu_time_ms, "all_times_ms": r.all_times_ms}
        if r.bandwidth_gbps is not None:
            rec["bandwidth_gbps"] = r.bandwidth_gbps
        if r.tflops is not None:
            rec["tflops"] = r.tflops
        if r.counters:
            rec["counters"] = r.counters
        if r.skipped:
            rec["skipped"], rec["skip_reason"] = True, r.skip_reason
        records.append(rec)
    return json.dumps(records, indent=2) + "\n"


def format_csv(results):
    if not results:
        return ""
    params = []
    for r in results:
        params += [k for k in r.params if k not in params]
    counters = _counter_names(results)
    out = io.StringIO()
    writer = csv.DictWriter(out, fieldnames=["benchmark", "world_size"] + params
                            + ["gpu_time_ms", "bandwidth_gbps", "tflops"] + counters + ["skipped", "skip_reason"])
    writer.writeheader()
    for r in results:
        row = {"benchmark": r.benchmark_name, "world_size": r.world_size,
               "gpu_time_ms": "" if r.skipped else f"{r.gpu_time_ms:.4f}",
               "bandwidth_gbps": "" if r.bandwidth_gbps is None else f"{r.bandwidth_gbps:.2f}",
               "tflops": "" if r.tflops is None else f"{r.tflops:.2f}",
               "skipped": r.skipped, "skip_reason": r.skip_reason}
        row.update({p: show(r.params.get(p, "")) for p in params})
        row.update({c: f"{r.counters[c]:.4f}" if c in r.counters else "" for c in counters})
        writer.writerow(row)
    return out.getvalue()


# -- execution -------------------------------------------------------------------------------------
def _run_world(benchmarks, world_size, rank, overrides, skips, heap_size, n_warmup, n_repeat, name_filter,
               make_context, time_fn):
    """Every benchmark that runs at this world size, each on a context with `world_size` heap slots."""
    results = []
    for bdef in benchmarks:
        if name_filter and not re.search(name_filter, bdef.name):
            continue
        declares_ranks = any(ax.name == RANKS_AXIS for ax in bdef.axes)
        if world_size not in _world_sizes(bdef, overrides, skips):
            continue
        axes = [AxisDef(ax.name, _values(ax, overrides, skips)) for ax in bdef.axes if ax.name != RANKS_AXIS]
        if any(not ax.values for ax in axes):
            continue  # an axis emptied by --skip_* drops the whole benchmark
        # A fresh heap per benchmark: the bump allocator never frees, and a sweep allocates per combination.
        ctx = make_context(heap_size, world_size, rank)
        results += _run_benchmark(bdef, axes, ctx, world_size, declares_ranks or RANKS_AXIS in overrides,
                                  n_warmup, n_repeat, time_fn)
        ctx.barrier()
        # The heap lives as long as its last tensor: everything the benchmark allocated (tensors held by
        # the callables it registered included) went out of scope with _run_benchmark; collect what sits
        # in reference cycles before the next benchmark asks for a heap of its own.
        del ctx
        gc.collect()
    return results


def _run_benchmark(bdef, axes, ctx, world_size, show_ranks, n_warmup, n_repeat, time_fn):
    """All parameter combinations of one benchmark on one context."""
    results = []
    for combo in itertools.product(*[ax.values for ax in axes]):
        params = {RANKS_AXIS: world_size} if show_ranks else {}
        params.update(zip([ax.name for ax in axes], combo))
        state = State(params, n_warmup, n_repeat)
        try:
            bdef.fn(state, ctx)
        except _Skip as skip:
            results.append(Result(bdef.name, params, 0.0, [], skipped=True, skip_reason=skip.reason,
                                  world_size=world_size))
            continue
        if state._exec_fn is None:
            raise RuntimeError(f"Benchmark '{bdef.name}' with params {params} did not call state.exec(fn). "
                               f"Every benchmark must register a callable to time.")
        times = time_fn(state._exec_fn, barrier_fn=ctx.barrier, preamble_fn=state._preamble_fn,
                        n_warmup=state._n_warmup, n_repeat=state._n_repeat, return_mode="all")
        mean_ms = statistics.mean(times)
        per_second = (lambda n: n / (mean_ms * 1e-3)) if mean_ms > 0 else (lambda n: None)
        results.append(Result(
            bdef.name, params, mean_ms, times,
            bandwidth_gbps=None if state._bytes is None else per_second(state._bytes / 1e9),
            tflops=None if state._flops is None else per_second(state._flops / 1e12),
            counters=dict(state._counters), world_size=world_size))
    return results


def _gpu_context(heap_size, world_size, rank):
    from ..host.iris import iris as make_iris

    ctx = make_iris(heap_size, num_ranks=world_size, rank=rank)
    ctx.stand_in_peers = True
    return ctx


def run_registered(benchmarks=None, *, axis_overrides=None, skip_overrides=None, heap_size=1 << 34, rank=0,
                   n_warmup=25, n_repeat=100, benchmark_filter=None, make_context=None, time_fn=None):
    """Run the sweep and return the list of Result rows (what main() formats).  make_context and
    time_fn are injection points for tests: they default to a GPU Iris context and iris_amd.do_bench."""
    benchmarks = list(_registry) if benchmarks is None else list(benchmarks)
    overrides, skips = axis_overrides or {}, skip_overrides or {}
    if time_fn is None:
        from ..host.bench import do_bench as time_fn
    make_context = make_context or _gpu_context
    worlds = set()
    for bdef in benchmarks:
        if benchmark_filter and not re.search(benchmark_filter, bdef.name):
            continue
        worlds.update(_world_sizes(bdef, overrides, skips))
    results = []
    for world_size in sorted(worlds):
        if rank >= world_size:
            continue
        results += _run_world(benchmarks, world_size, rank, overrides, skips, heap_size, n_warmup, n_repeat,
                              benchmark_filter, make_context, time_fn)
    return results


def build_parser():
    parser = argparse.ArgumentParser(description="iris_amd.bench - GPU benchmarking harness",
                                     formatter_class=argparse.ArgumentDefaultsHelpFormatter)
    parser.add_argument("--benchmark_filter", type=str, default=None, help="Regex filter for benchmark names")
    parser.add_argument("--benchmark_format", type=str, default="console", choices=["console", "json", "csv"],
                        help="Output format")
    parser.add_argument("--benchmark_out", type=str, default=None, help="Write results to this file")
    parser.add_argument("--heap_size", type=int, default=1 << 34,
                        help="Symmetric heap size in bytes per rank slot (num_ranks slots share one GPU)")
    parser.add_argument("--use_gluon", action="store_true", help="Rejected: there is no Gluon backend here")
    parser.add_argument("--n_warmup", type=int, default=25, help="Number of warmup iterations")
    parser.add_argument("--n_repeat", type=int, default=100, help="Number of timed iterations")
    parser.add_argument("--rank", type=int, default=0, help="The rank whose launch is timed")
    return parser


def main(argv=None):
    """Command-line entry: `if __name__ == "__main__": bench.main()`.

    Besides the flags of --help: `--axis_<name>=<values>` replaces an axis, `--skip_<name>=<values>`
    removes values from it.
    """
    parser = build_parser()
    args, rest = parser.parse_known_args(argv)
    if args.use_gluon:
        parser.error("--use_gluon: this package has HIP kernels only")
    overrides, skips = {}, {}
    for token in rest:
        m = re.match(r"^--(axis|skip)_(\w+)=(.+)$", token)
        if not m:
            parser.error(f"Unrecognized argument: {token}")
        (overrides if m.group(1) == "axis" else skips)[m.group(2)] = parse_axis_values(m.group(3), m.group(2))
    if not _registry:
        print("No benchmarks registered.", file=sys.stderr)
        sys.exit(1)
    selected = [b for b in _registry if not args.benchmark_filter or re.search(args.benchmark_filter, b.name)]
    if not any(_world_sizes(b, overrides, skips) for b in selected):
        print("No benchmark configurations to run after applying filters/skips.", file=sys.stderr)
        sys.exit(1)
    results = run_registered(axis_overrides=overrides, skip_overrides=skips, heap_size=args.heap_size, rank=args.rank,
                             n_warmup=args.n_warmup, n_repeat=args.n_repeat, benchmark_filter=args.benchmark_filter)
    text = {"json": format_json, "csv": format_csv}.get(args.benchmark_format, format_console)(results)
    print(text, end="")
    if args.benchmark_out:
        with open(args.benchmark_out, "w") as f:
            f.write(text)
