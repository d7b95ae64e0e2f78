"""Timing helper with the protocol of the reference's iris.do_bench
(iris/host/platform/utils.py:137-201): one cold call, warm-up, then timed repetitions, each preceded
by the preamble and a 256 MiB cache-clearing write, bracketed by GPU events."""

import statistics

import torch


def _summarize(times, quantiles, return_mode):
    if quantiles is not None:
        ret = torch.quantile(torch.tensor(times, dtype=torch.float), torch.tensor(quantiles, dtype=torch.float)).tolist()
        return ret[0] if len(ret) == 1 else ret
    if return_mode == "all":
        return times
    return {"min": min, "max": max, "mean": statistics.mean, "median": statistics.median}[return_mode](times)


def do_bench(fn, barrier_fn=lambda: None, preamble_fn=lambda: None, n_warmup=25, n_repeat=100, quantiles=None,
             return_mode="mean"):
    """Time `fn` in milliseconds.  `barrier_fn` synchronises (e.g. ctx.barrier), `preamble_fn` runs
    untimed before every call."""
    barrier_fn()
    preamble_fn()
    fn()
    barrier_fn()
    cache = torch.empty(int(256e6 // 4), dtype=torch.int, device="cuda")
    start = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    end = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    for _ in range(n_warmup):
        barrier_fn()
        preamble_fn()
        cache.zero_()
        barrier_fn()
        fn()
    for i in range(n_repeat):
        barrier_fn()
        preamble_fn()
        cache.zero_()
        barrier_fn()
        start[i].record()
        fn()
        end[i].record()
    barrier_fn()
    times = [s.elapsed_time(e) for s, e in zip(start, end)]
    return _summarize(times, quantiles, return_mode)
