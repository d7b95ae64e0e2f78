"""Where the time of one fused launch goes: phase boundaries stamped inside the kernel.

    python -m iris_amd.csrc.build --stamps          # builds lib/libiris_hip_stamps.so
    python -m iris_amd.bench.phase_stamps [--workload NAME] [--world W] [--flush zero|read|none] [--reps N]

The diagnostic build of the library records the device's constant-rate counter (s_memrealtime) in
thread 0 of every workgroup at the phase boundaries of its first eight tiles.  This tool runs a workload of
bench.py against that build and prints, per phase, the mean and the maximum over the workgroups, and
the span from the first workgroup's entry to the last workgroup's last store.  Figures include the cost
of the stamps themselves (one store per phase and workgroup).
"""

import argparse
import ctypes
import os
import statistics
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
STAMPS_LIB = os.path.join(os.path.dirname(HERE), "lib", "libiris_hip_stamps.so")

PHASES = ["entry -> first operands in LDS", "K loop", "tile staged in LDS", "phase-1 stores issued",
          "phase-1 stores acknowledged", "flags raised, peers' flags seen", "phase-2 (slot sum) stores issued",
          "last store acknowledged"]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default=None)
    ap.add_argument("--world", type=int, default=8)
    ap.add_argument("--flush", default="zero", choices=["zero", "read", "none"],
                    help="before every launch: zero a 256 MB buffer (the reference's do_bench), read it, or nothing")
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--dump", default=None, metavar="FILE.npy",
                    help="save the last launch's stamps (microseconds, one row of 9 per tile) for other tools")
    ap.add_argument("--items", type=int, default=0, metavar="GRID",
                    help="also print, for the last launch of GRID workgroups, the mean stamps of every workgroup's first, "
                         "second, ... tile separately (split launches: helpers' pieces end at stamp 3, 'partial sum out')")
    ap.add_argument("--split", type=int, default=None, metavar="MODE", help="iris_hip_set_split_tiles(MODE) before the launches")
    ap.add_argument("--deciles", action="store_true",
                    help="also print, for the last launch, the deciles over the stamped tiles of every phase")
    args = ap.parse_args()
    if not os.path.exists(STAMPS_LIB):
        sys.exit(f"{STAMPS_LIB} is missing: build it with `python -m iris_amd.csrc.build --stamps`")
    sys.path.insert(0, ROOT)
    import torch

    import bench
    import iris_amd as iris
    from iris_amd import _lib
    from iris_amd.host import hip

    if _lib._lib is not None:
        sys.exit("the kernel library was loaded before the diagnostic build could be selected")
    _lib.LIBRARY_PATH = STAMPS_LIB  # the library is loaded on first use
    lib = _lib.library()
    lib.iris_hip_debug_set_stamps.argtypes = [ctypes.c_void_p, ctypes.c_longlong]
    lib.iris_hip_debug_set_stamps.restype = None
    rate_khz = ctypes.c_int(0)
    hip.gpu_try(hip.runtime().hipDeviceGetAttribute(ctypes.byref(rate_khz), 10017, 0))  # hipDeviceAttributeWallClockRate
    us_per_tick = 1e3 / rate_khz.value

    if args.split is not None:
        lib.iris_hip_set_split_tiles(args.split)
    wl = bench.WORKLOADS[args.workload or bench.DEFAULT]()
    wl.setup(iris, args.world)
    max_wgs = 65536  # rows of the stamp buffer: tiles stamped per launch (eight per workgroup at most)
    stamps = torch.zeros((max_wgs, 16), dtype=torch.int64, device="cuda")
    cache = torch.empty(int(256e6) // 4, dtype=torch.int, device="cuda")
    per_phase = [[] for _ in PHASES]
    per_phase_max = [[] for _ in PHASES]
    spans, entry_spread = [], []
    for rep in range(-5, args.reps):
        torch.cuda.synchronize()
        if args.flush == "zero":
            cache.zero_()
        elif args.flush == "read":
            cache.sum()
        stamps.zero_()
        torch.cuda.synchronize()
        lib.iris_hip_debug_set_stamps(ctypes.c_void_p(stamps.data_ptr()), stamps.shape[0])
        wl.step()
        torch.cuda.synchronize()
        lib.iris_hip_debug_set_stamps(ctypes.c_void_p(0), 0)
        if rep < 0:
            continue
        t = stamps.cpu()
        raw = t.double() * us_per_tick
        t = t[t[:, 0] != 0].double() * us_per_tick
        last = 8
        while last > 0 and float(t[:, last].max()) == 0.0:  # phases this launch does not have
            last -= 1
        t0 = float(t[:, 0].min())
        entry_spread.append(float((t[:, 0] - t0).mean()))
        prev = t[:, 0]
        for i in range(len(PHASES)):
            cur = t[:, i + 1]
            if float(cur.max()) == 0.0:
                per_phase[i].append(0.0)
                per_phase_max[i].append(0.0)
                continue
            both = (cur != 0) & (prev != 0)  # helpers' pieces of a split launch stop at stamp 3
            d = (cur - prev)[both]
            per_phase[i].append(float(d.mean()) if d.numel() else 0.0)
            per_phase_max[i].append(float(d.max()) if d.numel() else 0.0)
            prev = torch.where(cur != 0, cur, prev)
        spans.append(float(t[:, last].max()) - t0)
    print(f"workload {wl.name}  W={args.world}  kernel {_lib.last_kernel()}  tiles stamped {t.shape[0]}  flush={args.flush}  "
          f"{args.reps} launches; microseconds, mean over launches of (mean | max over tiles)")
    print(f"  {'workgroup entry after the first one':40s} {statistics.mean(entry_spread):8.2f}")
    for name, mean, mx in zip(PHASES, per_phase, per_phase_max):
        print(f"  {name:40s} {statistics.mean(mean):8.2f} | {statistics.mean(mx):8.2f}")
    print(f"  {'first entry -> last stamp':40s} {statistics.mean(spans):8.2f}")
    if args.items:
        grid = args.items
        print(f"  last launch, per workgroup item (rows item * {grid} + workgroup), mean stamp in us after the first entry:")
        print("    item   rows  " + " ".join(f"{i:>7d}" for i in range(9)))
        for item in range(8):
            rows = raw[item * grid:(item + 1) * grid]
            if not bool((rows[:, 0] != 0).any()):
                continue
            for name, part in (("workgroups of the first half of the grid", rows[: grid // 2]), ("second half", rows[grid // 2:])):
                part = part[part[:, 0] != 0]
                if part.shape[0] == 0:
                    continue
                cols = [f"{float((part[:, i][part[:, i] != 0] - t0).mean()):7.1f}" if bool((part[:, i] != 0).any()) else "      -" for i in range(9)]
                print(f"    {item:4d} {part.shape[0]:6d}  " + " ".join(cols) + f"   ({name})")
    if args.dump:
        import numpy
        os.makedirs(os.path.dirname(os.path.abspath(args.dump)), exist_ok=True)
        numpy.save(args.dump, (t - t0).numpy())
    if args.deciles:
        print("last launch, deciles over tiles (min, 10 %, ..., 90 %, max):")
        prev = t[:, 0]
        q = torch.linspace(0, 1, 11, dtype=torch.float64)
        for i, name in enumerate(PHASES):
            cur = t[:, i + 1]
            if float(cur.max()) != 0.0:
                print(f"  {name:40s} " + " ".join(f"{v:6.2f}" for v in torch.quantile(cur - prev, q).tolist()))
                prev = cur



if __name__ == "__main__":
    main()
