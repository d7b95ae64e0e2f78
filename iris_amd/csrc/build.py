"""Build libiris_hip.so for gfx950 with hipcc.

    python -m iris_amd.csrc.build [--force]

The library lands in iris_amd/lib/ next to the package so that it travels with the source tree.
"""

import concurrent.futures
import os
import shutil
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
# One translation unit per input type of the MFMA kernel (they hold most of the compile time and are
# compiled side by side), the entry points with the generic kernel, and the stand-alone collectives.
SOURCES = [os.path.join(HERE, f) for f in (
    "iris_hip.hip", "iris_hip_mfma_bf16.hip", "iris_hip_mfma_f16.hip", "iris_hip_mfma_fp8.hip", "iris_ccl.hip")]
HEADERS = [os.path.join(HERE, h) for h in ("fused_kernel.h", "decode_kernel.h", "layout.h", "device_util.h", "host_common.h")] + [
    os.path.join(ROOT, "include", "iris_hip.h")]
OUTPUT = os.path.join(os.path.dirname(HERE), "lib", "libiris_hip.so")

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # Keep hipcc from forming packed fp32 instructions out of scalar float code.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unknown-warning-option",
    "-I" + os.path.join(ROOT, "include"),
    "-I" + HERE,
]


def up_to_date():
    if not os.path.exists(OUTPUT):
        return False
    built = os.path.getmtime(OUTPUT)
    return all(os.path.getmtime(f) <= built for f in SOURCES + HEADERS + [os.path.abspath(__file__)])


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass does not know the packed-fp32 feature and says so; that line is noise.
    noise = "is not a recognized feature for this target"
    out = "\n".join(l for l in proc.stdout.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}): {' '.join(cmd)}\n{out}")
    if verbose and out.strip():
        print(out)


STAMPS_OUTPUT = os.path.join(os.path.dirname(HERE), "lib", "libiris_hip_stamps.so")


def build(force=True, verbose=True, stamps=False):
    """Compile the library.  With force=False an up-to-date library is left alone.  stamps=True builds
    the diagnostic variant (kernels record time stamps at their phase boundaries; see
    iris_amd/bench/phase_stamps.py) as libiris_hip_stamps.so next to the regular library."""
    if stamps:
        return _build(STAMPS_OUTPUT, FLAGS + ["-DIRIS_HIP_PHASE_STAMPS"], verbose)
    if not force and up_to_date():
        return OUTPUT
    return _build(OUTPUT, FLAGS, verbose)


def _build(output, flags, verbose):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    os.makedirs(os.path.dirname(output), exist_ok=True)
    with tempfile.TemporaryDirectory(prefix="iris_hip_build_") as tmpdir:
        objects = [os.path.join(tmpdir, os.path.splitext(os.path.basename(src))[0] + ".o") for src in SOURCES]
        with concurrent.futures.ThreadPoolExecutor(max_workers=min(len(SOURCES), os.cpu_count() or 1)) as pool:
            jobs = [pool.submit(_run, [hipcc] + flags + ["-c", "-o", obj, src], verbose)
                    for src, obj in zip(SOURCES, objects)]
            for job in jobs:
                job.result()
        tmp = output + ".tmp"
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-o", tmp] + objects, verbose)
        os.replace(tmp, output)
    return output


if __name__ == "__main__":
    print(build(force=True, stamps="--stamps" in sys.argv))
