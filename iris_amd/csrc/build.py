"""Build libiris_hip.so for gfx950 with hipcc.

    python -m iris_amd.csrc.build [--force]

The library lands in iris_amd/lib/ next to the package so that it travels with the source tree.
"""

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
SOURCES = [os.path.join(HERE, "iris_hip.hip"), os.path.join(HERE, "iris_ccl.hip")]
HEADERS = [os.path.join(HERE, h) for h in ("layout.h", "device_util.h", "host_common.h")] + [
    os.path.join(ROOT, "include", "iris_hip.h")]
OUTPUT = os.path.join(os.path.dirname(HERE), "lib", "libiris_hip.so")

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
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


def build(force=True, verbose=True):
    """Compile the library.  With force=False an up-to-date library is left alone."""
    if not force and up_to_date():
        return OUTPUT
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    os.makedirs(os.path.dirname(OUTPUT), exist_ok=True)
    tmp = OUTPUT + ".tmp"
    cmd = [hipcc] + FLAGS + ["-o", tmp] + SOURCES
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass does not know the packed-fp32 feature and says so; that line is noise.
    noise = "is not a recognized feature for this target"
    out = "\n".join(l for l in proc.stdout.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{out}")
    if verbose and out.strip():
        print(out)
    os.replace(tmp, OUTPUT)
    return OUTPUT


if __name__ == "__main__":
    build(force="--force" in sys.argv or True)
    print(OUTPUT)
