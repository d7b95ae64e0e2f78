"""Plumbing shared by the operator wrappers: element-type codes, the launch seam, argument checks."""

import ctypes
import logging

import torch

from .. import _lib
from ..host.hip import error_string
from ..host.logging import log_rank

_DTYPE_CODES = {
    torch.bfloat16: _lib.BF16,
    torch.float16: _lib.FP16,
    torch.float32: _lib.FP32,
}
if hasattr(torch, "float8_e4m3fn"):
    _DTYPE_CODES[torch.float8_e4m3fn] = _lib.FP8_E4M3

_PATHS = {"auto": _lib.PATH_AUTO, "mfma": _lib.PATH_MFMA, "generic": _lib.PATH_GENERIC}
_ACC = {"fp32": _lib.ACC_FP32, "reference": _lib.ACC_REFERENCE}


def dtype_code(dtype):
    try:
        return _DTYPE_CODES[dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {dtype}") from None


def is_fp8(dtype):
    return hasattr(torch, "float8_e4m3fn") and dtype == torch.float8_e4m3fn


def path_code(path):
    try:
        return _PATHS[path]
    except KeyError:
        raise ValueError(f"kernel path must be one of {sorted(_PATHS)}, got {path!r}") from None


def acc_code(acc):
    try:
        return _ACC[acc]
    except KeyError:
        raise ValueError(f"slot_sum must be one of {sorted(_ACC)}, got {acc!r}") from None


def require_gpu_tensors(shmem, **tensors):
    """The kernels only run on the GPU that holds the heap."""
    dev = shmem.get_device()
    if dev.type != "cuda":
        raise RuntimeError("fused operators need a GPU context; this Iris context is host-backed")
    for name, t in tensors.items():
        if t is not None and t.device != dev:
            raise RuntimeError(f"{name} is on {t.device}, but the Iris context is on {dev}")


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def current_stream(shmem):
    """The raw HIP stream torch would launch on for the context's device right now (honours
    `with torch.cuda.stream(...)` and graph capture)."""
    return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(shmem.get_device_id()))


def iris_launch(entry_name, grid, *args, algorithm, rank, dtype=None):
    """Launch seam: the reference launches `kernel_fn[grid](*args)` here
    (iris/host/tracing/kernel_artifacts.py:54-83); this calls the C entry point of the same operator
    and turns a non-zero hipError_t into RuntimeError the way gpu_try does."""
    log_rank(logging.DEBUG, "iris_launch: algorithm=%s kernel=%s grid=%s rank=%d", algorithm, entry_name, grid,
             rank, rank=rank)
    lib = _lib.library()
    err = getattr(lib, entry_name)(*args)
    if err != 0:
        detail = _lib.last_error()
        text = detail if detail else error_string(err)
        log_rank(logging.ERROR, "HIP error code %d: %s", err, text, rank=rank)
        raise RuntimeError(f"HIP error code {err}: {text}")
    return None


def stage_idle_peers(shmem, workspace):
    """One GPU standing in for all ranks: make the other ranks look finished with nothing to add.

    Called by the preambles when the context has `stand_in_peers` set (the benchmark harness sets it):
    the peers' flags are raised and their aux buffers zeroed, so that a fused launch neither waits for
    ranks that do not run nor sums uninitialised memory.  The reference has no counterpart - its peers
    are live processes.
    """
    if not getattr(shmem, "stand_in_peers", False):
        return
    for r in range(shmem.get_num_ranks()):
        if r == shmem.get_rank():
            continue
        if workspace.locks is not None:
            shmem.peer_view(workspace.locks, r).fill_(1)
        if workspace.aux_buffer is not None:
            shmem.peer_view(workspace.aux_buffer, r).zero_()
