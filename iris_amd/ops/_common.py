"""Plumbing shared by the operator wrappers: element-type codes, the launch seam, argument checks."""

import logging

import torch

from .. import _lib
from ..host.hip import error_string
from ..host.logging import debug_on, log_rank

_DTYPE_CODES = {
    torch.bfloat16: _lib.BF16,
    torch.float16: _lib.FP16,
    torch.float32: _lib.FP32,
}
_FP8 = getattr(torch, "float8_e4m3fn", None)
if _FP8 is not None:
    _DTYPE_CODES[_FP8] = _lib.FP8_E4M3

_ENTRY_POINTS = {}  # name -> bound foreign function (prototypes applied by _lib.library())

_PATHS = {"auto": _lib.PATH_AUTO, "mfma": _lib.PATH_MFMA, "generic": _lib.PATH_GENERIC}
_ACC = {"fp32": _lib.ACC_FP32, "reference": _lib.ACC_REFERENCE}


def dtype_code(dtype):
    try:
        return _DTYPE_CODES[dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {dtype}") from None


def is_fp8(dtype):
    return _FP8 is not None and dtype == _FP8


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
    """Device address of a tensor as the prototypes' void* takes it: a plain integer, None for no tensor
    (the operators are called once per few microseconds for small shapes; a ctypes object per argument
    was a tenth of the call)."""
    return t.data_ptr() if t is not None else None


def current_stream(shmem):
    """The raw HIP stream torch would launch on for the context's device right now (honours
    `with torch.cuda.stream(...)` and graph capture)."""
    return torch._C._cuda_getCurrentRawStream(shmem.get_device_id())


def iris_launch(entry_name, grid, *args, algorithm, rank, dtype=None):
    """Launch seam: the reference launches `kernel_fn[grid](*args)` here
    (iris/host/tracing/kernel_artifacts.py:54-83); this calls the C entry point of the same operator
    and turns a non-zero hipError_t into RuntimeError the way gpu_try does."""
    if debug_on():
        log_rank(logging.DEBUG, "iris_launch: algorithm=%s kernel=%s grid=%s rank=%d", algorithm, entry_name, grid,
                 rank, rank=rank)
    entry = _ENTRY_POINTS.get(entry_name)
    if entry is None:
        entry = _ENTRY_POINTS[entry_name] = getattr(_lib.library(), entry_name)
    err = entry(*args)
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
