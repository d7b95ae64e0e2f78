"""Thin ctypes access to the HIP runtime, in the manner of iris/host/platform/hip.py:13-39,113-126,
248-262 of the reference: only what the single-GPU symmetric heap needs (malloc/free, device
selection, error strings)."""

import ctypes
import logging

from .logging import log_rank

_runtime = None


def runtime():
    """libamdhip64, loaded on first use."""
    global _runtime
    if _runtime is None:
        _runtime = ctypes.cdll.LoadLibrary("libamdhip64.so")
        _runtime.hipGetErrorString.restype = ctypes.c_char_p
        _runtime.hipGetErrorString.argtypes = [ctypes.c_int]
        _runtime.hipMalloc.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t]
        _runtime.hipFree.argtypes = [ctypes.c_void_p]
        _runtime.hipMemset.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t]
    return _runtime


def error_string(err):
    return runtime().hipGetErrorString(ctypes.c_int(err)).decode("utf-8")


def gpu_try(err):
    """Raise RuntimeError for a non-zero hipError_t, worded like the reference's gpu_try."""
    if err != 0:
        text = error_string(err)
        log_rank(logging.ERROR, "HIP error code %d: %s", err, text)
        raise RuntimeError(f"HIP error code {err}: {text}")


def count_devices():
    n = ctypes.c_int(0)
    gpu_try(runtime().hipGetDeviceCount(ctypes.byref(n)))
    return n.value


def set_device(device_id):
    gpu_try(runtime().hipSetDevice(ctypes.c_int(device_id)))


def get_device_id():
    d = ctypes.c_int(0)
    gpu_try(runtime().hipGetDevice(ctypes.byref(d)))
    return d.value


def hip_malloc(size):
    """hipMalloc(size) -> device address as int."""
    ptr = ctypes.c_void_p()
    gpu_try(runtime().hipMalloc(ctypes.byref(ptr), ctypes.c_size_t(size)))
    return int(ptr.value or 0)


def hip_free(ptr):
    gpu_try(runtime().hipFree(ctypes.c_void_p(ptr)))


def hip_memset(ptr, value, size):
    gpu_try(runtime().hipMemset(ctypes.c_void_p(ptr), ctypes.c_int(value), ctypes.c_size_t(size)))
