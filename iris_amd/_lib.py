"""Loader for libiris_hip.so, the C-ABI library that holds every kernel of this package.

The prototypes below restate include/iris_hip.h for ctypes.  There is no other compute path: if the
library has not been built, using an operator raises.
"""

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# IRIS_HIP_LIBRARY names another build of the same library (e.g. one compiled with other tile shapes).
LIBRARY_PATH = os.environ.get("IRIS_HIP_LIBRARY") or os.path.join(_HERE, "lib", "libiris_hip.so")

ABI_VERSION = 5

# Enumerations of include/iris_hip.h
BF16, FP16, FP32, FP8_E4M3 = 0, 1, 2, 3
VARIANT_ATOMIC, VARIANT_ONE_SHOT, VARIANT_TWO_SHOT = 0, 2, 3
ACC_FP32, ACC_REFERENCE = 0, 1
GATHER_K, GATHER_M = 1, 2
PATH_AUTO, PATH_MFMA, PATH_GENERIC = 0, 1, 2
STATUS_SPIN_TIMEOUT = 1
DISTRIBUTION_STRIDED, DISTRIBUTION_BLOCK = 0, 1
NOALLOC_MAX_AUX_BYTES, NOALLOC_MAX_FLAGS = 32 * 1024 * 1024, 16384

_i32, _i64, _f32, _ptr = ctypes.c_int32, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p

_GEMM_HEAD = [_ptr, _ptr, _ptr, _ptr, _ptr,  # A, B, C, aux_buffer, locks
              _i64, _i64, _i64,  # M, N, K
              _i64, _i64, _i64, _i64, _i64, _i64,  # strides am ak bk bn cm cn
              _ptr, _i32, _i32,  # context_tensor, cur_rank, world_size
              _i32, _i32, _i32]  # block sizes m n k

_CCL_HEAD = [_ptr, _ptr, _i64, _i64,  # input, output, M, N
             _i64, _i64, _i64, _i64,  # strides in_m in_n out_m out_n
             _ptr, _i32, _i32, _i32, _i32, _i32,  # heap_bases, group_rank, iris_rank, world_size, rank_start, rank_stride
             _i32, _i32, _i32, _i32, _i32, _i32]  # block m, block n, swizzle_size, comm_sms, num_xcds, chunk_size

PROTOTYPES = {
    "iris_hip_matmul_all_reduce": (
        _i32,
        _GEMM_HEAD + [_i32,  # variant
                      _i32, _i32, _f32, _i32,  # in_dtype, out_dtype, scale, acc_mode
                      _i64, _ptr, _i32, _ptr],  # spin_limit, status, path, stream
    ),
    "iris_hip_matmul_all_reduce_noalloc": (
        _i32,
        [_ptr, _ptr, _ptr,  # A, B, C
         _i64, _i64, _i64,  # M, N, K
         _i64, _i64, _i64, _i64, _i64, _i64,  # strides am ak bk bn cm cn
         _i32, _i32, _i32,  # block sizes m n k
         _i32,  # variant
         _i32, _i32, _f32,  # in_dtype, out_dtype, scale
         _i32, _ptr],  # path, stream
    ),
    "iris_hip_matmul_reduce_scatter": (
        _i32,
        _GEMM_HEAD + [_i32, _i32,  # all_owners, sum_peers
                      _i32, _i32, _f32, _i32,
                      _i64, _ptr, _i32, _ptr],
    ),
    "iris_hip_all_gather_matmul": (
        _i32,
        [_ptr, _ptr, _ptr, _ptr,  # A_sharded, B, C, bias
         _i64, _i64, _i64, _i64,  # M, N, K, K_local
         _i64, _i64, _i64, _i64, _i64, _i64, _i64,  # strides am ak bk bn cm cn bias
         _ptr, _i32, _i32,  # context_tensor, cur_rank, world_size
         _i32, _i32, _i32,  # block sizes
         _i32,  # gather_dim
         _i32, _i32, _i32, _f32,  # in_dtype, out_dtype, bias_dtype, scale
         _i32, _ptr],  # path, stream
    ),
    "iris_hip_matmul_all_gather": (
        _i32,
        [_ptr, _ptr, _ptr, _ptr,  # A, B, C_gathered, bias
         _i64, _i64, _i64, _i64,  # M_local, M, N, K
         _i64, _i64, _i64, _i64, _i64, _i64, _i64,  # strides am ak bk bn cm cn bias
         _ptr, _i32, _i32,  # context_tensor, cur_rank, world_size
         _i32, _i32, _i32,  # block sizes
         _i32, _i32, _i32, _f32,  # in_dtype, out_dtype, bias_dtype, scale
         _i32, _ptr],  # path, stream
    ),
    "iris_hip_all_reduce": (_i32, _CCL_HEAD + [_i32, _i32, _i32, _ptr]),  # variant, distribution, dtype, stream
    "iris_hip_reduce_scatter": (_i32, _CCL_HEAD + [_i32, _i32, _ptr]),  # distribution, dtype, stream
    "iris_hip_register_context": (_i32, [_ptr, _ptr, _i32]),
    "iris_hip_unregister_context": (_i32, [_ptr]),
    "iris_hip_query": (_i32, [_i32, _ptr, _ptr, _ptr]),
    "iris_hip_set_split_tiles": (None, [_i32]),
    "iris_hip_last_error": (ctypes.c_char_p, []),
    "iris_hip_last_kernel": (ctypes.c_char_p, []),
    "iris_hip_abi_version": (_i32, []),
}

_lib = None


def library():
    """The loaded library (ctypes.CDLL) with prototypes applied.  Raises if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIBRARY_PATH):
            raise RuntimeError(
                f"{LIBRARY_PATH} is missing: build it with `python -m iris_amd.csrc.build` "
                "(hipcc, --offload-arch=gfx950). There is no fallback compute path."
            )
        lib = ctypes.CDLL(LIBRARY_PATH)
        for name, (restype, argtypes) in PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        if lib.iris_hip_abi_version() != ABI_VERSION:
            raise RuntimeError(
                f"{LIBRARY_PATH} has ABI version {lib.iris_hip_abi_version()}, expected {ABI_VERSION}: rebuild it"
            )
        _lib = lib
    return _lib


def last_error():
    return library().iris_hip_last_error().decode("utf-8")


def last_kernel():
    return library().iris_hip_last_kernel().decode("utf-8")


def query(device):
    """(cu_count, xcc_count, lds_bytes_per_block) of GPU `device`."""
    cu, xcc, lds = _i32(), _i32(), _i32()
    err = library().iris_hip_query(device, ctypes.byref(cu), ctypes.byref(xcc), ctypes.byref(lds))
    if err:
        raise RuntimeError(f"HIP error code {err}: {last_error()}")
    return cu.value, xcc.value, lds.value
