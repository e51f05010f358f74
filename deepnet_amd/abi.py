"""ctypes mirror of include/tensor_hip.h: the blittable descriptor, the enums and the dtype tables.

Pure declarations, loads no library.  The F# binding a Deep.Net maintainer would write declares the same
struct with [<StructLayout(LayoutKind.Sequential)>] (reference precedent for by-value marshalling:
Tensor/Tensor/Cuda/NativeTensor.fs:96-112).
"""
import ctypes as C

import numpy as np

DNH_MAX_DIMS = 8

# DnhStatus
DNH_OK = 0
DNH_ERR_INVALID_ARG = 1
DNH_ERR_NOT_SUPPORTED = 2
DNH_ERR_OUT_OF_MEMORY = 3
DNH_ERR_HIP = 4
DNH_ERR_INDEX_OUT_OF_RANGE = 5
DNH_ERR_NOT_INITIALIZED = 6
DNH_ERR_SINGULAR_MATRIX = 7
DNH_ERR_NO_CONVERGENCE = 8

# DnhDType
DNH_BOOL, DNH_U8, DNH_I8, DNH_I32, DNH_U32, DNH_I64, DNH_U64, DNH_F32, DNH_F64, DNH_I16, DNH_U16 = range(11)

DTYPE_TO_NUMPY = {
    DNH_BOOL: np.dtype(np.bool_),
    DNH_U8: np.dtype(np.uint8),
    DNH_I8: np.dtype(np.int8),
    DNH_I32: np.dtype(np.int32),
    DNH_U32: np.dtype(np.uint32),
    DNH_I64: np.dtype(np.int64),
    DNH_U64: np.dtype(np.uint64),
    DNH_F32: np.dtype(np.float32),
    DNH_F64: np.dtype(np.float64),
    DNH_I16: np.dtype(np.int16),
    DNH_U16: np.dtype(np.uint16),
}
NUMPY_TO_DTYPE = {v: k for k, v in DTYPE_TO_NUMPY.items()}


def dtype_code(dt) -> int:
    dt = np.dtype(dt)
    if dt not in NUMPY_TO_DTYPE:
        raise NotImplementedError(f"element type {dt} has no tensor_hip dtype")
    return NUMPY_TO_DTYPE[dt]


# DnhUnaryOp
(DNH_UNARY_PLUS, DNH_UNARY_MINUS, DNH_ABS, DNH_SGN, DNH_LOG, DNH_LOG10, DNH_EXP, DNH_SIN, DNH_COS, DNH_TAN,
 DNH_ASIN, DNH_ACOS, DNH_ATAN, DNH_SINH, DNH_COSH, DNH_TANH, DNH_SQRT, DNH_CEILING, DNH_FLOOR, DNH_ROUND,
 DNH_TRUNCATE, DNH_NEGATE) = range(22)
# DnhBinaryOp
(DNH_ADD, DNH_SUBTRACT, DNH_MULTIPLY, DNH_DIVIDE, DNH_MODULO, DNH_POWER, DNH_MAX_ELEMWISE, DNH_MIN_ELEMWISE,
 DNH_AND, DNH_OR, DNH_XOR) = range(11)
# DnhCompareOp
DNH_EQUAL, DNH_NOT_EQUAL, DNH_LESS, DNH_LESS_OR_EQUAL, DNH_GREATER, DNH_GREATER_OR_EQUAL = range(6)
# DnhReduceOp
DNH_SUM, DNH_PRODUCT, DNH_MIN, DNH_MAX, DNH_ALL, DNH_ANY, DNH_COUNT_TRUE = range(7)
# DnhArgReduceOp
DNH_ARG_MIN, DNH_ARG_MAX = range(2)

# SpecialIdx.NotFound (Tensor/Tensor/TensorRng.fs:24)
NOT_FOUND = -(2 ** 63) + 4


class DnhTensor(C.Structure):
    _fields_ = [
        ("base", C.c_void_p),
        ("offset", C.c_int64),
        ("ndims", C.c_int32),
        ("dtype", C.c_int32),
        ("shape", C.c_int64 * DNH_MAX_DIMS),
        ("stride", C.c_int64 * DNH_MAX_DIMS),
    ]


class DnhDeviceInfo(C.Structure):
    _fields_ = [
        ("device", C.c_int32),
        ("compute_units", C.c_int32),
        ("wavefront_size", C.c_int32),
        ("max_threads_per_block", C.c_int32),
        ("lds_bytes_per_block", C.c_int64),
        ("total_memory_bytes", C.c_int64),
        ("l2_bytes", C.c_int64),
        ("clock_khz", C.c_int32),
        ("memory_clock_khz", C.c_int32),
        ("name", C.c_char * 128),
        ("arch", C.c_char * 64),
    ]


class DnhPoolStats(C.Structure):
    _fields_ = [("live_bytes", C.c_int64), ("cached_bytes", C.c_int64), ("limit_bytes", C.c_int64),
                ("hits", C.c_int64), ("misses", C.c_int64)]


def make_descriptor(base: int, dtype, shape, stride, offset: int) -> DnhTensor:
    """Builds a descriptor from a storage pointer and a TensorLayout triple (elements, not bytes)."""
    nd = len(shape)
    if nd > DNH_MAX_DIMS:
        raise ValueError(f"rank {nd} exceeds the backend's limit of {DNH_MAX_DIMS}")
    d = DnhTensor()
    d.base = base
    d.offset = int(offset)
    d.ndims = nd
    d.dtype = dtype_code(dtype)
    for i in range(nd):
        d.shape[i] = int(shape[i])
        d.stride[i] = int(stride[i])
    return d


# name -> (argtypes after which product entry points append `void* stream`)
P = C.POINTER
_T = P(DnhTensor)
_TT = P(P(DnhTensor))
OP_SIGNATURES = {
    "fill_const": [_T, C.c_void_p],
    "fill_incrementing": [_T, C.c_void_p, C.c_void_p],
    "copy": [_T, _T],
    "convert": [_T, _T],
    "unary": [C.c_int32, _T, _T],
    "is_finite": [_T, _T],
    "binary": [C.c_int32, _T, _T, _T],
    "compare": [C.c_int32, _T, _T, _T],
    "if_then_else": [_T, _T, _T, _T],
    "reduce_last_axis": [C.c_int32, _T, _T],
    "arg_reduce_last_axis": [C.c_int32, _T, _T],
    "find_last_axis": [C.c_void_p, _T, _T],
    "gather": [_T, _TT, C.c_int32, _T],
    "scatter": [_T, _TT, C.c_int32, _T],
    "masked_get": [_T, _T, _TT, C.c_int32],
    "masked_set": [_T, _TT, C.c_int32, _T],
    "true_indices": [_T, _T],
    "dot": [_T, _T, _T],
    "batched_invert": [_T, _T],
}

# entry points the CPU oracle does not restate in C (it uses numpy's LAPACK, which is what the reference's host backend calls)
LAPACK_OP_SIGNATURES = {
    "batched_svd": [_T, _T, _T, _T],          # s, u (or NULL), v (or NULL), src
    "symmetric_eig": [C.c_int32, _T, _T, _T],  # part (0 upper, 1 lower), eigvals, eigvecs, src
}

# entry points with no counterpart in the reference's interface (hence none in the oracle)
DEVICE_ONLY_OP_SIGNATURES = {
    "reduce_last_axis_noalloc": [C.c_int32, _T, _T],   # dnh_reduce_last_axis with its partial results in a static device array
}
STATIC_SCRATCH_BYTES = 8 << 20

# every symbol include/tensor_hip.h declares
EXPORTED_SYMBOLS = [
    "dnh_init", "dnh_device_info", "dnh_last_error", "dnh_async_error", "dnh_set_option", "dnh_get_option", "dnh_scatter_workspace_bytes",
    "dnh_alloc", "dnh_free", "dnh_alloc_async", "dnh_free_async", "dnh_pool_trim", "dnh_pool_set_limit", "dnh_pool_stats",
    "dnh_host_alloc", "dnh_host_free", "dnh_memset",
    "dnh_memcpy_h2d", "dnh_memcpy_d2h", "dnh_memcpy_d2d",
    "dnh_stream_create", "dnh_stream_destroy", "dnh_stream_sync", "dnh_device_sync",
    "dnh_event_create", "dnh_event_destroy", "dnh_event_record", "dnh_event_sync", "dnh_event_elapsed_ms",
] + ["dnh_" + k for k in OP_SIGNATURES] + ["dnh_" + k for k in LAPACK_OP_SIGNATURES] + ["dnh_" + k for k in DEVICE_ONLY_OP_SIGNATURES]
