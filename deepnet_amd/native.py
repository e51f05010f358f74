"""Loader of libtensor_hip.so — the only way into the HIP kernels.  There is no CPU fallback: if the library is not
built, or no GPU is present when an entry point runs, the failure is raised to the caller."""
import ctypes as C
import os

from . import abi

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libtensor_hip.so")
_lib = None


from .backend import SingularMatrixException  # noqa: E402


class HipError(RuntimeError):
    pass


def lib_path() -> str:
    return _LIB_PATH


def load() -> C.CDLL:
    """Loads the library and declares every entry point of include/tensor_hip.h."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise ImportError(f"{_LIB_PATH} is missing: build it with `make -C deepnet_amd/csrc` "
                          "(or `python -c 'import __graft_entry__ as g; g.build()'`)")
    lib = C.CDLL(_LIB_PATH)
    vp, i32, sz = C.c_void_p, C.c_int32, C.c_size_t
    sigs = {
        "dnh_init": [i32],
        "dnh_device_info": [C.POINTER(abi.DnhDeviceInfo)],
        "dnh_last_error": [C.c_char_p, sz],
        "dnh_async_error": [vp, C.POINTER(i32)],
        "dnh_set_option": [C.c_char_p, i32],
        "dnh_get_option": [C.c_char_p, C.POINTER(i32)],
        "dnh_scatter_workspace_bytes": [i32, C.c_int64, C.c_int64, C.POINTER(sz)],
        "dnh_alloc": [sz, C.POINTER(vp)],
        "dnh_free": [vp],
        "dnh_alloc_async": [sz, vp, C.POINTER(vp)],
        "dnh_free_async": [vp, vp],
        "dnh_pool_trim": [],
        "dnh_pool_set_limit": [sz],
        "dnh_pool_stats": [C.POINTER(abi.DnhPoolStats)],
        "dnh_host_alloc": [sz, C.POINTER(vp)],
        "dnh_host_free": [vp],
        "dnh_memset": [vp, i32, sz, vp],
        "dnh_memcpy_h2d": [vp, vp, sz, vp, i32],
        "dnh_memcpy_d2h": [vp, vp, sz, vp, i32],
        "dnh_memcpy_d2d": [vp, vp, sz, vp, i32],
        "dnh_stream_create": [C.POINTER(vp)],
        "dnh_stream_destroy": [vp],
        "dnh_stream_sync": [vp],
        "dnh_device_sync": [],
        "dnh_event_create": [C.POINTER(vp)],
        "dnh_event_destroy": [vp],
        "dnh_event_record": [vp, vp],
        "dnh_event_sync": [vp],
        "dnh_event_elapsed_ms": [vp, vp, C.POINTER(C.c_float)],
    }
    for name, args in list(abi.OP_SIGNATURES.items()) + list(abi.LAPACK_OP_SIGNATURES.items()) + list(abi.DEVICE_ONLY_OP_SIGNATURES.items()):
        sigs["dnh_" + name] = list(args) + [vp]  # every op takes the stream last
    for name, args in sigs.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = i32
    _lib = lib
    return lib


_EXC = {
    abi.DNH_ERR_INVALID_ARG: ValueError,
    abi.DNH_ERR_NOT_SUPPORTED: NotImplementedError,
    abi.DNH_ERR_OUT_OF_MEMORY: MemoryError,
    abi.DNH_ERR_HIP: HipError,
    abi.DNH_ERR_INDEX_OUT_OF_RANGE: IndexError,
    abi.DNH_ERR_NOT_INITIALIZED: HipError,
    abi.DNH_ERR_SINGULAR_MATRIX: SingularMatrixException,
    abi.DNH_ERR_NO_CONVERGENCE: ArithmeticError,
}


def set_option(name: str, value: int) -> None:
    """dnh_set_option: a process-wide tuning switch of the library (which kernel computes a result, never its contract)."""
    check(load().dnh_set_option(name.encode(), int(value)))


def get_option(name: str) -> int:
    v = C.c_int32()
    check(load().dnh_get_option(name.encode(), C.byref(v)))
    return v.value


class option:
    """`with native.option("dot_bf16x3", 0): ...` sets a switch for the calls issued inside the block."""

    def __init__(self, name: str, value: int):
        self.name, self.value = name, value

    def __enter__(self):
        self.saved = get_option(self.name)
        set_option(self.name, self.value)
        return self

    def __exit__(self, *exc):
        set_option(self.name, self.saved)
        return False


def last_error() -> str:
    buf = C.create_string_buffer(1024)
    load().dnh_last_error(buf, len(buf))
    return buf.value.decode("utf-8", "replace")


def check(status: int):
    """Maps a DnhStatus to the exception the reference's backend would raise."""
    if status != abi.DNH_OK:
        raise _EXC.get(status, HipError)(last_error() or f"libtensor_hip status {status}")
