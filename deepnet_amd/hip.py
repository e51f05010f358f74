"""HipTensor device: TensorHipDevice / TensorHipStorage / TensorHipBackend and the `HipTensor` creation functions.

Python mirror of what a Deep.Net `Tensor/Tensor/Hip/*.fs` would contain, structured as the reference's CUDA files are:
storage + backend + device (Tensor/Tensor/Cuda/CudaBackend.fs:54-93, 117-508), thread-local configuration
(Tensor/Tensor/Cuda/CudaCfg.fs:14-60) and the frontend module (Tensor/Tensor/Cuda/CudaFrontend.fs:30-149).
All computation is done by libtensor_hip.so through the C ABI of include/tensor_hip.h.
"""
from __future__ import annotations

import ctypes as C
import threading

import numpy as np

from . import abi, native
from .backend import CAbiTensorBackend, ITensorDevice, ITensorStorage
from .layout import TensorLayout
from . import layout as L
from .tensor import Tensor


class _Cfg(threading.local):
    """Thread-local options, as Tensor.Cuda.Cfg (CudaCfg.fs:14-60).
    Stream: hipStream_t (int) all ops of this thread are issued on; 0 = default stream.
    Stacktrace: when True (default) every Gather/Scatter is followed by a read of the device index-error flag so an
    out-of-range index raises IndexError at the faulting call, like the host backend does."""

    def __init__(self):
        self.Stream = 0
        self.Stacktrace = True


Cfg = _Cfg()


class TensorHipStorage(ITensorStorage):
    """Owns one device allocation (CudaBackend.fs:54-93).  Released when collected.

    The block comes from the library's stream-ordered cache, tagged with the stream that is current at creation.  While
    every operation on the storage is issued on that stream, release hands the block back to the cache without waiting
    for the device; once its pointer has been taken under another stream it is released with the synchronising free."""

    def __init__(self, nElems: int, dtype, dev: "TensorHipDevice", external_ptr: int = 0):
        self.Dev = dev
        self.DataType = np.dtype(dtype)
        self.NElems = int(nElems)
        self._lib = native.load()
        self._stream = Cfg.Stream
        self._single_stream = True
        self._owned = not external_ptr     # a storage made by usingPtr references memory it never frees
        if external_ptr:
            self._ptr = int(external_ptr)
            return
        ptr = C.c_void_p()
        native.check(self._lib.dnh_alloc_async(max(self.NElems, 1) * self.DataType.itemsize, self._stream, C.byref(ptr)))
        self._ptr = ptr.value

    def Pointer(self) -> int:
        # every operation fetches the pointer when it is issued, under the stream it is issued on
        if Cfg.Stream != self._stream:
            self._single_stream = False
        return self._ptr

    @property
    def ByteSize(self) -> int:
        return self.NElems * self.DataType.itemsize

    def Backend(self, layout: TensorLayout) -> "TensorHipBackend":
        return TensorHipBackend(layout, self)

    def __del__(self):
        try:
            if getattr(self, "_ptr", None) and getattr(self, "_owned", False):
                if self._single_stream:
                    self._lib.dnh_free_async(self._ptr, self._stream)
                else:
                    self._lib.dnh_free(self._ptr)
                self._ptr = None
        except Exception:
            pass


class TensorHipBackend(CAbiTensorBackend):
    def __init__(self, layout, storage: TensorHipStorage):
        super().__init__(layout, storage)
        self._lib = storage._lib

    def _call(self, name, *args):
        native.check(getattr(self._lib, "dnh_" + name)(*args, Cfg.Stream))

    def _after_indexed_op(self):
        if Cfg.Stacktrace:
            code = C.c_int32(0)
            native.check(self._lib.dnh_async_error(Cfg.Stream, C.byref(code)))
            native.check(code.value)

    # single elements cross with a synchronous 1-element copy (CudaBackend.fs:77-93)
    def GetItem(self, idx):
        a = L.addr(idx, self.Layout)
        out = np.empty(1, dtype=self.Storage.DataType)
        isz = self.Storage.DataType.itemsize
        native.check(self._lib.dnh_memcpy_d2h(out.ctypes.data, self.Storage.Pointer() + a * isz, isz, Cfg.Stream, 1))
        return out[0]

    def SetItem(self, idx, value):
        a = L.addr(idx, self.Layout)
        v = np.array([value], dtype=self.Storage.DataType)
        isz = self.Storage.DataType.itemsize
        native.check(self._lib.dnh_memcpy_h2d(self.Storage.Pointer() + a * isz, v.ctypes.data, isz, Cfg.Stream, 1))

    def Transfer(self, trgt, src) -> bool:
        """Host <-> device (CudaBackend.fs:206-270).  A host storage is any storage exposing `HostArray` (a 1-d NumPy
        array of its elements).  The device side must be row-major contiguous; other layouts go through a device copy."""
        ts, ss = trgt.Storage, src.Storage
        if isinstance(ts, TensorHipStorage) and hasattr(ss, "HostArray"):
            host = _gather_host(ss.HostArray, src.Layout)            # contiguous row-major host copy of the view
            if L.isC(trgt.Layout):
                dst = ts.Pointer() + trgt.Layout.Offset * ts.DataType.itemsize
                native.check(self._lib.dnh_memcpy_h2d(dst, host.ctypes.data, host.nbytes, Cfg.Stream, 1))
            else:
                tmp = Tensor.new(trgt.Shape, trgt.Dev, trgt.DataType)
                native.check(self._lib.dnh_memcpy_h2d(tmp.Storage.Pointer(), host.ctypes.data, host.nbytes, Cfg.Stream, 1))
                trgt.Backend.Copy(trgt, tmp)
                native.check(self._lib.dnh_stream_sync(Cfg.Stream))
            return True
        if hasattr(ts, "HostArray") and isinstance(ss, TensorHipStorage):
            if not L.isC(src.Layout):
                src = src.Copy()
            host = np.empty(src.NElems, dtype=src.DataType)
            p = src.Storage.Pointer() + src.Layout.Offset * src.DataType.itemsize
            native.check(self._lib.dnh_memcpy_d2h(host.ctypes.data, p, host.nbytes, Cfg.Stream, 1))
            _scatter_host(ts.HostArray, trgt.Layout, host)
            return True
        return False


def _gather_host(flat: np.ndarray, lay: TensorLayout) -> np.ndarray:
    """Row-major contiguous copy of the view `lay` of a flat host array (pure data movement on the host side of a transfer)."""
    isz = flat.dtype.itemsize
    view = np.lib.stride_tricks.as_strided(flat[lay.Offset:] if lay.NElems else flat[:0], shape=lay.Shape,
                                           strides=[s * isz for s in lay.Stride], writeable=False) if lay.NElems else np.empty(lay.Shape, flat.dtype)
    return np.ascontiguousarray(view)


def _scatter_host(flat: np.ndarray, lay: TensorLayout, data: np.ndarray):
    if lay.NElems == 0:
        return
    isz = flat.dtype.itemsize
    view = np.lib.stride_tricks.as_strided(flat[lay.Offset:], shape=lay.Shape, strides=[s * isz for s in lay.Stride])
    view[...] = data.reshape(lay.Shape)


class TensorHipDevice(ITensorDevice):
    """CudaBackend.fs:497-507: Id, Create, Zeroed=false (fresh storage is uninitialised; `zeros` launches FillConst)."""
    Id = "Hip"
    Zeroed = False

    def Create(self, nElems, dtype):
        return TensorHipStorage(nElems, dtype, self)

    def Info(self) -> abi.DnhDeviceInfo:
        info = abi.DnhDeviceInfo()
        native.check(native.load().dnh_device_info(C.byref(info)))
        return info


Dev = TensorHipDevice()


# ---- the HipTensor "module" (CudaFrontend.fs:30-149) ------------------------------------------------------------------------

def ofNumpy(arr: np.ndarray) -> Tensor:
    """Uploads a NumPy array (any strides) into a new row-major device tensor (analogue of CudaTensor.transfer of a host tensor)."""
    arr = np.asarray(arr)
    if arr.dtype not in abi.NUMPY_TO_DTYPE:
        raise NotImplementedError(f"element type {arr.dtype} is not supported by the HIP backend")
    host = np.ascontiguousarray(arr)
    t = Tensor.new(arr.shape, Dev, arr.dtype)
    if host.nbytes:
        native.check(native.load().dnh_memcpy_h2d(t.Storage.Pointer(), host.ctypes.data, host.nbytes, Cfg.Stream, 1))
    return t


def toNumpy(t: Tensor) -> np.ndarray:
    """Downloads a device tensor (any layout) as a row-major NumPy array."""
    if not isinstance(t.Storage, TensorHipStorage):
        raise ValueError("toNumpy expects a tensor stored on the Hip device")
    if not L.isC(t.Layout):
        t = t.Copy()
    out = np.empty(t.Shape, dtype=t.DataType)
    if out.nbytes:
        p = t.Storage.Pointer() + t.Layout.Offset * t.DataType.itemsize
        native.check(native.load().dnh_memcpy_d2h(out.ctypes.data, p, out.nbytes, Cfg.Stream, 1))
    return out


def zeros(shape, dtype) -> Tensor: return Tensor.zeros(shape, Dev, dtype)
def ones(shape, dtype) -> Tensor: return Tensor.ones(shape, Dev, dtype)
def filled(shape, value, dtype) -> Tensor: return Tensor.filled(shape, value, Dev, dtype)
def scalar(value, dtype) -> Tensor: return Tensor.scalar(value, Dev, dtype)
def counting(n, dtype=np.int64) -> Tensor: return Tensor.counting(n, Dev, dtype)
def transfer(t: Tensor) -> Tensor: return t.Transfer(Dev)


def usingPtr(ptr: int, sizeInBytes: int, dtype, layout: TensorLayout) -> Tensor:
    """A tensor over existing device memory (CudaTensor.usingPtr / usingPtrAndType, Cuda/CudaFrontend.fs:129-149): the data is
    referenced, not copied, and never freed by the tensor."""
    dt = np.dtype(dtype)
    if not ptr:
        raise ValueError("usingPtr: null device pointer")
    nElems = int(sizeInBytes) // dt.itemsize
    if layout.NElems:
        lo = layout.Offset + sum((n - 1) * st for n, st in zip(layout.Shape, layout.Stride) if st < 0)
        hi = layout.Offset + sum((n - 1) * st for n, st in zip(layout.Shape, layout.Stride) if st > 0)
        if lo < 0 or hi >= nElems:
            raise ValueError(f"usingPtr: the layout addresses elements {lo}..{hi} but the allocation holds {nElems}")
    return Tensor(layout, TensorHipStorage(nElems, dt, Dev, external_ptr=int(ptr)))


def synchronize():
    native.check(native.load().dnh_stream_sync(Cfg.Stream))
