"""HostRef device — the CPU oracle behind the same frontend (TEST INFRASTRUCTURE ONLY).

Loads oracle/libhostref.so (the C++ restatement of the reference's Host backend, oracle/hostref.cpp) and exposes it as a
device with the ITensorDevice / ITensorStorage / ITensorBackend shape, so parity tests run the identical frontend call
sequence on both devices.  Storage is a flat NumPy array, like TensorHostStorage's .NET array
(Tensor/Tensor/Host/HostBackend.fs:20-98); the device is Zeroed=true (HostBackend.fs:690).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

from deepnet_amd import abi
from deepnet_amd import layout as L
from deepnet_amd.backend import CAbiTensorBackend, ITensorDevice, ITensorStorage, SingularMatrixException
from deepnet_amd.tensor import Tensor

_DIR = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_DIR, "libhostref.so")
_lib = None


def build():
    subprocess.check_call(["make", "-C", _DIR, "-s"])


def load() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        lib = C.CDLL(_LIB_PATH)
        for name, args in abi.OP_SIGNATURES.items():
            fn = getattr(lib, "href_" + name)
            fn.argtypes = list(args)
            fn.restype = C.c_int32
        lib.href_set_threads.argtypes = [C.c_int32]
        lib.href_get_threads.restype = C.c_int32
        _lib = lib
    return _lib


_EXC = {
    abi.DNH_ERR_INVALID_ARG: ValueError,
    abi.DNH_ERR_NOT_SUPPORTED: NotImplementedError,
    abi.DNH_ERR_INDEX_OUT_OF_RANGE: IndexError,
    abi.DNH_ERR_SINGULAR_MATRIX: SingularMatrixException,
}


class TensorHostRefStorage(ITensorStorage):
    def __init__(self, nElems, dtype, dev, array=None):
        self.Dev = dev
        self.DataType = np.dtype(dtype)
        self.NElems = int(nElems)
        self.HostArray = np.zeros(max(self.NElems, 1), dtype=self.DataType) if array is None else array

    def Pointer(self) -> int:
        return self.HostArray.ctypes.data

    def Backend(self, layout):
        return TensorHostRefBackend(layout, self)


class TensorHostRefBackend(CAbiTensorBackend):
    def _call(self, name, *args):
        status = getattr(load(), "href_" + name)(*args)
        if status != abi.DNH_OK:
            raise _EXC.get(status, RuntimeError)(f"hostref {name} failed with status {status}")

    def GetItem(self, idx):
        return self.Storage.HostArray[L.addr(idx, self.Layout)]

    def SetItem(self, idx, value):
        self.Storage.HostArray[L.addr(idx, self.Layout)] = value

    def Transfer(self, trgt, src) -> bool:
        return False  # HostBackend.fs:210-211: the device backends implement transfers

    # The reference's host backend hands these two to LAPACK (HostBackend.fs:579-628: gesdd with job 'A' / 'N', syevd with job 'V');
    # numpy.linalg.svd and numpy.linalg.eigh call the same routines, so they are the restatement.  Bit-level parity with MKL is
    # unpinned (library build and threading), and vectors are only defined up to sign: the tests compare through properties.
    def BatchedSVD(self, trgtS, trgtUV, src1):
        a = toNumpy(src1)
        if a.dtype.kind != "f":
            raise NotImplementedError("this operation is only supported for floating point numbers")
        if trgtUV is None:
            _assign(trgtS, np.linalg.svd(a, compute_uv=False))
        else:
            u, s, vt = np.linalg.svd(a, full_matrices=True)
            _assign(trgtS, s)
            _assign(trgtUV[0], u)
            _assign(trgtUV[1], np.swapaxes(vt, -1, -2))

    def SymmetricEigenDecomposition(self, part, trgtEigVals, trgtEigVecs, src):
        a = toNumpy(src)
        if a.dtype.kind != "f":
            raise NotImplementedError("this operation is only supported for floating point numbers")
        w, v = np.linalg.eigh(a, UPLO="U" if part == "Upper" else "L")
        _assign(trgtEigVals, w)
        _assign(trgtEigVecs, v)


class TensorHostRefDevice(ITensorDevice):
    Id = "HostRef"
    Zeroed = True

    def Create(self, nElems, dtype):
        return TensorHostRefStorage(nElems, dtype, self)


Dev = TensorHostRefDevice()


def ofNumpy(arr: np.ndarray) -> Tensor:
    """Row-major host tensor holding a copy of `arr`."""
    arr = np.asarray(arr)
    shape = arr.shape                       # np.ascontiguousarray turns a 0-d array into shape (1,)
    arr = np.ascontiguousarray(arr)
    flat = arr.reshape(-1).copy()
    if flat.size == 0:
        flat = np.zeros(1, dtype=arr.dtype)
    st = TensorHostRefStorage(arr.size, arr.dtype, Dev, flat)
    return Tensor(L.newC(shape), st)


def toNumpy(t: Tensor) -> np.ndarray:
    lay = t.Layout
    out = np.empty(lay.Shape, dtype=t.DataType)
    if lay.NElems:
        isz = t.DataType.itemsize
        view = np.lib.stride_tricks.as_strided(t.Storage.HostArray[lay.Offset:], shape=lay.Shape, strides=[s * isz for s in lay.Stride])
        out[...] = view
    return out


def _assign(t: Tensor, values: np.ndarray):
    """Writes `values` into the (possibly strided) host tensor t."""
    lay = t.Layout
    if lay.NElems:
        isz = t.DataType.itemsize
        view = np.lib.stride_tricks.as_strided(t.Storage.HostArray[lay.Offset:], shape=lay.Shape, strides=[s * isz for s in lay.Stride])
        view[...] = np.asarray(values, dtype=t.DataType).reshape(lay.Shape)


def transfer(t: Tensor) -> Tensor:
    """HostTensor.transfer: brings a tensor of any device to this host device (Tensor.fs:696-711)."""
    return t.Transfer(Dev)


def set_threads(n: int):
    load().href_set_threads(int(n))


def get_threads() -> int:
    return int(load().href_get_threads())
