"""Plugin surface: Python mirror of the reference's ITensorDevice / ITensorStorage / ITensorBackend
(Tensor/Tensor/TensorBackend.fs:13-146) and a backend base class that implements every ITensorBackend member on top
of a C ABI whose entry points take DnhTensor descriptors (include/tensor_hip.h).

Member names, argument order and meaning follow the reference interface one to one; .NET exceptions map to Python
ones: InvalidOperation/Argument -> ValueError, NotSupported -> NotImplementedError, IndexOutOfRange -> IndexError.
"""
from __future__ import annotations

import ctypes as C
from typing import List, Optional, Sequence

import numpy as np

from . import abi
from .layout import TensorLayout


MatrixPart = ("Upper", "Lower")   # Tensor/Tensor/TensorBackend.fs: which triangle a symmetric operation reads


class SingularMatrixException(ArithmeticError):
    """Raised when a matrix that is not invertible is inverted (Tensor/Tensor/Tensor.fs:2831-2834)."""


class ITensorDevice:
    """TensorBackend.fs:22-30.  Devices compare by Id (BaseTensorDevice, TensorBackend.fs:149-180)."""
    Id: str = "?"
    Zeroed: bool = False

    def Create(self, nElems: int, dtype) -> "ITensorStorage":
        raise NotImplementedError

    def __eq__(self, other):
        return isinstance(other, ITensorDevice) and self.Id == other.Id

    def __hash__(self):
        return hash(self.Id)

    def __repr__(self):
        return self.Id


class ITensorStorage:
    """TensorBackend.fs:13-20."""
    Dev: ITensorDevice
    DataType: np.dtype
    NElems: int

    def Backend(self, layout: TensorLayout) -> "CAbiTensorBackend":
        raise NotImplementedError

    # device pointer (or host address) of element 0, as an integer
    def Pointer(self) -> int:
        raise NotImplementedError


def _scalar_buf(value, dtype):
    """One host element of `dtype` as a ctypes buffer (the `const void* value` arguments of the ABI)."""
    arr = np.array([value], dtype=dtype)
    return arr, arr.ctypes.data_as(C.c_void_p)


class CAbiTensorBackend:
    """ITensorBackend<'T> (TensorBackend.fs:64-146) over a C ABI.  Subclasses provide `_call(name, *args)`, which invokes
    entry point `name` (a key of abi.OP_SIGNATURES) and raises on a non-zero status, and the Item / Transfer members."""

    def __init__(self, layout: TensorLayout, storage: ITensorStorage):
        self.Layout = layout
        self.Storage = storage

    # -- plumbing ---------------------------------------------------------------------------------------------------
    def _call(self, name: str, *args):
        raise NotImplementedError

    def _after_indexed_op(self):
        """Hook run after Gather/Scatter (device backends read their index error flag here)."""

    @staticmethod
    def _desc(t) -> abi.DnhTensor:
        lay = t.Layout
        return abi.make_descriptor(t.Storage.Pointer(), t.Storage.DataType, lay.Shape, lay.Stride, lay.Offset)

    @classmethod
    def _desc_list(cls, ts: Sequence[Optional[object]]):
        """NULL-able array of descriptor pointers (index tensors / masks); returns (array, keepalive)."""
        descs = [cls._desc(t) if t is not None else None for t in ts]
        arr = (C.POINTER(abi.DnhTensor) * max(len(ts), 1))()
        for i, d in enumerate(descs):
            arr[i] = C.pointer(d) if d is not None else C.POINTER(abi.DnhTensor)()
        return arr, descs

    def _unary(self, op, trgt, src1):
        self._call("unary", op, C.byref(self._desc(trgt)), C.byref(self._desc(src1)))

    def _binary(self, op, trgt, src1, src2):
        self._call("binary", op, C.byref(self._desc(trgt)), C.byref(self._desc(src1)), C.byref(self._desc(src2)))

    def _compare(self, op, trgt, src1, src2):
        self._call("compare", op, C.byref(self._desc(trgt)), C.byref(self._desc(src1)), C.byref(self._desc(src2)))

    def _reduce(self, op, trgt, src1):
        self._call("reduce_last_axis", op, C.byref(self._desc(trgt)), C.byref(self._desc(src1)))

    # -- ITensorBackend members (TensorBackend.fs:65-146) --------------------------------------------------------------
    def Copy(self, trgt, src):
        self._call("copy", C.byref(self._desc(trgt)), C.byref(self._desc(src)))

    def Convert(self, trgt, src):
        self._call("convert", C.byref(self._desc(trgt)), C.byref(self._desc(src)))

    def FillConst(self, value, trgt):
        keep, p = _scalar_buf(value, trgt.Storage.DataType)
        self._call("fill_const", C.byref(self._desc(trgt)), p)

    def FillIncrementing(self, start, incr, trgt):
        k1, p1 = _scalar_buf(start, trgt.Storage.DataType)
        k2, p2 = _scalar_buf(incr, trgt.Storage.DataType)
        self._call("fill_incrementing", C.byref(self._desc(trgt)), p1, p2)

    def UnaryPlus(self, trgt, src1): self._unary(abi.DNH_UNARY_PLUS, trgt, src1)
    def UnaryMinus(self, trgt, src1): self._unary(abi.DNH_UNARY_MINUS, trgt, src1)
    def Abs(self, trgt, src1): self._unary(abi.DNH_ABS, trgt, src1)
    def Sgn(self, trgt, src1): self._unary(abi.DNH_SGN, trgt, src1)
    def Log(self, trgt, src1): self._unary(abi.DNH_LOG, trgt, src1)
    def Log10(self, trgt, src1): self._unary(abi.DNH_LOG10, trgt, src1)
    def Exp(self, trgt, src1): self._unary(abi.DNH_EXP, trgt, src1)
    def Sin(self, trgt, src1): self._unary(abi.DNH_SIN, trgt, src1)
    def Cos(self, trgt, src1): self._unary(abi.DNH_COS, trgt, src1)
    def Tan(self, trgt, src1): self._unary(abi.DNH_TAN, trgt, src1)
    def Asin(self, trgt, src1): self._unary(abi.DNH_ASIN, trgt, src1)
    def Acos(self, trgt, src1): self._unary(abi.DNH_ACOS, trgt, src1)
    def Atan(self, trgt, src1): self._unary(abi.DNH_ATAN, trgt, src1)
    def Sinh(self, trgt, src1): self._unary(abi.DNH_SINH, trgt, src1)
    def Cosh(self, trgt, src1): self._unary(abi.DNH_COSH, trgt, src1)
    def Tanh(self, trgt, src1): self._unary(abi.DNH_TANH, trgt, src1)
    def Sqrt(self, trgt, src1): self._unary(abi.DNH_SQRT, trgt, src1)
    def Ceiling(self, trgt, src1): self._unary(abi.DNH_CEILING, trgt, src1)
    def Floor(self, trgt, src1): self._unary(abi.DNH_FLOOR, trgt, src1)
    def Round(self, trgt, src1): self._unary(abi.DNH_ROUND, trgt, src1)
    def Truncate(self, trgt, src1): self._unary(abi.DNH_TRUNCATE, trgt, src1)

    def IsFinite(self, trgt, src1):
        self._call("is_finite", C.byref(self._desc(trgt)), C.byref(self._desc(src1)))

    def Add(self, trgt, src1, src2): self._binary(abi.DNH_ADD, trgt, src1, src2)
    def Subtract(self, trgt, src1, src2): self._binary(abi.DNH_SUBTRACT, trgt, src1, src2)
    def Multiply(self, trgt, src1, src2): self._binary(abi.DNH_MULTIPLY, trgt, src1, src2)
    def Divide(self, trgt, src1, src2): self._binary(abi.DNH_DIVIDE, trgt, src1, src2)
    def Modulo(self, trgt, src1, src2): self._binary(abi.DNH_MODULO, trgt, src1, src2)
    def Power(self, trgt, src1, src2): self._binary(abi.DNH_POWER, trgt, src1, src2)
    def MaxElemwise(self, trgt, src1, src2): self._binary(abi.DNH_MAX_ELEMWISE, trgt, src1, src2)
    def MinElemwise(self, trgt, src1, src2): self._binary(abi.DNH_MIN_ELEMWISE, trgt, src1, src2)

    def Equal(self, trgt, src1, src2): self._compare(abi.DNH_EQUAL, trgt, src1, src2)
    def NotEqual(self, trgt, src1, src2): self._compare(abi.DNH_NOT_EQUAL, trgt, src1, src2)
    def Less(self, trgt, src1, src2): self._compare(abi.DNH_LESS, trgt, src1, src2)
    def LessOrEqual(self, trgt, src1, src2): self._compare(abi.DNH_LESS_OR_EQUAL, trgt, src1, src2)
    def Greater(self, trgt, src1, src2): self._compare(abi.DNH_GREATER, trgt, src1, src2)
    def GreaterOrEqual(self, trgt, src1, src2): self._compare(abi.DNH_GREATER_OR_EQUAL, trgt, src1, src2)

    def Negate(self, trgt, src1): self._unary(abi.DNH_NEGATE, trgt, src1)
    def And(self, trgt, src1, src2): self._binary(abi.DNH_AND, trgt, src1, src2)
    def Or(self, trgt, src1, src2): self._binary(abi.DNH_OR, trgt, src1, src2)
    def Xor(self, trgt, src1, src2): self._binary(abi.DNH_XOR, trgt, src1, src2)

    def IfThenElse(self, trgt, cond, ifTrue, ifFalse):
        self._call("if_then_else", C.byref(self._desc(trgt)), C.byref(self._desc(cond)), C.byref(self._desc(ifTrue)),
                   C.byref(self._desc(ifFalse)))

    def Gather(self, trgt, srcIdxs: List[Optional[object]], src):
        arr, keep = self._desc_list(srcIdxs)
        self._call("gather", C.byref(self._desc(trgt)), arr, len(srcIdxs), C.byref(self._desc(src)))
        self._after_indexed_op()

    def Scatter(self, trgt, trgtIdxs: List[Optional[object]], src):
        arr, keep = self._desc_list(trgtIdxs)
        self._call("scatter", C.byref(self._desc(trgt)), arr, len(trgtIdxs), C.byref(self._desc(src)))
        self._after_indexed_op()

    def MaskedGet(self, trgt, src, masks: List[Optional[object]]):
        arr, keep = self._desc_list(masks)
        self._call("masked_get", C.byref(self._desc(trgt)), C.byref(self._desc(src)), arr, len(masks))

    def MaskedSet(self, trgt, masks: List[Optional[object]], src):
        arr, keep = self._desc_list(masks)
        self._call("masked_set", C.byref(self._desc(trgt)), arr, len(masks), C.byref(self._desc(src)))

    def TrueIndices(self, trgt, src1):
        self._call("true_indices", C.byref(self._desc(trgt)), C.byref(self._desc(src1)))

    def SumLastAxis(self, trgt, src1): self._reduce(abi.DNH_SUM, trgt, src1)
    def ProductLastAxis(self, trgt, src1): self._reduce(abi.DNH_PRODUCT, trgt, src1)
    def MinLastAxis(self, trgt, src1): self._reduce(abi.DNH_MIN, trgt, src1)
    def MaxLastAxis(self, trgt, src1): self._reduce(abi.DNH_MAX, trgt, src1)
    def AllLastAxis(self, trgt, src1): self._reduce(abi.DNH_ALL, trgt, src1)
    def AnyLastAxis(self, trgt, src1): self._reduce(abi.DNH_ANY, trgt, src1)
    def CountTrueLastAxis(self, trgt, src1): self._reduce(abi.DNH_COUNT_TRUE, trgt, src1)

    def ArgMinLastAxis(self, trgt, src1):
        self._call("arg_reduce_last_axis", abi.DNH_ARG_MIN, C.byref(self._desc(trgt)), C.byref(self._desc(src1)))

    def ArgMaxLastAxis(self, trgt, src1):
        self._call("arg_reduce_last_axis", abi.DNH_ARG_MAX, C.byref(self._desc(trgt)), C.byref(self._desc(src1)))

    def FindLastAxis(self, value, trgt, src1):
        keep, p = _scalar_buf(value, src1.Storage.DataType)
        self._call("find_last_axis", p, C.byref(self._desc(trgt)), C.byref(self._desc(src1)))

    def _dot(self, trgt, src1, src2):
        self._call("dot", C.byref(self._desc(trgt)), C.byref(self._desc(src1)), C.byref(self._desc(src2)))

    def VecVecDot(self, trgt, src1, src2): self._dot(trgt, src1, src2)
    def MatVecDot(self, trgt, src1, src2): self._dot(trgt, src1, src2)
    def MatMatDot(self, trgt, src1, src2): self._dot(trgt, src1, src2)
    def BatchedMatMatDot(self, trgt, src1, src2): self._dot(trgt, src1, src2)

    # the reference's CUDA backend also leaves SVD/eigen unsupported (CudaBackend.fs:486-492)
    def BatchedSVD(self, trgtS, trgtUV, src1):
        u, v = (None, None) if trgtUV is None else (C.byref(self._desc(trgtUV[0])), C.byref(self._desc(trgtUV[1])))
        self._call("batched_svd", C.byref(self._desc(trgtS)), u, v, C.byref(self._desc(src1)))

    def BatchedInvert(self, trgt, src1):
        self._call("batched_invert", C.byref(self._desc(trgt)), C.byref(self._desc(src1)))

    def SymmetricEigenDecomposition(self, part, trgtEigVals, trgtEigVecs, src):
        self._call("symmetric_eig", MatrixPart.index(part), C.byref(self._desc(trgtEigVals)), C.byref(self._desc(trgtEigVecs)),
                   C.byref(self._desc(src)))
