"""Tensor — the device-agnostic frontend, restricted to what drives the accelerated backend path.

Python mirror of the reference's `Tensor<'T>` (Tensor/Tensor/Tensor.fs): every operation prepares a target (allocates
it row-major on the sources' device, broadcasts the sources — Tensor.fs:4520-4597) and then makes exactly one backend
call, `trgt.Backend.<Op>(trgt, srcs...)` (e.g. Tensor.fs:1343-1344, 2098, 2270-2271, 2727).  Nothing here computes on
tensor data; all arithmetic happens behind the ITensorBackend boundary.

F# operator -> Python:  + - * / % ** unary-  as usual;  .*  -> @;  ==== <<>> <<<< <<== >>>> >>==  -> == != < <= > >=;
~~~~ &&&& |||| ^^^^ -> ~ & | ^;  a.[rng] -> a[...] (slices are half-open as in Python; F# ranges are inclusive);
a.M(m) -> a.M(m) / a.setM([m], v).
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np

from . import layout as L
from .layout import TensorLayout, Rng, NewAxis, NotFound

RowMajor = "RowMajor"
ColumnMajor = "ColumnMajor"


def _same_storage(xs):
    """Tensor.CheckSameStorage (Tensor.fs:4507-4512)."""
    xs = [x for x in xs if x is not None]
    if xs and any(x.Dev != xs[0].Dev for x in xs[1:]):
        raise ValueError(f"Storage devices must be equal for this operation, but they are {[x.Dev.Id for x in xs]}.")


class Tensor:
    # ---- construction (Tensor.fs:45-60, 317-325) -----------------------------------------------------------------------
    def __init__(self, layout: TensorLayout, storage):
        self._layout = layout
        self._storage = storage
        self._backend = storage.Backend(layout)

    @staticmethod
    def new(shape: Sequence[int], dev, dtype, order=RowMajor) -> "Tensor":
        """Allocates uninitialised (or zeroed, per dev.Zeroed) storage with the given memory order (Tensor.fs:317-325)."""
        shape = tuple(int(s) for s in shape)
        if order == RowMajor:
            lay = L.newC(shape)
        elif order == ColumnMajor:
            lay = L.newF(shape)
        else:
            lay = L.newOrdered(shape, order)
        storage = dev.Create(lay.NElems, np.dtype(dtype))
        return Tensor(lay, storage)

    # ---- ITensorFrontend (TensorBackend.fs:33-61) ---------------------------------------------------------------------
    @property
    def Storage(self): return self._storage
    @property
    def Dev(self): return self._storage.Dev
    @property
    def Backend(self): return self._backend
    @property
    def Layout(self) -> TensorLayout: return self._layout
    @property
    def Shape(self): return list(self._layout.Shape)
    @property
    def Stride(self): return list(self._layout.Stride)
    @property
    def Offset(self): return self._layout.Offset
    @property
    def NDims(self): return self._layout.NDims
    @property
    def NElems(self): return self._layout.NElems
    @property
    def DataType(self): return self._storage.DataType

    def Relayout(self, layout: TensorLayout) -> "Tensor":
        return Tensor(layout, self._storage)

    def Copy(self, order=RowMajor) -> "Tensor":
        """Tensor.copy (Tensor.fs:640-646)."""
        trgt = Tensor.new(self.Shape, self.Dev, self.DataType, order)
        trgt.CopyFrom(self)
        return trgt

    def CopyFrom(self, src: "Tensor"):
        """Tensor.fs:648-661: same device, source broadcast to the target's shape."""
        _same_storage([self, src])
        src = src.broadcastTo(self.Shape)
        self.Backend.Copy(self, src)

    def Transfer(self, dev) -> "Tensor":
        """Tensor.transfer (Tensor.fs:696-711): the target's backend is asked first, then the source's."""
        if self.Dev == dev:
            return self
        trgt = Tensor.new(self.Shape, dev, self.DataType)
        if not trgt.Backend.Transfer(trgt, self):
            if not self.Backend.Transfer(trgt, self):
                raise ValueError(f"Cannot transfer from storage {self.Dev.Id} to storage {dev.Id}.")
        return trgt

    @property
    def T(self) -> "Tensor":
        return self.Relayout(L.transpose(self._layout))

    # ---- element access (Tensor.fs:3750-3790) ----------------------------------------------------------------------------
    def item(self, *idx):
        return self.Backend.GetItem([int(i) for i in idx])

    def setItem(self, idx, value):
        self.Backend.SetItem([int(i) for i in idx], value)

    @property
    def Value(self):
        """Value of a 0-d tensor (Tensor.fs:3761-3777): one element crosses to the host."""
        if self.NDims != 0:
            raise ValueError(f"Value requires a scalar tensor, but the tensor has shape {self.Shape}.")
        return self.Backend.GetItem([])

    @Value.setter
    def Value(self, v):
        if self.NDims != 0:
            raise ValueError(f"Value requires a scalar tensor, but the tensor has shape {self.Shape}.")
        self.Backend.SetItem([], v)

    # ---- creation on a device (Tensor.fs:3653-3780) --------------------------------------------------------------------------
    @staticmethod
    def zeros(shape, dev, dtype) -> "Tensor":
        t = Tensor.new(shape, dev, dtype)
        if not dev.Zeroed:
            t.FillConst(np.dtype(dtype).type(0))
        return t

    @staticmethod
    def filled(shape, value, dev, dtype) -> "Tensor":
        t = Tensor.new(shape, dev, dtype)
        t.FillConst(value)
        return t

    @staticmethod
    def ones(shape, dev, dtype) -> "Tensor":
        return Tensor.filled(shape, np.dtype(dtype).type(1), dev, dtype)

    @staticmethod
    def scalar(value, dev, dtype) -> "Tensor":
        t = Tensor.new([], dev, dtype)
        t.Value = value
        return t

    def scalarLike(self, value) -> "Tensor":
        return Tensor.scalar(value, self.Dev, self.DataType)

    @staticmethod
    def counting(n, dev, dtype=np.int64) -> "Tensor":
        t = Tensor.new([n], dev, dtype)
        t.Backend.FillIncrementing(np.dtype(dtype).type(0), np.dtype(dtype).type(1), t)
        return t

    @staticmethod
    def arange(start, incr, stop, dev, dtype) -> "Tensor":
        """Tensor.fs:3853-3861: max 0 ((stop - start) / incr) elements, the division done in the element type."""
        dt = np.dtype(dtype)
        if dt.kind == "f":
            n = int(dt.type(dt.type(stop) - dt.type(start)) / dt.type(incr))
        else:
            q = abs(int(stop) - int(start)) // abs(int(incr))             # integer division truncates toward zero
            n = q if (int(stop) - int(start)) * int(incr) >= 0 else -q
        t = Tensor.new([max(0, n)], dev, dtype)
        t.Backend.FillIncrementing(dt.type(start), dt.type(incr), t)
        return t

    @staticmethod
    def linspace(start, stop, nElems, dev, dtype) -> "Tensor":
        """Tensor.fs:3879-3886."""
        if nElems < 2:
            raise ValueError("linspace requires at least two elements.")
        dt = np.dtype(dtype)
        incr = dt.type(dt.type(stop) - dt.type(start)) / dt.type(nElems - 1)
        t = Tensor.new([nElems], dev, dtype)
        t.Backend.FillIncrementing(dt.type(start), dt.type(incr), t)
        return t

    @staticmethod
    def identity(size, dev, dtype) -> "Tensor":
        """Tensor.fs:3813-3817: zeros, then ones on the diagonal view."""
        x = Tensor.zeros([size, size], dev, dtype)
        x.diagAxis(0, 1).FillConst(np.dtype(dtype).type(1))
        return x

    def FillConst(self, value):
        self.Backend.FillConst(value, self)

    # ---- shape operations (views; Tensor.fs:330-640) ------------------------------------------------------------------------------
    def broadcastTo(self, shape) -> "Tensor":
        return self.Relayout(L.broadcastToShape(shape, self._layout))

    @staticmethod
    def broadcastToSame(*ts: "Tensor"):
        lays = L.broadcastToSameMany([t.Layout for t in ts])
        return tuple(t.Relayout(l) for t, l in zip(ts, lays))

    def permuteAxes(self, permut) -> "Tensor":
        return self.Relayout(L.permuteAxes(permut, self._layout))

    def swapDim(self, ax1, ax2) -> "Tensor":
        return self.Relayout(L.swapDim(ax1, ax2, self._layout))

    def reverseAxis(self, ax) -> "Tensor":
        return self.Relayout(L.reverseAxis(ax, self._layout))

    def padLeft(self) -> "Tensor":
        return self.Relayout(L.padLeft(self._layout))

    def padRight(self) -> "Tensor":
        return self.Relayout(L.padRight(self._layout))

    def insertAxis(self, ax) -> "Tensor":
        return self.Relayout(L.insertAxis(ax, self._layout))

    def diagAxis(self, ax1, ax2) -> "Tensor":
        return self.Relayout(L.diagAxis(ax1, ax2, self._layout))

    def tryReshapeView(self, shape) -> Optional["Tensor"]:
        lay = L.tryReshape(shape, self._layout)
        return self.Relayout(lay) if lay is not None else None

    def reshape(self, shape) -> "Tensor":
        """View when the layout allows, else a row-major copy is reshaped (ITensor.fs:292-316)."""
        v = self.tryReshapeView(shape)
        if v is not None:
            return v
        return self.Copy().tryReshapeView(shape)

    def flatten(self) -> "Tensor":
        return self.reshape([L.Remainder])

    def __getitem__(self, key) -> "Tensor":
        if not isinstance(key, tuple):
            key = (key,)
        rngs = []
        for k in key:
            if k is Ellipsis:
                rngs.append(Rng.AllFill)
            elif k is None or (isinstance(k, int) and k == NewAxis):
                rngs.append(Rng.NewAxis)
            elif isinstance(k, slice):
                if k.step not in (None, 1):
                    raise ValueError("strided slices are not part of the range grammar")
                last = None if k.stop is None else int(k.stop) - 1
                rngs.append(Rng.Range(k.start, last))
            else:
                rngs.append(Rng.Elem(int(k)))
        if not any(r.kind == "allfill" for r in rngs):
            rngs.append(Rng.AllFill)
        return self.Relayout(L.view(rngs, self._layout))

    def __setitem__(self, key, value):
        """a.[rng] <- value (Tensor.fs:3232-3245): the value is broadcast to the view and copied into it."""
        view = self[key]
        if not isinstance(value, Tensor):
            value = self.scalarLike(value)
        view.CopyFrom(value)

    # ---- diagonals, trace, concatenation (Tensor.fs:4100-4215, 4401-4436) -------------------------------------------------------
    def diag(self) -> "Tensor":
        if self.NDims < 2:
            raise ValueError(f"Need at least a two dimensional array for diagonal but got shape {self.Shape}.")
        return self.diagAxis(self.NDims - 2, self.NDims - 1)

    def diagMatAxis(self, ax1, ax2) -> "Tensor":
        if ax1 == ax2:
            raise ValueError("axes to use for diagonal must be different")
        ax1, ax2 = (ax1, ax2) if ax1 < ax2 else (ax2, ax1)
        if not 0 <= ax1 < self.NDims:
            raise ValueError(f"Axis {ax1} out of range for tensor of shape {self.Shape}.")
        if not 0 <= ax2 <= self.NDims:
            raise ValueError(f"Cannot insert axis at position {ax2} into array of shape {self.Shape}.")
        dShp = list(self.Shape)
        dShp.insert(ax2, self.Shape[ax1])
        d = Tensor.zeros(dShp, self.Dev, self.DataType)
        d.diagAxis(ax1, ax2).CopyFrom(self)
        return d

    def diagMat(self) -> "Tensor":
        if self.NDims < 1:
            raise ValueError("need at leat a one-dimensional array to create a diagonal matrix")
        return self.diagMatAxis(self.NDims - 1, self.NDims)

    def traceAxis(self, ax1, ax2) -> "Tensor":
        tax = ax1 if ax1 < ax2 else ax1 - 1
        return self.diagAxis(ax1, ax2).sumAxis(tax)

    def trace(self) -> "Tensor":
        if self.NDims < 2:
            raise ValueError(f"Need at least a two dimensional array for trace but got shape {self.Shape}.")
        return self.traceAxis(self.NDims - 2, self.NDims - 1)

    @staticmethod
    def concat(ax: int, ts) -> "Tensor":
        ts = list(ts)
        if not ts:
            raise ValueError("Cannot concatenate empty sequence of tensors.")
        shp = ts[0].Shape
        if not 0 <= ax < len(shp):
            raise ValueError(f"Concatenation axis {ax} is out of range for shape {shp}.")
        for i, t in enumerate(ts):
            if t.Shape[:ax] + t.Shape[ax + 1:] != shp[:ax] + shp[ax + 1:]:
                raise ValueError(f"Concatentation element with index {i} with shape {t.Shape} must be equal to shape {shp} "
                                 f"of the first element, except in the concatenation axis {ax}")
        total = sum(t.Shape[ax] for t in ts)
        cc = Tensor.new(shp[:ax] + [total] + shp[ax + 1:], ts[0].Dev, ts[0].DataType)
        pos = 0
        for t in ts:
            n = t.Shape[ax]
            if n > 0:
                key = [slice(None)] * len(shp)
                key[ax] = slice(pos, pos + n)
                cc[tuple(key)] = t
                pos += n
        return cc

    # ---- element-wise: prepare helpers (Tensor.fs:4520-4597) -------------------------------------------------------------------------
    def _prep1(self, dtype=None) -> "Tensor":
        return Tensor.new(self.Shape, self.Dev, dtype or self.DataType)

    @staticmethod
    def _prep2(a: "Tensor", b, dtype=None):
        if not isinstance(b, Tensor):
            b = a.scalarLike(b)
        elif not isinstance(a, Tensor):
            a = b.scalarLike(a)
        _same_storage([a, b])
        a, b = Tensor.broadcastToSame(a, b)
        return Tensor.new(a.Shape, a.Dev, dtype or a.DataType), a, b

    def _srcs(self, *srcs):
        """PrepareElemwiseSources: same device, broadcast to the target's shape."""
        _same_storage([self, *srcs])
        return tuple(s.broadcastTo(self.Shape) for s in srcs)

    def _unary(self, name, dtype=None) -> "Tensor":
        trgt = self._prep1(dtype)
        getattr(trgt.Backend, name)(trgt, self)
        return trgt

    @staticmethod
    def _binary(name, a, b, dtype=None) -> "Tensor":
        trgt, a, b = Tensor._prep2(a, b, dtype)
        getattr(trgt.Backend, name)(trgt, a, b)
        return trgt

    # Fill* variants write into an existing target (Tensor.fs:1342-1344 and siblings), enabling in-place use.
    def _fill1(self, name, a):
        (a,) = self._srcs(a)
        getattr(self.Backend, name)(self, a)

    def _fill2(self, name, a, b):
        a, b = self._srcs(a, b)
        getattr(self.Backend, name)(self, a, b)

    def FillAdd(self, a, b): self._fill2("Add", a, b)
    def FillSubtract(self, a, b): self._fill2("Subtract", a, b)
    def FillMultiply(self, a, b): self._fill2("Multiply", a, b)
    def FillDivide(self, a, b): self._fill2("Divide", a, b)
    def FillUnaryMinus(self, a): self._fill1("UnaryMinus", a)
    def FillTanh(self, a): self._fill1("Tanh", a)
    def FillExp(self, a): self._fill1("Exp", a)

    def __pos__(self): return self._unary("UnaryPlus")
    def __neg__(self): return self._unary("UnaryMinus")
    def __abs__(self): return self._unary("Abs")
    def abs(self): return self._unary("Abs")
    def sgn(self): return self._unary("Sgn")
    def log(self): return self._unary("Log")
    def log10(self): return self._unary("Log10")
    def exp(self): return self._unary("Exp")
    def sin(self): return self._unary("Sin")
    def cos(self): return self._unary("Cos")
    def tan(self): return self._unary("Tan")
    def asin(self): return self._unary("Asin")
    def acos(self): return self._unary("Acos")
    def atan(self): return self._unary("Atan")
    def sinh(self): return self._unary("Sinh")
    def cosh(self): return self._unary("Cosh")
    def tanh(self): return self._unary("Tanh")
    def sqrt(self): return self._unary("Sqrt")
    def ceiling(self): return self._unary("Ceiling")
    def floor(self): return self._unary("Floor")
    def round(self): return self._unary("Round")
    def truncate(self): return self._unary("Truncate")
    def isFinite(self): return self._unary("IsFinite", np.bool_)
    def __invert__(self): return self._unary("Negate")

    def __add__(self, o): return Tensor._binary("Add", self, o)
    def __radd__(self, o): return Tensor._binary("Add", o, self)
    def __sub__(self, o): return Tensor._binary("Subtract", self, o)
    def __rsub__(self, o): return Tensor._binary("Subtract", o, self)
    def __mul__(self, o): return Tensor._binary("Multiply", self, o)
    def __rmul__(self, o): return Tensor._binary("Multiply", o, self)
    def __truediv__(self, o): return Tensor._binary("Divide", self, o)
    def __rtruediv__(self, o): return Tensor._binary("Divide", o, self)
    def __mod__(self, o): return Tensor._binary("Modulo", self, o)
    def __pow__(self, o): return Tensor._binary("Power", self, o)
    def __and__(self, o): return Tensor._binary("And", self, o)
    def __or__(self, o): return Tensor._binary("Or", self, o)
    def __xor__(self, o): return Tensor._binary("Xor", self, o)

    def __eq__(self, o): return Tensor._binary("Equal", self, o, np.bool_)
    def __ne__(self, o): return Tensor._binary("NotEqual", self, o, np.bool_)
    def __lt__(self, o): return Tensor._binary("Less", self, o, np.bool_)
    def __le__(self, o): return Tensor._binary("LessOrEqual", self, o, np.bool_)
    def __gt__(self, o): return Tensor._binary("Greater", self, o, np.bool_)
    def __ge__(self, o): return Tensor._binary("GreaterOrEqual", self, o, np.bool_)
    __hash__ = object.__hash__

    @staticmethod
    def maxElemwise(a, b): return Tensor._binary("MaxElemwise", a, b)
    @staticmethod
    def minElemwise(a, b): return Tensor._binary("MinElemwise", a, b)

    @staticmethod
    def ifThenElse(cond: "Tensor", ifTrue: "Tensor", ifFalse: "Tensor") -> "Tensor":
        """Tensor.fs:2055-2083."""
        _same_storage([cond, ifTrue, ifFalse])
        cond, ifTrue, ifFalse = Tensor.broadcastToSame(cond, ifTrue, ifFalse)
        trgt = Tensor.new(ifTrue.Shape, ifTrue.Dev, ifTrue.DataType)
        trgt.Backend.IfThenElse(trgt, cond, ifTrue, ifFalse)
        return trgt

    def convert(self, dtype) -> "Tensor":
        """Tensor.convert (Tensor.fs:720-731)."""
        trgt = self._prep1(dtype)
        trgt.Backend.Convert(trgt, self)
        return trgt

    # ---- gather / scatter (Tensor.fs:2090-2198) ------------------------------------------------------------------------------------------
    def FillGather(self, indices: List[Optional["Tensor"]], src: "Tensor"):
        _same_storage([src] + [i for i in indices if i is not None])
        if src.NDims != len(indices):
            raise ValueError("For each dimension of src an index tensor must be specified.")
        if any(i is None for i in indices[self.NDims:]):
            raise ValueError("Index dimensions beyond the number of target dimensions must not be None.")
        indices = [i.broadcastTo(self.Shape) if i is not None else None for i in indices]
        self.Backend.Gather(self, indices, src)

    @staticmethod
    def gather(indices: List[Optional["Tensor"]], src: "Tensor") -> "Tensor":
        spec = [i for i in indices if i is not None]
        if not spec:
            raise ValueError("At least one index tensor must not be None.")
        bc = list(Tensor.broadcastToSame(*spec))
        it = iter(bc)
        bcIndices = [next(it) if i is not None else None for i in indices]
        trgt = Tensor.new(bc[0].Shape, src.Dev, src.DataType)
        trgt.FillGather(bcIndices, src)
        return trgt

    def FillScatter(self, indices: List[Optional["Tensor"]], src: "Tensor"):
        _same_storage([src] + [i for i in indices if i is not None])
        if self.NDims != len(indices):
            raise ValueError("For each dimension of the target an index tensor must be specified.")
        if any(i is None for i in indices[src.NDims:]):
            raise ValueError("Index dimensions beyond the number of source dimensions must not be None.")
        indices = [i.broadcastTo(src.Shape) if i is not None else None for i in indices]
        self.Backend.FillConst(self.DataType.type(0), self)
        self.Backend.Scatter(self, indices, src)

    @staticmethod
    def scatter(indices, trgtShp, src: "Tensor") -> "Tensor":
        trgt = Tensor.new(trgtShp, src.Dev, src.DataType)
        trgt.FillScatter(indices, src)
        return trgt

    # ---- reductions (Tensor.fs:2204-2707, helpers :4544-4574) --------------------------------------------------------------------------------
    def _axis_reduce(self, name, ax, dtype=None, value=None) -> "Tensor":
        L.checkAxis(ax, self._layout)
        redShp = self.Shape[:ax] + self.Shape[ax + 1:]
        trgt = Tensor.new(redShp, self.Dev, dtype or self.DataType)
        trgt._fill_axis_reduce(name, ax, self, value)
        return trgt

    def _fill_axis_reduce(self, name, ax, src: "Tensor", value=None):
        """PrepareAxisReduceSources: permute `ax` to the last position as a view (Tensor.fs:4544-4567)."""
        _same_storage([self, src])
        L.checkAxis(ax, src.Layout)
        redShp = src.Shape[:ax] + src.Shape[ax + 1:]
        if self.Shape != redShp:
            raise ValueError(f"Reduction of tensor {src.Shape} along axis {ax} gives shape {redShp} but target has shape {self.Shape}.")
        axisToLast = list(range(ax)) + [src.NDims - 1] + [d - 1 for d in range(ax + 1, src.NDims)]
        src = src.permuteAxes(axisToLast)
        if value is None:
            getattr(self.Backend, name)(self, src)
        else:
            getattr(self.Backend, name)(value, self, src)

    def FillSumAxis(self, ax, src): self._fill_axis_reduce("SumLastAxis", ax, src)

    def sumAxis(self, ax): return self._axis_reduce("SumLastAxis", ax)
    def productAxis(self, ax): return self._axis_reduce("ProductLastAxis", ax)
    def minAxis(self, ax): return self._axis_reduce("MinLastAxis", ax)
    def maxAxis(self, ax): return self._axis_reduce("MaxLastAxis", ax)
    def allAxis(self, ax): return self._axis_reduce("AllLastAxis", ax)
    def anyAxis(self, ax): return self._axis_reduce("AnyLastAxis", ax)
    def countTrueAxis(self, ax): return self._axis_reduce("CountTrueLastAxis", ax, np.int64)
    def argMaxAxis(self, ax): return self._axis_reduce("ArgMaxLastAxis", ax, np.int64)
    def argMinAxis(self, ax): return self._axis_reduce("ArgMinLastAxis", ax, np.int64)
    def findAxis(self, value, ax): return self._axis_reduce("FindLastAxis", ax, np.int64, value=value)

    # whole-tensor forms: flatten |> xAxis 0 (Tensor.fs:2293-2294 and siblings)
    def sumTensor(self): return self.flatten().sumAxis(0)
    def sum(self): return self.sumTensor().Value
    def productTensor(self): return self.flatten().productAxis(0)
    def product(self): return self.productTensor().Value
    def minTensor(self): return self.flatten().minAxis(0)
    def min(self): return self.minTensor().Value
    def maxTensor(self): return self.flatten().maxAxis(0)
    def max(self): return self.maxTensor().Value
    def allTensor(self): return self.flatten().allAxis(0)
    def all(self): return bool(self.allTensor().Value)
    def anyTensor(self): return self.flatten().anyAxis(0)
    def any(self): return bool(self.anyTensor().Value)
    def countTrueTensor(self): return self.flatten().countTrueAxis(0)
    def countTrue(self): return int(self.countTrueTensor().Value)

    def argMax(self) -> List[int]:
        """Tensor.fs:2526-2531: position of the maximum as an index list."""
        if self.NElems == 0:
            raise ValueError("cannot compute argMax of an empty tensor")
        return L.linearToIdx(self._layout, int(self.flatten().argMaxAxis(0).Value))

    def argMin(self) -> List[int]:
        if self.NElems == 0:
            raise ValueError("cannot compute argMin of an empty tensor")
        return L.linearToIdx(self._layout, int(self.flatten().argMinAxis(0).Value))

    def tryFind(self, value) -> Optional[List[int]]:
        """Tensor.fs:2575-2590."""
        pos = int(self.flatten().findAxis(value, 0).Value)
        return None if pos == NotFound else L.linearToIdx(self._layout, pos)

    def trueIdx(self) -> "Tensor":
        """Tensor.fs:2259-2263."""
        nTrue = self.countTrue()
        trgt = Tensor.new([nTrue, self.NDims], self.Dev, np.int64)
        trgt.Backend.TrueIndices(trgt, self)
        return trgt

    # ---- masking (Tensor.fs:3011-3069) ------------------------------------------------------------------------------------------------------------
    @staticmethod
    def _mask_shapes(masks, shape):
        out = []
        shape = list(shape)
        for m in masks:
            if m is None:
                if not shape:
                    raise ValueError("Dimension mismatch between masks and tensor shape.")
                out.append((shape[0], shape[0]))
                shape = shape[1:]
            else:
                if m.NDims > len(shape):
                    raise ValueError("Dimension mismatch between masks and tensor shape.")
                s, shape = shape[:m.NDims], shape[m.NDims:]
                if m.Shape != s:
                    raise ValueError(f"Shape of mask {m.Shape} does not match part {s} of tensor shape it applies to.")
                out.append((m.countTrue(), m.NElems))
        if shape:
            raise ValueError("Dimension mismatch between masks and tensor shape.")
        return out

    def M(self, *masks: Optional["Tensor"]) -> "Tensor":
        """Masked get: collects the elements where the masks are true (None = NoMask for that dimension)."""
        masks = list(masks)
        _same_storage([self] + [m for m in masks if m is not None])
        shapes = Tensor._mask_shapes(masks, self.Shape)
        trgtShp = [t for t, _ in shapes]
        srcShp = [s for _, s in shapes]
        trgt = Tensor.new(trgtShp, self.Dev, self.DataType)
        src = self.reshape(srcShp)
        flat = [m.flatten() if m is not None else None for m in masks]
        self.Backend.MaskedGet(trgt, src, flat)
        return trgt

    def setM(self, masks: List[Optional["Tensor"]], value: "Tensor"):
        """Masked set (Tensor.fs:3054-3069)."""
        masks = list(masks)
        _same_storage([self, value] + [m for m in masks if m is not None])
        shapes = Tensor._mask_shapes(masks, self.Shape)
        valueShp = [t for t, _ in shapes]
        trgtShp = [s for _, s in shapes]
        flat = [m.flatten() if m is not None else None for m in masks]
        value = value.broadcastTo(valueShp)
        view = self.tryReshapeView(trgtShp)
        if view is not None:
            self.Backend.MaskedSet(view, flat, value)
        else:
            trgt = self.reshape(trgtShp)
            self.Backend.MaskedSet(trgt, flat, value)
            self.CopyFrom(trgt.reshape(self.Shape))

    # ---- dot (Tensor.fs:2714-2797) ---------------------------------------------------------------------------------------------------------------------
    def FillDot(self, a: "Tensor", b: "Tensor"):
        _same_storage([self, a, b])
        nt, na, nb = self.NDims, a.NDims, b.NDims
        if (nt, na, nb) == (0, 1, 1) and a.Shape == b.Shape:
            self.Backend.VecVecDot(self, a, b)
        elif (nt, na, nb) == (1, 2, 1) and self.Shape[0] == a.Shape[0] and a.Shape[1] == b.Shape[0]:
            self.Backend.MatVecDot(self, a, b)
        elif (nt, na, nb) == (2, 2, 2) and self.Shape[0] == a.Shape[0] and self.Shape[1] == b.Shape[1] and a.Shape[1] == b.Shape[0]:
            self.Backend.MatMatDot(self, a, b)
        elif na > 2 and nt == na and na == nb and a.Shape[na - 1] == b.Shape[na - 2]:
            a = a.broadcastTo(self.Shape[:na - 2] + a.Shape[na - 2:])
            b = b.broadcastTo(self.Shape[:na - 2] + b.Shape[na - 2:])
            self.Backend.BatchedMatMatDot(self, a, b)
        else:
            raise ValueError(f"Cannot compute dot product between tensors of shapes {a.Shape} and {b.Shape} into tensor of shape {self.Shape}.")

    # ---- inversion (Tensor.fs:2799-2839) ----------------------------------------------------------------------------------
    def FillInvert(self, a: "Tensor"):
        _same_storage([self, a])
        if a.NDims < 2:
            raise ValueError(f"Need at least a matrix to invert but got shape {a.Shape}.")
        a = a.broadcastTo(self.Shape)
        self.Backend.BatchedInvert(self, a)

    @staticmethod
    def invert(a: "Tensor") -> "Tensor":
        trgt = Tensor.new(a.Shape, a.Dev, a.DataType)
        trgt.FillInvert(a)
        return trgt

    # ---- SVD, pseudo-inverse, symmetric eigendecomposition (Tensor.fs:2841-2977) -------------------------------------------------------
    @staticmethod
    def SVDSizes(a: "Tensor"):
        if a.NDims < 2:
            raise ValueError(f"Need at least a matrix to SVD but got shape {a.Shape}.")
        batchShp = list(a.Shape[:a.NDims - 2])
        M, N = a.Shape[a.NDims - 2], a.Shape[a.NDims - 1]
        return batchShp, M, N, min(M, N)

    def FillSVD(self, a: "Tensor", trgtUV=None):
        """Fills this tensor with the (batched) singular values of `a`; trgtUV = (U, V) also receives the transformation matrices."""
        batchShp, M, N, K = Tensor.SVDSizes(a)
        _same_storage([self, a])
        if list(self.Shape) != batchShp + [K]:
            raise ValueError(f"Need a tensor of shape {batchShp + [K]} for SVD singular values but got shape {self.Shape}.")
        if trgtUV is not None:
            trgtU, trgtV = trgtUV
            _same_storage([self, a, trgtU, trgtV])
            if list(trgtU.Shape) != batchShp + [M, M]:
                raise ValueError(f"Need a tensor of shape {batchShp + [M, M]} for SVD left unitary matrices but got shape {trgtU.Shape}.")
            if list(trgtV.Shape) != batchShp + [N, N]:
                raise ValueError(f"Need a tensor of shape {batchShp + [N, N]} for SVD right unitary matrices but got shape {trgtV.Shape}.")
        self.Backend.BatchedSVD(self, trgtUV, a)

    @staticmethod
    def SVD(a: "Tensor"):
        """(U, S, V) with a = U .* diagMat(S) .* V.T, batched over the leading dimensions."""
        batchShp, M, N, K = Tensor.SVDSizes(a)
        U = Tensor.new(batchShp + [M, M], a.Dev, a.DataType, order=ColumnMajor)
        S = Tensor.new(batchShp + [K], a.Dev, a.DataType, order=ColumnMajor)
        V = Tensor.new(batchShp + [N, N], a.Dev, a.DataType, order=RowMajor)
        S.FillSVD(a, trgtUV=(U, V))
        return U, S, V

    @staticmethod
    def SVDWithoutUV(a: "Tensor") -> "Tensor":
        batchShp, M, N, K = Tensor.SVDSizes(a)
        S = Tensor.new(batchShp + [K], a.Dev, a.DataType, order=ColumnMajor)
        S.FillSVD(a)
        return S

    def FillPseudoInvert(self, a: "Tensor", rCond=1e-15):
        """Moore-Penrose pseudo-inverse through the SVD; singular values below rCond count as zero (Tensor.fs:2911-2924)."""
        _same_storage([self, a])
        if a.NDims < 2:
            raise ValueError(f"Need at least a matrix to pseudo invert but got shape {a.Shape}.")
        a = a.broadcastTo(self.Shape)
        u, s, v = Tensor.SVD(a)
        dt = np.dtype(a.DataType).type
        rc, zero, one = s.scalarLike(dt(rCond)), s.scalarLike(dt(0)), s.scalarLike(dt(1))
        sinv = Tensor.ifThenElse(s >= rc, one / s, zero)
        self.FillDot(v, sinv.padRight() * u.T)

    @staticmethod
    def pseudoInvert(a: "Tensor", rCond=1e-15) -> "Tensor":
        trgt = Tensor.new(a.Shape, a.Dev, a.DataType)
        trgt.FillPseudoInvert(a, rCond)
        return trgt

    @staticmethod
    def FillSymmetricEigenDecomposition(part, trgtEigVals: "Tensor", trgtEigVecs: "Tensor", a: "Tensor"):
        _same_storage([trgtEigVals, trgtEigVecs, a])
        if a.NDims != 2 or a.Shape[0] != a.Shape[1]:
            raise ValueError(f"Require a square matrix for symmetric eigen-decomposition but got {a.Shape}.")
        if list(trgtEigVecs.Shape) != list(a.Shape):
            raise ValueError(f"trgtEigVecs and src must have the same shapes but got {trgtEigVecs.Shape} and {a.Shape}.")
        if trgtEigVals.NDims != 1 or trgtEigVals.Shape[0] != a.Shape[0]:
            raise ValueError(f"trgtEigVals must be a vector of length {a.Shape[0]} but it has shape {trgtEigVals.Shape}.")
        trgtEigVals.Backend.SymmetricEigenDecomposition(part, trgtEigVals, trgtEigVecs, a)

    @staticmethod
    def symmetricEigenDecomposition(part, a: "Tensor"):
        """(vals, vecs): ascending eigenvalues, column k of vecs the eigenvector of vals[k]; only the `part` triangle is read."""
        if a.NDims != 2:
            raise ValueError("require a square matrix for symmetric eigen-decomposition")
        trgtEigVals = Tensor.new([a.Shape[0]], a.Dev, a.DataType)
        trgtEigVecs = Tensor.new(a.Shape, a.Dev, a.DataType, order=ColumnMajor)
        Tensor.FillSymmetricEigenDecomposition(part, trgtEigVals, trgtEigVecs, a)
        return trgtEigVals, trgtEigVecs

    def __matmul__(self, b: "Tensor") -> "Tensor":
        a = self
        _same_storage([a, b])
        na, nb = a.NDims, b.NDims
        if na == 1 and nb == 1 and a.Shape == b.Shape:
            trgt = Tensor.new([], a.Dev, a.DataType)
        elif na == 2 and nb == 1 and a.Shape[1] == b.Shape[0]:
            trgt = Tensor.new([a.Shape[0]], a.Dev, a.DataType)
        elif na == 2 and nb == 2 and a.Shape[1] == b.Shape[0]:
            trgt = Tensor.new([a.Shape[0], b.Shape[1]], a.Dev, a.DataType)
        elif na > 2 and na == nb and a.Shape[na - 1] == b.Shape[na - 2]:
            la, lb = L.broadcastToSameInDimsMany(range(na - 2), [a.Layout, b.Layout])
            a, b = a.Relayout(la), b.Relayout(lb)
            trgt = Tensor.new(a.Shape[:na - 2] + [a.Shape[na - 2], b.Shape[na - 1]], a.Dev, a.DataType)
        elif na > 2 and na == nb + 1 and a.Shape[na - 1] == b.Shape[nb - 1]:
            res = a @ b.padRight()
            return res[..., 0]
        else:
            raise ValueError(f"Cannot compute dot product between tensors of shapes {a.Shape} and {b.Shape}.")
        trgt.FillDot(a, b)
        return trgt

    # ---- comparison helpers (Tensor.fs:3901-3925) -----------------------------------------------------------------------------------------------------------
    def isClose(self, b: "Tensor", absTol=1e-8, relTol=1e-5) -> "Tensor":
        """|a-b| <= absTol + relTol*|b| for float types, exact equality otherwise."""
        if np.issubdtype(self.DataType, np.floating):
            diff = abs(self - b)
            return diff <= (abs(b) * self.DataType.type(relTol) + self.DataType.type(absTol))
        return self == b

    def almostEqual(self, b: "Tensor", absTol=1e-8, relTol=1e-5) -> bool:
        if self.Shape != b.Shape:
            return False
        return self.isClose(b, absTol, relTol).all()

    def __repr__(self):
        return f"Tensor<{self.DataType}>(shape={self.Shape}, dev={self.Dev.Id})"
