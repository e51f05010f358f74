"""TensorLayout — shape / offset / stride algebra, device-free.

Host-side mirror of the reference's layout record and module (Tensor/Tensor/TensorLayout.fs): same names, same argument
meaning, same failure cases (InvalidOperationException -> ValueError, IndexOutOfRangeException -> IndexError).
Offsets and strides are in elements and may be zero (broadcast) or negative (reverseAxis).
"""
from __future__ import annotations

from dataclasses import dataclass, replace
from typing import List, Optional, Sequence, Tuple

# SpecialIdx (Tensor/Tensor/TensorRng.fs:9-24)
NewAxis = -(2 ** 63) + 1
Fill = -(2 ** 63) + 2
Remainder = -(2 ** 63) + 3
NotFound = -(2 ** 63) + 4


def _prod(xs) -> int:
    n = 1
    for x in xs:
        n *= int(x)
    return n


@dataclass(frozen=True)
class TensorLayout:
    """TensorLayout.fs:12-24."""
    Shape: Tuple[int, ...]
    Offset: int
    Stride: Tuple[int, ...]

    def __post_init__(self):
        object.__setattr__(self, "Shape", tuple(int(s) for s in self.Shape))
        object.__setattr__(self, "Stride", tuple(int(s) for s in self.Stride))
        object.__setattr__(self, "Offset", int(self.Offset))
        if len(self.Shape) != len(self.Stride):
            raise ValueError(f"shape {self.Shape} and stride {self.Stride} must have same number of entries")
        if any(s < 0 for s in self.Shape):
            raise ValueError(f"shape {self.Shape} cannot have negative entries")

    @property
    def NDims(self) -> int:
        return len(self.Shape)

    @property
    def NElems(self) -> int:
        return _prod(self.Shape)


# ---- construction (TensorLayout.fs:96-125) -----------------------------------------------------------------------------

def orderedStride(shape: Sequence[int], order: Sequence[int]) -> Tuple[int, ...]:
    """Strides so that dimension order[0] is the fastest varying (TensorLayout.fs:96-106)."""
    if sorted(order) != list(range(len(order))):
        raise ValueError(f"the stride order {list(order)} is not a permutation")
    if len(order) != len(shape):
        raise ValueError(f"the stride order {list(order)} is incompatible with the shape {list(shape)}")
    stride = [0] * len(shape)
    cum = 1
    for o in order:
        stride[o] = cum
        cum *= int(shape[o])
    return tuple(stride)


def cStride(shape: Sequence[int]) -> Tuple[int, ...]:
    return orderedStride(shape, list(reversed(range(len(shape)))))


def fStride(shape: Sequence[int]) -> Tuple[int, ...]:
    return orderedStride(shape, list(range(len(shape))))


def newC(shape: Sequence[int]) -> TensorLayout:
    return TensorLayout(tuple(shape), 0, cStride(shape))


def newF(shape: Sequence[int]) -> TensorLayout:
    return TensorLayout(tuple(shape), 0, fStride(shape))


def newOrdered(shape: Sequence[int], order: Sequence[int]) -> TensorLayout:
    return TensorLayout(tuple(shape), 0, orderedStride(shape, order))


# ---- predicates (TensorLayout.fs:127-147) ----------------------------------------------------------------------------------

def stridesEqual(shape, a, b) -> bool:
    return all(x == y for s, x, y in zip(shape, a, b) if s > 1)


def isC(a: TensorLayout) -> bool:
    return stridesEqual(a.Shape, a.Stride, cStride(a.Shape))


def isF(a: TensorLayout) -> bool:
    return stridesEqual(a.Shape, a.Stride, fStride(a.Shape))


def hasContiguousMemory(a: TensorLayout) -> bool:
    return isC(a) or isF(a)


def isBroadcasted(a: TensorLayout) -> bool:
    return any(st == 0 and sh > 1 for sh, st in zip(a.Shape, a.Stride))


def checkAxis(ax: int, a: TensorLayout) -> None:
    if not (0 <= ax < a.NDims):
        raise IndexError(f"axis {ax} out of range for tensor with shape {list(a.Shape)}")


def addr(idx: Sequence[int], a: TensorLayout) -> int:
    """Checked element address (TensorLayout.fs:32-42)."""
    if len(idx) != a.NDims:
        raise IndexError(f"index {list(idx)} has other dimensionality than tensor of shape {list(a.Shape)}")
    if not all(0 <= i < s for i, s in zip(idx, a.Shape)):
        raise IndexError(f"index {list(idx)} out of range for tensor of shape {list(a.Shape)}")
    return a.Offset + sum(int(i) * st for i, st in zip(idx, a.Stride))


# ---- padding / broadcasting (TensorLayout.fs:149-271) ----------------------------------------------------------------------

def padLeft(a: TensorLayout) -> TensorLayout:
    return TensorLayout((1,) + a.Shape, a.Offset, (0,) + a.Stride)


def padRight(a: TensorLayout) -> TensorLayout:
    return TensorLayout(a.Shape + (1,), a.Offset, a.Stride + (0,))


def insertAxis(ax: int, a: TensorLayout) -> TensorLayout:
    if not (0 <= ax <= a.NDims):
        raise IndexError(f"axis {ax} out of range for tensor with shape {list(a.Shape)}")
    return TensorLayout(a.Shape[:ax] + (1,) + a.Shape[ax:], a.Offset, a.Stride[:ax] + (0,) + a.Stride[ax:])


def cutLeft(a: TensorLayout) -> TensorLayout:
    if a.NDims == 0:
        raise ValueError("cannot remove dimensions from scalar")
    return TensorLayout(a.Shape[1:], a.Offset, a.Stride[1:])


def cutRight(a: TensorLayout) -> TensorLayout:
    if a.NDims == 0:
        raise ValueError("cannot remove dimensions from scalar")
    return TensorLayout(a.Shape[:-1], a.Offset, a.Stride[:-1])


def broadcastDim(dim: int, size: int, a: TensorLayout) -> TensorLayout:
    if size < 0:
        raise ValueError("size must be positive")
    if a.Shape[dim] != 1:
        raise ValueError(f"Dimension {dim} of shape {list(a.Shape)} must be of size 1 to broadcast.")
    shp, st = list(a.Shape), list(a.Stride)
    shp[dim], st[dim] = size, 0
    return TensorLayout(tuple(shp), a.Offset, tuple(st))


def padToSame(a: TensorLayout, b: TensorLayout):
    while a.NDims < b.NDims:
        a = padLeft(a)
    while b.NDims < a.NDims:
        b = padLeft(b)
    return a, b


def padToSameMany(sas: List[TensorLayout]) -> List[TensorLayout]:
    need = max(sa.NDims for sa in sas)
    out = []
    for sa in sas:
        while sa.NDims < need:
            sa = padLeft(sa)
        out.append(sa)
    return out


def broadcastToSameInDimsMany(dims: Sequence[int], sas: List[TensorLayout]) -> List[TensorLayout]:
    sas = list(sas)
    for d in dims:
        if not all(d < sa.NDims for sa in sas):
            raise ValueError(f"Cannot broadcast shapes {[list(s.Shape) for s in sas]} to same size in non-existant dimension {d}.")
        ls = [sa.Shape[d] for sa in sas]
        if 1 in ls:
            nonbc = {l for l in ls if l != 1}
            if len(nonbc) == 1:
                target = next(iter(nonbc))
                sas = [broadcastDim(d, target, sa) if sa.Shape[d] != target else sa for sa in sas]
            elif len(nonbc) > 1:
                raise ValueError(f"Cannot broadcast shapes {[list(s.Shape) for s in sas]} to same size in dimension {d} "
                                 "because they do not agree in the target size.")
        elif len(set(ls)) > 1:
            raise ValueError(f"Non-broadcast dimension {d} of shapes {[list(s.Shape) for s in sas]} does not agree.")
    return sas


def broadcastToSameMany(sas: List[TensorLayout]) -> List[TensorLayout]:
    if not sas:
        return []
    sas = padToSameMany(sas)
    try:
        return broadcastToSameInDimsMany(range(sas[0].NDims), sas)
    except ValueError:
        raise ValueError(f"Cannot broadcast shapes {[list(s.Shape) for s in sas]} to same size.")


def broadcastToSame(a: TensorLayout, b: TensorLayout):
    r = broadcastToSameMany([a, b])
    return r[0], r[1]


def broadcastToShape(bs: Sequence[int], ain: TensorLayout) -> TensorLayout:
    bs = tuple(int(b) for b in bs)
    if len(bs) < ain.NDims:
        raise ValueError(f"Cannot broadcast to shape {list(bs)} from shape {list(ain.Shape)} of higher rank.")
    a = ain
    while a.NDims < len(bs):
        a = padLeft(a)
    for d in range(len(bs)):
        al, bl = a.Shape[d], bs[d]
        if al == bl:
            continue
        if al == 1:
            a = broadcastDim(d, bl, a)
        else:
            raise ValueError(f"Cannot broadcast shape {list(ain.Shape)} to shape {list(bs)}.")
    return a


# ---- reshape (TensorLayout.fs:282-342) -----------------------------------------------------------------------------------------

def tryReshape(shp: Sequence[int], a: TensorLayout) -> Optional[TensorLayout]:
    shp = [int(s) for s in shp]
    nrem = sum(1 for s in shp if s == Remainder)
    if nrem == 1:
        sofar = _prod(s for s in shp if s != Remainder)
        need = a.NElems
        if sofar == 0 or need % sofar != 0:
            raise ValueError(f"cannot reshape from {list(a.Shape)} to {shp} because {need} / {sofar} is not an integer")
        shp = [need // sofar if s == Remainder else s for s in shp]
    elif nrem > 1:
        raise ValueError(f"only the size of one dimension can be determined automatically, but shape was {shp}")
    if _prod(shp) != a.NElems:
        raise ValueError(f"cannot reshape from shape {list(a.Shape)} (with {a.NElems} elements) to shape {shp} (with {_prod(shp)} elements)")

    def tf(newStr, newShp, aStr, aShp):
        # singleton insertions and removals only (TensorLayout.fs:308-319)
        while True:
            if newShp and aStr and aShp and newShp[0] == aShp[0]:
                newStr = newStr + [aStr[0]]
                newShp, aStr, aShp = newShp[1:], aStr[1:], aShp[1:]
            elif newShp and newShp[0] == 1:
                newStr = newStr + [0]
                newShp = newShp[1:]
            elif aStr and aShp and aShp[0] == 1:
                aStr, aShp = aStr[1:], aShp[1:]
            elif not newShp and not aStr and not aShp:
                return newStr
            else:
                return None

    if isC(a):
        return TensorLayout(tuple(shp), a.Offset, cStride(shp))
    ns = tf([], list(shp), list(a.Stride), list(a.Shape))
    if ns is not None:
        return TensorLayout(tuple(shp), a.Offset, tuple(ns))
    return None


def canReshape(shp, a) -> bool:
    return tryReshape(shp, a) is not None


def reshape(shp, a) -> TensorLayout:
    r = tryReshape(shp, a)
    if r is None:
        raise ValueError(f"Cannot reshape layout {a} into shape {list(shp)} without copying.")
    return r


# ---- axis manipulation (TensorLayout.fs:344-371) ----------------------------------------------------------------------------------

def swapDim(ax1: int, ax2: int, a: TensorLayout) -> TensorLayout:
    if not (0 <= ax1 < a.NDims and 0 <= ax2 < a.NDims):
        raise ValueError(f"Cannot swap dimension {ax1} with {ax2} of for shape {list(a.Shape)}.")
    shp, st = list(a.Shape), list(a.Stride)
    shp[ax1], shp[ax2] = shp[ax2], shp[ax1]
    st[ax1], st[ax2] = st[ax2], st[ax1]
    return TensorLayout(tuple(shp), a.Offset, tuple(st))


def transpose(a: TensorLayout) -> TensorLayout:
    if a.NDims < 2:
        raise ValueError(f"cannot transpose non-matrix of shape {list(a.Shape)}")
    return swapDim(a.NDims - 2, a.NDims - 1, a)


def permuteAxes(permut: Sequence[int], a: TensorLayout) -> TensorLayout:
    """permut[i] is the DESTINATION of axis i (F# List.permute; TensorLayout.fs:358-365)."""
    if a.NDims != len(permut):
        raise ValueError(f"Permutation {list(permut)} must have same rank as shape {list(a.Shape)}.")
    if sorted(permut) != list(range(a.NDims)):
        raise ValueError(f"{list(permut)} is not a permutation")
    shp, st = [0] * a.NDims, [0] * a.NDims
    for i, p in enumerate(permut):
        shp[p], st[p] = a.Shape[i], a.Stride[i]
    return TensorLayout(tuple(shp), a.Offset, tuple(st))


def reverseAxis(ax: int, a: TensorLayout) -> TensorLayout:
    checkAxis(ax, a)
    st = list(a.Stride)
    st[ax] = -st[ax]
    return TensorLayout(a.Shape, a.Offset + (a.Shape[ax] - 1) * a.Stride[ax], tuple(st))


def diagAxis(ax1: int, ax2: int, a: TensorLayout) -> TensorLayout:
    checkAxis(ax1, a)
    checkAxis(ax2, a)
    if ax1 == ax2:
        raise ValueError("Axes to use for diagonal must be different.")
    if a.Shape[ax1] != a.Shape[ax2]:
        raise ValueError(f"Array must have same dimensions along axis {ax1} and {ax2} to extract diagonal but it has shape {list(a.Shape)}.")
    shp, st = [], []
    for ax, (sh, s) in enumerate(zip(a.Shape, a.Stride)):
        if ax == ax1:
            shp.append(sh)
            st.append(a.Stride[ax1] + a.Stride[ax2])
        elif ax == ax2:
            continue
        else:
            shp.append(sh)
            st.append(s)
    return TensorLayout(tuple(shp), a.Offset, tuple(st))


# ---- slicing (TensorLayout.fs:374-422) ------------------------------------------------------------------------------------------

class Rng:
    """Range over one dimension (Tensor/Tensor/TensorRng.fs:29-60): Elem i | Rng(first,last inclusive) | NewAxis | AllFill."""
    __slots__ = ("kind", "a", "b")

    def __init__(self, kind, a=None, b=None):
        self.kind, self.a, self.b = kind, a, b

    @staticmethod
    def Elem(i):
        return Rng("elem", int(i))

    @staticmethod
    def Range(first=None, last=None):
        return Rng("rng", first, last)

    All = None  # set below
    NewAxis = None
    AllFill = None

    def __repr__(self):
        return f"Rng({self.kind},{self.a},{self.b})"


Rng.All = Rng("rng", None, None)
Rng.NewAxis = Rng("newaxis")
Rng.AllFill = Rng("allfill")


def view(ranges: Sequence[Rng], a: TensorLayout) -> TensorLayout:
    """Sub-view by per-dimension ranges; `last` is inclusive (TensorLayout.fs:374-422)."""
    ranges = list(ranges)

    def fail():
        raise IndexError(f"Slice {ranges} is incompatible with shape {list(a.Shape)}.")

    def rec(rs, shp, st, off):
        if rs and rs[0].kind == "allfill":
            rest = rs[1:]
            if shp and len(shp) - 1 > len(rest):
                return rec([Rng.All, Rng.AllFill] + rest, shp, st, off)
            if shp and len(shp) - 1 == len(rest):
                return rec([Rng.All] + rest, shp, st, off)
            return rec(rest, shp, st, off)
        if rs and rs[0].kind in ("elem", "rng"):
            if not shp:
                fail()
            r, n, s = rs[0], shp[0], st[0]
            sub_shape, sub_stride, sub_off = rec(rs[1:], shp[1:], st[1:], off)
            if r.kind == "elem":
                if not (0 <= r.a < n):
                    raise IndexError(f"Index {r.a} out of range in slice {ranges} for shape {list(a.Shape)}.")
                return sub_shape, sub_stride, sub_off + r.a * s
            start = 0 if r.a is None else int(r.a)
            stop = n - 1 if r.b is None else int(r.b)
            if stop >= start:
                if not (0 <= start < n) or not (0 <= stop < n + 1):
                    raise IndexError(f"Index out of range in slice {ranges} for shape {list(a.Shape)}.")
                return [stop + 1 - start] + sub_shape, [s] + sub_stride, sub_off + start * s
            return [0] + sub_shape, [s] + sub_stride, sub_off
        if rs and rs[0].kind == "newaxis":
            sub_shape, sub_stride, sub_off = rec(rs[1:], shp, st, off)
            return [1] + sub_shape, [0] + sub_stride, sub_off
        if not rs and not shp:
            return [], [], off
        fail()

    shp, st, off = rec(ranges, list(a.Shape), list(a.Stride), a.Offset)
    return TensorLayout(tuple(shp), off, tuple(st))


def idxToLinear(a: TensorLayout, idx: Sequence[int]) -> int:
    if len(idx) != a.NDims or not all(0 <= i < s for i, s in zip(idx, a.Shape)):
        raise IndexError(f"index {list(idx)} out of range for tensor of shape {list(a.Shape)}")
    return sum(i * s for i, s in zip(idx, cStride(a.Shape)))


def linearToIdx(a: TensorLayout, linear: int) -> List[int]:
    idx = []
    for s in cStride(a.Shape):
        idx.append(linear // s)
        linear %= s
    if not all(0 <= i < sh for i, sh in zip(idx, a.Shape)):
        raise IndexError(f"linear index out of range for tensor of shape {list(a.Shape)}")
    return idx
