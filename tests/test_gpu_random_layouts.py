"""Differential test over seeded random shapes and views: the same frontend call sequence on the oracle device and on the GPU,
integer element types so every comparison is bit-exact.  Views are built from permutations, slices, reversed axes, inserted and
broadcast axes; extents include 1 and ragged sizes around the vector widths and tile edges of the kernels."""
import os

import numpy as np
import pytest

from deepnet_amd.tensor import Tensor
from util import assert_exact

pytestmark = pytest.mark.gpu

MORE = int(os.environ.get("DNH_FUZZ_SEEDS_FACTOR", "1"))   # more seeds for an occasional longer run

EXTENTS = [1, 2, 3, 4, 5, 7, 8, 15, 16, 17, 31, 33, 63, 64, 65, 127, 130, 257]


def random_view(rng, t):
    """A random view of tensor t (same on both devices because only layout operations are applied)."""
    nd = t.NDims
    if nd >= 2 and rng.random() < 0.6:
        perm = list(rng.permutation(nd))
        t = t.permuteAxes([int(p) for p in perm])
    for ax in range(t.NDims):
        r = rng.random()
        n = t.Shape[ax]
        if r < 0.25 and n > 2:
            lo = int(rng.integers(0, n // 2))
            hi = int(rng.integers(lo + 1, n + 1))
            key = [slice(None)] * t.NDims
            key[ax] = slice(lo, hi)
            t = t[tuple(key)]
        elif r < 0.4 and n > 1:
            t = t.reverseAxis(ax)
    return t


def make_operands(rng, H, G, dtype, max_elems=200_000):
    nd = int(rng.integers(0, 5))
    shape = []
    total = 1
    for _ in range(nd):
        e = int(rng.choice(EXTENTS))
        if total * e > max_elems:
            e = 1
        shape.append(e)
        total *= e
    info = np.iinfo(dtype) if np.dtype(dtype).kind in "iu" else None
    lo, hi = (max(info.min, -1000), min(info.max, 1000)) if info else (0, 1)
    a = rng.integers(lo, hi + 1, size=shape).astype(dtype) if info else (rng.random(shape) < 0.5)
    return a


@pytest.mark.parametrize("seed", range(40 * MORE))
def test_random_views_elementwise_and_folds(H, G, seed):
    rng = np.random.default_rng(1000 + seed)
    for case in range(25):
        dtype = [np.int32, np.int64, np.uint8, np.int8, np.int16, np.uint16][int(rng.integers(0, 6))]
        a_np = make_operands(rng, H, G, dtype)
        b_np = rng.integers(-50, 50, size=a_np.shape).astype(dtype) if dtype not in (np.uint8, np.uint16) else rng.integers(0, 100, size=a_np.shape).astype(dtype)
        state = rng.bit_generator.state
        outs = []
        for M in (H, G):
            rng.bit_generator.state = state                      # identical random choices on both devices
            a = random_view(rng, M.ofNumpy(a_np))
            # b: same shape as the view of a, possibly with broadcast axes
            b_full = M.ofNumpy(b_np)
            b = b_full
            # bring b to a's view shape by replaying a compatible construction: copy a's view of b_np's layout
            b = b.Relayout(type(a.Layout)(a.Layout.Shape, a.Layout.Offset, a.Layout.Stride)) if b_np.shape == a_np.shape else b
            r = []
            r.append(M.toNumpy(a + b))
            r.append(M.toNumpy(a * b - a))
            r.append(M.toNumpy(a > b))
            r.append(M.toNumpy(Tensor.ifThenElse(a > b, a, b)))
            r.append(M.toNumpy(a.Copy()))
            r.append(M.toNumpy(Tensor.maxElemwise(a, b)))
            if a.NDims >= 1:
                ax = int(rng.integers(0, a.NDims))
                r.append(M.toNumpy(a.sumAxis(ax)))
                r.append(M.toNumpy(a.maxAxis(ax)))
                r.append(M.toNumpy(a.argMaxAxis(ax)))
                r.append(M.toNumpy(a.argMinAxis(ax)))
                r.append(M.toNumpy((a > b).countTrueAxis(ax)))
                r.append(M.toNumpy(a.findAxis(dtype(3), ax)))
                if a.Shape[ax] > 1 and rng.random() < 0.5:         # broadcast operand along one axis
                    col = a.sumAxis(ax).insertAxis(ax)
                    r.append(M.toNumpy(a - col))
            if a.NElems > 0:
                r.append(M.toNumpy(a.convert(np.int64)))
                m = a > b
                r.append(M.toNumpy(a.flatten().M(m.flatten())))
                r.append(M.toNumpy(m.trueIdx()))
            outs.append(r)
        assert len(outs[0]) == len(outs[1])
        for k, (ref, got) in enumerate(zip(*outs)):
            try:
                assert_exact(ref, got)
            except AssertionError as e:
                raise AssertionError(f"seed {seed} case {case} result {k} dtype {np.dtype(dtype)} shape {a_np.shape}: {e}") from None


@pytest.mark.parametrize("seed", range(12 * MORE))
def test_random_gather_scatter(H, G, seed):
    rng = np.random.default_rng(2000 + seed)
    for case in range(15):
        nd = int(rng.integers(1, 4))
        shape = [int(rng.choice([1, 3, 8, 17, 64, 100])) for _ in range(nd)]
        # integers, and floats spread over many decades: scatter adds repeated indices in source order on both devices, so the
        # floating-point sums agree bit for bit as well
        dtype = [np.int32, np.float32, np.float64][int(rng.integers(0, 3))]
        if dtype == np.int32:
            src_np = rng.integers(-1000, 1000, size=shape).astype(np.int32)
        else:
            src_np = (rng.standard_normal(shape) * 10.0 ** rng.uniform(-6, 6, shape)).astype(dtype)
        ishape = [int(rng.choice([1, 5, 33, 200])) for _ in range(int(rng.integers(1, 3)))]
        use = [bool(rng.random() < 0.7) for _ in range(nd)]
        if not any(use):
            use[0] = True
        # unspecified dimensions take the target position, so the index shape must cover them: pad the index shape to rank nd
        full_ishape = ([1] * (nd - len(ishape)) + ishape)[-nd:] if len(ishape) <= nd else ishape[-nd:]
        for d in range(nd):
            if not use[d]:
                full_ishape[d] = min(full_ishape[d], shape[d]) if full_ishape[d] > shape[d] else full_ishape[d]
                full_ishape[d] = shape[d] if full_ishape[d] > shape[d] else full_ishape[d]
        idx_np = [rng.integers(0, shape[d], size=full_ishape).astype(np.int64) if use[d] else None for d in range(nd)]
        outs = []
        for M in (H, G):
            src = M.ofNumpy(src_np)
            idx = [M.ofNumpy(i) if i is not None else None for i in idx_np]
            g = Tensor.gather(idx, src)
            s = Tensor.scatter(idx, shape, g)
            outs.append([M.toNumpy(g), M.toNumpy(s)])
        for ref, got in zip(*outs):
            assert_exact(ref, got)


@pytest.mark.parametrize("seed", range(16 * MORE))
def test_random_views_float(H, G, seed):
    """fp32 / fp64: exactly rounded operations, comparisons, max/min and arg folds are bit-exact; sums within (n + 64) u S."""
    rng = np.random.default_rng(3000 + seed)
    for case in range(20):
        dtype = [np.float32, np.float64][int(rng.integers(0, 2))]
        shape = list(make_operands(rng, H, G, np.int32).shape)
        a_np = rng.standard_normal(shape).astype(dtype)
        b_np = (rng.standard_normal(shape) + 3.0).astype(dtype)
        if rng.random() < 0.3 and a_np.size:                       # planted ties and infinities
            a_np.flat[rng.integers(0, a_np.size, size=max(1, a_np.size // 7))] = dtype(1.5)
            a_np.flat[rng.integers(0, a_np.size)] = -np.inf
        state = rng.bit_generator.state
        outs, sums = [], []
        for M in (H, G):
            rng.bit_generator.state = state
            a = random_view(rng, M.ofNumpy(a_np))
            b = M.ofNumpy(b_np).Relayout(type(a.Layout)(a.Layout.Shape, a.Layout.Offset, a.Layout.Stride))
            r = [M.toNumpy(a + b), M.toNumpy(a * b), M.toNumpy(a / b), M.toNumpy(a - b), M.toNumpy(a > b), M.toNumpy(a.abs().sqrt()),
                 M.toNumpy(Tensor.minElemwise(a, b)), M.toNumpy(Tensor.ifThenElse(a < b, a, b)), M.toNumpy(-a), M.toNumpy(a.floor()),
                 M.toNumpy(a.round()), M.toNumpy(a.sgn()), M.toNumpy(a.isFinite())]
            s = []
            if a.NDims >= 1:
                ax = int(rng.integers(0, a.NDims))
                r += [M.toNumpy(a.maxAxis(ax)), M.toNumpy(a.minAxis(ax)), M.toNumpy(a.argMaxAxis(ax)), M.toNumpy(a.argMinAxis(ax))]
                s = [M.toNumpy(b.sumAxis(ax)), M.toNumpy(b.abs().sumAxis(ax)), b.Shape[ax]]      # b holds no infinities
            outs.append(r)
            sums.append(s)
        for k, (ref, got) in enumerate(zip(*outs)):
            try:
                assert_exact(ref, got)
            except AssertionError as e:
                raise AssertionError(f"seed {seed} case {case} result {k} dtype {np.dtype(dtype)} shape {a_np.shape}: {e}") from None
        if sums[0]:
            ref, got, S, n = sums[0][0], sums[1][0], sums[0][1], sums[0][2]
            u = 2.0 ** -24 if dtype == np.float32 else 2.0 ** -53
            assert np.all(np.abs(ref.astype(np.float64) - got.astype(np.float64)) <= (n + 64) * u * S.astype(np.float64))
