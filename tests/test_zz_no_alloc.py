"""GPU: dnh_reduce_last_axis_noalloc — the fold entry point that allocates nothing — against dnh_reduce_last_axis.

Both run the same kernels with the same splits, so every result, float sums included, must agree bit for bit.  Each case calls the
entry point twice in a row, the second time on a smaller input: the static scratch array keeps the first call's partial results,
and the second call must not be affected by them.  Called through the C ABI with ctypes.
"""
import ctypes as C

import numpy as np
import pytest

from deepnet_amd import abi, native

pytestmark = pytest.mark.gpu


def _fold(G, name, op, src, axis, out_dtype):
    """Folds device tensor `src` along `axis` through entry point `name`; returns the result as NumPy."""
    lib = native.load()
    # reduced axis last, as the frontend does it (a view, no copy)
    order = [d for d in range(src.NDims) if d != axis] + [axis]
    lay = src.Layout
    shape = [lay.Shape[d] for d in order]
    stride = [lay.Stride[d] for d in order]
    trgt = G.zeros(shape[:-1], out_dtype)
    sd = abi.make_descriptor(src.Storage.Pointer(), src.DataType, shape, stride, lay.Offset)
    td = trgt.Backend._desc(trgt)
    native.check(getattr(lib, name)(op, C.byref(td), C.byref(sd), G.Cfg.Stream))
    return G.toNumpy(trgt)


CASES = [
    # (dtype, op, out dtype, first shape, second (smaller) shape, axis)
    (np.float32, abi.DNH_SUM, np.float32, (2048, 4096), (700, 1000), 0),      # columns, split into partials
    (np.float32, abi.DNH_MAX, np.float32, (2048, 4096), (300, 520), 0),
    (np.float64, abi.DNH_SUM, np.float64, (1536, 2048), (512, 640), 0),
    (np.float32, abi.DNH_SUM, np.float32, (4, 1 << 20), (3, 300000), 1),      # few long rows, split into partials
    (np.int32, abi.DNH_PRODUCT, np.int32, (1 << 22,), (1 << 18,), 0),        # full fold of a vector
    (np.bool_, abi.DNH_COUNT_TRUE, np.int64, (1 << 24,), (123457,), 0),
    (np.bool_, abi.DNH_ALL, np.bool_, (1024, 1024), (100, 100), 0),
    (np.float32, abi.DNH_MIN, np.float32, (512, 512), (64, 64), 1),           # no partials at all
]


def _data(rng, dtype, shape):
    if dtype == np.bool_:
        return rng.random(shape) < 0.5
    if np.dtype(dtype).kind == "f":
        return rng.standard_normal(shape).astype(dtype)
    return rng.integers(-3, 4, shape).astype(dtype)


@pytest.mark.parametrize("dtype,op,out_dtype,shape1,shape2,axis", CASES)
def test_noalloc_fold_matches_the_allocating_entry_point_twice_in_a_row(G, rng, dtype, op, out_dtype, shape1, shape2, axis):
    a1, a2 = _data(rng, dtype, shape1), _data(rng, dtype, shape2)
    d1, d2 = G.ofNumpy(a1), G.ofNumpy(a2)
    want1 = _fold(G, "dnh_reduce_last_axis", op, d1, axis, out_dtype)
    want2 = _fold(G, "dnh_reduce_last_axis", op, d2, axis, out_dtype)
    got1 = _fold(G, "dnh_reduce_last_axis_noalloc", op, d1, axis, out_dtype)
    got2 = _fold(G, "dnh_reduce_last_axis_noalloc", op, d2, axis, out_dtype)
    for want, got in ((want1, got1), (want2, got2)):
        assert want.dtype == got.dtype and want.shape == got.shape
        assert want.tobytes() == got.tobytes()
    # and the values are the fold's, not merely equal to each other
    if op == abi.DNH_COUNT_TRUE:
        assert int(got1) == int(np.count_nonzero(a1)) and int(got2) == int(np.count_nonzero(a2))
    if op == abi.DNH_MAX:
        assert np.array_equal(got2, a2.max(axis=axis))


def _free_device_bytes():
    """hipMemGetInfo through the HIP runtime the library has already loaded into this process."""
    hip = C.CDLL("libamdhip64.so")
    free, total = C.c_size_t(), C.c_size_t()
    assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


def test_noalloc_fold_does_not_touch_the_allocator(G, rng):
    """A two-pass fold on a stream that has no workspace yet: the allocating entry point must ask the driver for one there (its
    partials live in the stream's workspace, which comes straight from hipMalloc and never shows in the block cache's counters),
    the entry point that may not allocate must leave the device's free memory and the block cache exactly as they were."""
    lib = native.load()
    a = G.ofNumpy(rng.standard_normal((2048, 2048)).astype(np.float32))
    _fold(G, "dnh_reduce_last_axis_noalloc", abi.DNH_SUM, a, 0, np.float32)   # first call on the device: looks the array up
    trgt = G.zeros((2048,), np.float32)
    want = _fold(G, "dnh_reduce_last_axis", abi.DNH_SUM, a, 0, np.float32)
    lay = a.Layout
    sd = abi.make_descriptor(a.Storage.Pointer(), a.DataType, [2048, 2048], [lay.Stride[1], lay.Stride[0]], lay.Offset)
    td = trgt.Backend._desc(trgt)
    native.check(lib.dnh_device_sync())
    fresh, control = C.c_void_p(), C.c_void_p()
    native.check(lib.dnh_stream_create(C.byref(fresh)))
    native.check(lib.dnh_stream_create(C.byref(control)))
    try:
        before, after = abi.DnhPoolStats(), abi.DnhPoolStats()
        native.check(lib.dnh_pool_stats(C.byref(before)))
        free0 = _free_device_bytes()
        native.check(lib.dnh_reduce_last_axis_noalloc(abi.DNH_SUM, C.byref(td), C.byref(sd), fresh))
        native.check(lib.dnh_stream_sync(fresh))
        free1 = _free_device_bytes()
        native.check(lib.dnh_pool_stats(C.byref(after)))
        assert free1 == free0, f"the no-alloc fold changed the device's free memory by {free0 - free1} bytes"
        assert (before.hits, before.misses, before.live_bytes, before.cached_bytes) == (after.hits, after.misses, after.live_bytes, after.cached_bytes)
        assert np.array_equal(G.toNumpy(trgt), want)
        # CountTrue of a whole mask: the allocating entry point takes a one-launch form whose arrival words the library allocates on a
        # stream's first use; the entry point that may not allocate must keep the fold that needs only the static array
        mask = rng.random(1 << 22) < 0.5
        tm = G.ofNumpy(mask)
        cnt = G.zeros([], np.int64)
        md, cd = tm.Backend._desc(tm), cnt.Backend._desc(cnt)
        native.check(lib.dnh_device_sync())
        free_c = _free_device_bytes()
        native.check(lib.dnh_reduce_last_axis_noalloc(abi.DNH_COUNT_TRUE, C.byref(cd), C.byref(md), fresh))
        native.check(lib.dnh_stream_sync(fresh))
        assert _free_device_bytes() == free_c
        assert int(G.toNumpy(cnt)) == int(mask.sum())
        # the probe does see an allocation: the same fold through the allocating entry point on a stream without a workspace
        free2 = _free_device_bytes()
        native.check(lib.dnh_reduce_last_axis(abi.DNH_SUM, C.byref(td), C.byref(sd), control))
        native.check(lib.dnh_stream_sync(control))
        assert _free_device_bytes() < free2, "control: the allocating entry point took no workspace, so this shape does not test the property"
        assert np.array_equal(G.toNumpy(trgt), want)
    finally:
        native.check(lib.dnh_stream_destroy(fresh))
        native.check(lib.dnh_stream_destroy(control))


def test_noalloc_fold_refuses_partials_beyond_the_static_array(G, rng):
    lib = native.load()
    # CountTrue down the columns of a bool matrix keeps one int64 partial per (chunk of rows, column): 65536 columns x 64 chunks
    # x 8 bytes = 32 MiB.  The matrix is one row of 65536 bools read 32768 times through a stride-0 view.
    cols, rows = 1 << 16, 1 << 15
    mask = rng.random(cols) < 0.5
    row = G.ofNumpy(mask)
    sd = abi.make_descriptor(row.Storage.Pointer(), np.bool_, [cols, rows], [1, 0], 0)
    trgt = G.zeros((cols,), np.int64)
    td = trgt.Backend._desc(trgt)
    status = lib.dnh_reduce_last_axis_noalloc(abi.DNH_COUNT_TRUE, C.byref(td), C.byref(sd), G.Cfg.Stream)
    assert status == abi.DNH_ERR_NOT_SUPPORTED
    assert "static scratch" in native.last_error()
    # the allocating entry point takes the same fold
    native.check(lib.dnh_reduce_last_axis(abi.DNH_COUNT_TRUE, C.byref(td), C.byref(sd), G.Cfg.Stream))
    assert np.array_equal(G.toNumpy(trgt), mask.astype(np.int64) * rows)
