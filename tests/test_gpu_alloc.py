"""Stream-ordered block cache (dnh_alloc_async / dnh_free_async) through the C ABI, and tensors that live in it."""
import ctypes as C

import numpy as np
import pytest

from deepnet_amd import abi, native

pytestmark = pytest.mark.gpu


def _stats(lib):
    st = abi.DnhPoolStats()
    native.check(lib.dnh_pool_stats(C.byref(st)))
    return st


def _alloc(lib, nbytes, stream=0):
    p = C.c_void_p()
    native.check(lib.dnh_alloc_async(nbytes, stream, C.byref(p)))
    return p.value


def test_block_is_reused_on_its_stream_only(G):
    lib = native.load()
    native.check(lib.dnh_pool_trim())
    s = C.c_void_p()
    native.check(lib.dnh_stream_create(C.byref(s)))
    try:
        p = _alloc(lib, 3 << 20)
        native.check(lib.dnh_free_async(p, 0))
        assert _stats(lib).cached_bytes == 4 << 20            # rounded to the 2 MiB granule
        q = _alloc(lib, 3 << 20, s.value)                     # other stream: must not take the cached block
        assert q != p
        r = _alloc(lib, (3 << 20) + 5)                        # same stream, same size class: reuse
        assert r == p
        assert _stats(lib).cached_bytes == 0
        big = _alloc(lib, 64 << 20)
        native.check(lib.dnh_free_async(big, 0))
        small = _alloc(lib, 8 << 20)                          # a block 8x larger than the request is not handed out
        assert small != big
        for ptr, st in ((q, s.value), (r, 0), (small, 0)):
            native.check(lib.dnh_free_async(ptr, st))
        assert _stats(lib).live_bytes >= 0
    finally:
        native.check(lib.dnh_stream_destroy(s))
    # the destroyed stream's blocks stay cached (moved to the default stream)
    assert _stats(lib).cached_bytes >= (4 << 20) + (64 << 20) + (8 << 20)
    native.check(lib.dnh_pool_trim())
    assert _stats(lib).cached_bytes == 0


def test_limit_and_synchronising_free(G):
    lib = native.load()
    native.check(lib.dnh_pool_trim())
    native.check(lib.dnh_pool_set_limit(1 << 20))
    try:
        p = _alloc(lib, 4 << 20)
        native.check(lib.dnh_free_async(p, 0))                # over the cap: goes back to the driver
        assert _stats(lib).cached_bytes == 0
        q = _alloc(lib, 1000)
        live = _stats(lib).live_bytes
        native.check(lib.dnh_free(q))                         # dnh_free takes cache blocks too
        assert _stats(lib).live_bytes == live - 1024
    finally:
        native.check(lib.dnh_pool_set_limit(0))


def test_chain_results_unchanged_by_reuse(G, H, rng):
    """Temporaries of a chain are released and reused while earlier kernels may still be queued."""
    a = rng.standard_normal((512, 300)).astype(np.float32)
    b = rng.standard_normal((512, 300)).astype(np.float32)
    lib = native.load()
    hits0 = _stats(lib).hits

    def chain(M, a, b):
        x = M.ofNumpy(a)
        y = M.ofNumpy(b)
        for _ in range(20):
            x = (x * y + x).abs() - y        # every step drops two temporaries of the same size
        return M.toNumpy(x), M.toNumpy(x.sumAxis(0))

    got, got_s = chain(G, a, b)
    want, want_s = chain(H, a, b)
    np.testing.assert_array_equal(got, want)
    np.testing.assert_allclose(got_s, want_s, rtol=1e-4)
    assert _stats(lib).hits > hits0 + 20


def test_storage_used_on_two_streams_takes_the_synchronising_free(G):
    lib = native.load()
    s = C.c_void_p()
    native.check(lib.dnh_stream_create(C.byref(s)))
    try:
        x = G.ofNumpy(np.arange(1000, dtype=np.float32))
        assert x.Storage._single_stream
        G.Cfg.Stream = s.value
        try:
            native.check(lib.dnh_device_sync())
            y = x + x
            assert not x.Storage._single_stream and y.Storage._single_stream and y.Storage._stream == s.value
            np.testing.assert_array_equal(G.toNumpy(y), 2 * np.arange(1000, dtype=np.float32))
        finally:
            G.Cfg.Stream = 0
        cached = _stats(lib).cached_bytes
        del x                                                 # used on two streams: not cached
        assert _stats(lib).cached_bytes == cached
        del y
    finally:
        native.check(lib.dnh_stream_destroy(s))


def test_device_is_chosen_once(G):
    """dnh_init with the device in use is a no-op; any other device is refused, since buffers, cached blocks and workspaces
    already live on the first one."""
    lib = native.load()
    assert lib.dnh_init(0) == abi.DNH_OK
    assert lib.dnh_init(1) == abi.DNH_ERR_INVALID_ARG
    buf = C.create_string_buffer(256)
    lib.dnh_last_error(buf, 256)
    assert b"device" in buf.value
    x = G.ofNumpy(np.arange(6, dtype=np.int32))
    assert G.toNumpy(x + x).tolist() == [0, 2, 4, 6, 8, 10]


def test_using_ptr_references_existing_device_memory(G):
    """HipTensor.usingPtr (the reference's CudaTensor.usingPtr, Cuda/CudaFrontend.fs:129-149): a tensor over memory somebody else
    owns; writes through it change the original data, and collecting it frees nothing."""
    import ctypes as C
    from deepnet_amd import layout as L
    lib = native.load()
    owner = G.ofNumpy(np.arange(24, dtype=np.float32))
    ptr = owner.Storage.Pointer()
    view = G.usingPtr(ptr, 24 * 4, np.float32, L.newC((4, 6)))
    assert np.array_equal(G.toNumpy(view), np.arange(24, dtype=np.float32).reshape(4, 6))
    view.Backend.Add(view, view, view)
    assert np.array_equal(G.toNumpy(owner), 2 * np.arange(24, dtype=np.float32))
    col = G.usingPtr(ptr, 24 * 4, np.float32, L.TensorLayout((4,), 1, (6,)))     # column 1 of the 4 x 6 matrix
    assert np.array_equal(G.toNumpy(col), 2 * np.arange(24, dtype=np.float32).reshape(4, 6)[:, 1])
    before = abi.DnhPoolStats()
    native.check(lib.dnh_pool_stats(C.byref(before)))
    del view, col
    after = abi.DnhPoolStats()
    native.check(lib.dnh_pool_stats(C.byref(after)))
    assert (before.live_bytes, before.cached_bytes) == (after.live_bytes, after.cached_bytes)
    assert np.array_equal(G.toNumpy(owner), 2 * np.arange(24, dtype=np.float32))
    with pytest.raises(ValueError):
        G.usingPtr(ptr, 24 * 4, np.float32, L.newC((5, 6)))                       # the layout does not fit the allocation
    with pytest.raises(ValueError):
        G.usingPtr(0, 24 * 4, np.float32, L.newC((4, 6)))


def test_block_released_on_a_destroyed_stream_is_reused(G):
    """A storage finalizer may run after its stream was destroyed: the block then goes to the default stream's list (everything
    queued on the dead stream has finished) instead of being filed under a handle nobody will ask for again."""
    import ctypes as C
    lib = native.load()
    st = C.c_void_p()
    native.check(lib.dnh_stream_create(C.byref(st)))
    p = C.c_void_p()
    size = 3 * (1 << 20) + 4096                                   # an unusual size, so the hit below is this block
    native.check(lib.dnh_alloc_async(size, st, C.byref(p)))
    native.check(lib.dnh_stream_destroy(st))
    native.check(lib.dnh_free_async(p, st))                       # late release, naming the dead stream
    before = abi.DnhPoolStats()
    native.check(lib.dnh_pool_stats(C.byref(before)))
    q = C.c_void_p()
    native.check(lib.dnh_alloc_async(size, None, C.byref(q)))     # default stream
    after = abi.DnhPoolStats()
    native.check(lib.dnh_pool_stats(C.byref(after)))
    assert after.hits == before.hits + 1 and q.value == p.value
    native.check(lib.dnh_free_async(q, None))
