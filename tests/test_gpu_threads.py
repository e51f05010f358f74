"""Thread safety of the C ABI: several host threads, each on its own stream (Cfg.Stream is thread-local, as in the reference's
Cuda/CudaCfg.fs:16), run chains that allocate from the block cache and use the per-stream workspace (split reductions,
compaction) at the same time.  ctypes releases the GIL during every call, so the calls really overlap."""
import ctypes as C
import threading

import numpy as np
import pytest

from deepnet_amd import native

pytestmark = pytest.mark.gpu


def test_concurrent_threads_on_their_own_streams(G, H):
    lib = native.load()
    nthreads, rounds = 4, 6
    rng = np.random.default_rng(7)
    inputs = [(rng.integers(-1000, 1000, (600, 700)).astype(np.int32), rng.integers(-1000, 1000, (600, 700)).astype(np.int32))
              for _ in range(nthreads)]

    def chain(M, a, b):
        x, y = M.ofNumpy(a), M.ofNumpy(b)
        out = []
        for _ in range(rounds):
            x = (x * y + x) - y                       # temporaries from the block cache
            out.append(M.toNumpy(x.sumAxis(0)))       # column fold with a finishing pass (per-stream workspace)
            out.append(M.toNumpy(x.flatten().sumAxis(0)))
            m = x > y
            out.append(M.toNumpy(x.flatten().M(m.flatten())))     # compaction: counts in the workspace
            out.append(M.toNumpy(x.argMaxAxis(1)))
        return out

    want = [chain(H, a, b) for a, b in inputs]
    got = [None] * nthreads
    errors = []

    def worker(i):
        try:
            s = C.c_void_p()
            native.check(lib.dnh_stream_create(C.byref(s)))
            G.Cfg.Stream = s.value
            try:
                got[i] = chain(G, *inputs[i])
            finally:
                G.synchronize()
                G.Cfg.Stream = 0
                native.check(lib.dnh_stream_destroy(s))
        except Exception as e:  # noqa: BLE001
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(nthreads)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    for i in range(nthreads):
        assert got[i] is not None
        for ref, g in zip(want[i], got[i]):
            np.testing.assert_array_equal(ref, g)


def test_concurrent_inversions_share_the_side_stream(G):
    """BatchedInvert by tournament updates part of the matrix on one stream of the library's own, ordered against the caller's stream
    by events of the call.  Four host threads on four streams invert at once: their side-stream work interleaves in one queue, and
    every result must be what the same call gives alone, bit for bit."""
    from deepnet_amd.tensor import Tensor
    lib = native.load()
    nthreads = 4
    rng = np.random.default_rng(11)
    inputs = [(rng.standard_normal((n, n)) / np.sqrt(n) + 2 * np.eye(n)).astype(dt)
              for n, dt in ((700, np.float32), (450, np.float64), (1100, np.float32), (260, np.float32))]
    want = [G.toNumpy(Tensor.invert(G.ofNumpy(a))) for a in inputs]
    got = [None] * nthreads
    errors = []

    def worker(i):
        try:
            s = C.c_void_p()
            native.check(lib.dnh_stream_create(C.byref(s)))
            G.Cfg.Stream = s.value
            try:
                t = G.ofNumpy(inputs[i])
                for _ in range(3):
                    r = Tensor.invert(t)
                got[i] = G.toNumpy(r)
            finally:
                G.synchronize()
                G.Cfg.Stream = 0
                native.check(lib.dnh_stream_destroy(s))
        except Exception as e:  # noqa: BLE001
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(nthreads)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    for i in range(nthreads):
        np.testing.assert_array_equal(got[i], want[i])
        n = inputs[i].shape[0]
        assert np.abs(got[i].astype(np.float64) @ inputs[i].astype(np.float64) - np.eye(n)).max() <= 64 * n * np.finfo(inputs[i].dtype).eps


def test_concurrent_threads_sharing_one_stream(G, H):
    """Host threads that never set Cfg.Stream all enqueue on the default stream and so share its workspace: an entry point keeps
    the buffer to itself until every kernel that uses it is queued, so split folds, compactions and split products of different
    threads cannot read each other's partials."""
    nthreads, rounds = 4, 8
    rng = np.random.default_rng(11)
    inputs = [(rng.integers(-1000, 1000, (512, 640)).astype(np.int32),
               rng.standard_normal((96, 2048)).astype(np.float64)) for _ in range(nthreads)]

    def chain(M, a, f):
        x, y = M.ofNumpy(a), M.ofNumpy(f)
        out = []
        for r in range(rounds):
            x = x + r
            out.append(M.toNumpy(x.sumAxis(0)))                        # column fold, partials + finishing pass
            out.append(M.toNumpy(x.flatten().maxAxis(0)))              # long row, split
            out.append(M.toNumpy(x.flatten().M((x > 0).flatten())))    # compaction, block counts
            out.append(M.toNumpy(y @ y.T))                             # 96 x 2048 x 96: one tile, K cut into chunks
        return out

    want = [chain(H, a, f) for a, f in inputs]
    got = [None] * nthreads
    errors = []

    def worker(i):
        try:
            got[i] = chain(G, *inputs[i])
        except Exception as e:  # noqa: BLE001
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(nthreads)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    for i in range(nthreads):
        assert got[i] is not None
        for k, (ref, g) in enumerate(zip(want[i], got[i])):
            if k % 4 == 3:   # the fp64 product: summation order differs from the oracle's
                np.testing.assert_allclose(g, ref, rtol=0, atol=1e-9)
            else:
                np.testing.assert_array_equal(ref, g)


def test_index_error_flag_is_per_stream(G):
    """An out-of-range gather index on one stream is reported on that stream only."""
    lib = native.load()
    s = C.c_void_p()
    native.check(lib.dnh_stream_create(C.byref(s)))
    try:
        src = G.ofNumpy(np.arange(10, dtype=np.int32))
        bad = G.ofNumpy(np.array([1, 99, 3], dtype=np.int64))
        good = G.ofNumpy(np.array([1, 2, 3], dtype=np.int64))
        G.synchronize()
        stack = G.Cfg.Stacktrace
        G.Cfg.Stacktrace = False                      # do not read the flag back after each call
        try:
            G.Cfg.Stream = s.value
            type(src).gather([bad], src)              # sets the flag of stream s
            G.Cfg.Stream = 0
            type(src).gather([good], src)
            code = C.c_int32(-1)
            native.check(lib.dnh_async_error(0, C.byref(code)))
            assert code.value == 0                    # the default stream saw no error
            native.check(lib.dnh_async_error(s.value, C.byref(code)))
            assert code.value == 5                    # DNH_ERR_INDEX_OUT_OF_RANGE, and the read cleared it
            native.check(lib.dnh_async_error(s.value, C.byref(code)))
            assert code.value == 0
        finally:
            G.Cfg.Stream = 0
            G.Cfg.Stacktrace = stack
    finally:
        native.check(lib.dnh_stream_destroy(s))
