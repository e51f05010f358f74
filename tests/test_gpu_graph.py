"""The entry points under HIP graph capture: a chain of element-wise ops and folds on preallocated targets is recorded once on a
stream (after a warm-up call on that stream has sized the library's workspace, so nothing allocates while recording) and
replayed several times with the program's own eager work and synchronisations in between; every replay must equal the eager
result on the same inputs, bit for bit.  No memset node is recorded (the chain clears nothing)."""
import ctypes as C

import numpy as np
import pytest

from deepnet_amd import abi, native
from deepnet_amd.backend import CAbiTensorBackend

pytestmark = pytest.mark.gpu

hipStreamCaptureModeThreadLocal = 1


def _hip():
    hip = C.CDLL("libamdhip64.so")
    for f in ("hipStreamBeginCapture", "hipStreamEndCapture", "hipGraphInstantiate", "hipGraphLaunch", "hipGraphExecDestroy",
              "hipGraphDestroy"):
        getattr(hip, f).restype = C.c_int
    return hip


def test_chain_replayed_from_a_graph_matches_eager(G):
    lib, hip = native.load(), _hip()
    rng = np.random.default_rng(5)
    n = 1000
    a0 = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    b0 = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    stream = C.c_void_p()
    native.check(lib.dnh_stream_create(C.byref(stream)))
    G.Cfg.Stream = stream.value
    try:
        a, b = G.ofNumpy(a0), G.ofNumpy(b0)
        y, z = G.zeros([n, n], np.float32), G.zeros([n, n], np.float32)
        rows, cols, amax = G.zeros([n], np.float32), G.zeros([n], np.float32), G.zeros([n], np.int64)
        total = G.zeros([], np.float32)
        keep = []

        def desc(t):
            d = CAbiTensorBackend._desc(t)
            keep.append(d)
            return C.byref(d)

        calls = [
            ("binary", (abi.DNH_ADD, desc(y), desc(a), desc(b))),
            ("unary", (abi.DNH_TANH, desc(z), desc(y))),
            ("reduce_last_axis", (abi.DNH_SUM, desc(rows), desc(z))),
            ("reduce_last_axis", (abi.DNH_SUM, desc(cols), desc(z.T))),          # column fold: partials in the stream's workspace
            ("arg_reduce_last_axis", (abi.DNH_ARG_MAX, desc(amax), desc(z))),
            ("reduce_last_axis", (abi.DNH_SUM, desc(total), desc(z.flatten()))),  # split fold + finishing pass
        ]

        def issue():
            for entry, args in calls:
                native.check(getattr(lib, "dnh_" + entry)(*args, stream))

        def snapshot():
            G.synchronize()
            return [G.toNumpy(t).copy() for t in (y, z, rows, cols, amax, total)]

        def poison():
            for t in (y, z, rows, cols, total):
                t.FillConst(np.float32(-7))
            amax.FillConst(np.int64(-7))
            G.synchronize()

        issue()                      # warm-up on this stream: sizes its workspace
        eager0 = snapshot()

        graph, gexec = C.c_void_p(), C.c_void_p()
        assert hip.hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal) == 0
        try:
            issue()
        finally:
            rc = hip.hipStreamEndCapture(stream, C.byref(graph))
        assert rc == 0 and graph.value
        assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)) == 0
        try:
            for rep in range(4):
                if rep:   # eager work between the replays: the inputs change in place
                    a.FillAdd(a, b)
                    G.synchronize()
                poison()                                # so that a replay that did nothing cannot pass
                assert hip.hipGraphLaunch(gexec, stream) == 0
                got = snapshot()
                poison()
                issue()
                want = snapshot()
                for g, w in zip(got, want):
                    np.testing.assert_array_equal(g, w)
                if rep == 0:
                    for g, w in zip(got, eager0):
                        np.testing.assert_array_equal(g, w)
        finally:
            hip.hipGraphExecDestroy(gexec)
            hip.hipGraphDestroy(graph)
    finally:
        G.synchronize()
        G.Cfg.Stream = 0
        native.check(lib.dnh_stream_destroy(stream))
