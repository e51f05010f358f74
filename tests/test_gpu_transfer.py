"""GPU: host <-> device copies through the C ABI.  Synchronous copies of 16 MiB and more between pageable host memory and the device
are staged by the library through pinned chunks on several threads; every byte must arrive whatever the size and alignment, from
pinned memory the plain path is taken, and concurrent callers take turns."""
import ctypes as C
import threading

import numpy as np
import pytest

from deepnet_amd import native

pytestmark = pytest.mark.gpu

MiB = 1 << 20


def roundtrip(lib, host_in, host_out_ptr, nbytes, dev):
    native.check(lib.dnh_memcpy_h2d(dev, host_in.ctypes.data, nbytes, None, 1))
    native.check(lib.dnh_memcpy_d2h(host_out_ptr, dev, nbytes, None, 1))


@pytest.mark.parametrize("nbytes", [16 * MiB - 1, 16 * MiB, 16 * MiB + 1, 24 * MiB + 12345, 100 * MiB + 7, 4 * MiB * 13])
def test_pageable_round_trip(nbytes):
    lib = native.load()
    rng = np.random.default_rng(nbytes)
    src = rng.integers(0, 256, nbytes + 3, dtype=np.uint8)[3:]            # not even 4-byte aligned
    back = np.zeros(nbytes + 5, np.uint8)[5:]
    dev = C.c_void_p()
    native.check(lib.dnh_alloc(nbytes, C.byref(dev)))
    try:
        roundtrip(lib, src, back.ctypes.data, nbytes, dev)
        assert np.array_equal(src, back)
        # a copy into the middle of the buffer leaves the rest alone
        part = rng.integers(0, 256, 17 * MiB, dtype=np.uint8)
        off = 1 * MiB + 1
        if nbytes >= off + part.size:
            native.check(lib.dnh_memcpy_h2d(dev.value + off, part.ctypes.data, part.size, None, 1))
            native.check(lib.dnh_memcpy_d2h(back.ctypes.data, dev, nbytes, None, 1))
            want = src.copy()
            want[off:off + part.size] = part
            assert np.array_equal(want, back)
    finally:
        native.check(lib.dnh_free(dev))


def test_pinned_round_trip_and_ordering_after_kernels():
    from deepnet_amd import hip as G
    lib = native.load()
    nbytes = 64 * MiB
    pinned = C.c_void_p()
    native.check(lib.dnh_host_alloc(nbytes, C.byref(pinned)))
    try:
        view = np.ctypeslib.as_array(C.cast(pinned, C.POINTER(C.c_uint8)), shape=(nbytes,))
        view[:] = np.random.default_rng(1).integers(0, 256, nbytes, dtype=np.uint8)
        t = G.zeros([nbytes], np.uint8)
        native.check(lib.dnh_memcpy_h2d(t.Storage.Pointer(), pinned, nbytes, None, 1))
        doubled = t + t                                                    # queued on the stream, not waited for
        out = np.empty(nbytes, np.uint8)                                   # pageable: the staged path must wait for the kernel
        native.check(lib.dnh_memcpy_d2h(out.ctypes.data, doubled.Storage.Pointer(), nbytes, None, 1))
        assert np.array_equal(out, view + view)
    finally:
        native.check(lib.dnh_host_free(pinned))


def test_concurrent_staged_copies():
    lib = native.load()
    nbytes = 40 * MiB + 3
    errors = []

    def worker(seed):
        try:
            src = np.random.default_rng(seed).integers(0, 256, nbytes, dtype=np.uint8)
            back = np.zeros(nbytes, np.uint8)
            dev = C.c_void_p()
            native.check(lib.dnh_alloc(nbytes, C.byref(dev)))
            for _ in range(3):
                roundtrip(lib, src, back.ctypes.data, nbytes, dev)
            native.check(lib.dnh_free(dev))
            if not np.array_equal(src, back):
                errors.append(f"thread {seed}: data differs")
        except Exception as e:  # noqa: BLE001
            errors.append(repr(e))
    threads = [threading.Thread(target=worker, args=(s,)) for s in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
