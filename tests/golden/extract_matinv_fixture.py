#!/usr/bin/env python3
"""Writes tests/golden/matinv_kk.json: the dataset "Kk" (single, shape [3; 10; 10]) of the reference's test data file
Tensor/Tensor.Test/TestData/MatInv.h5, which its test ``Invert Kk matrix`` (Tensor.Test/BaseTests.fs:214-233) inverts and
checks with  invert(Kk) .* Kk = identity  to absTol = relTol = 1e-5.

No HDF5 library is installed, so the few structures needed are read by hand (HDF5 file format 1.x, superblock version 0):
the symbol-table node gives the object header of "Kk"; its messages give the dataspace (0x0001), the datatype (0x0003,
checked to be little-endian IEEE single) and the contiguous data layout (0x0008: address and size of the raw data).
Only data is taken from the file; run it where /root/reference is present.
"""
import json
import os
import struct
import sys

import numpy as np

SRC = "/root/reference/Tensor/Tensor.Test/TestData/MatInv.h5"


def read_dataset(path, name):
    d = open(path, "rb").read()
    assert d[:8] == b"\x89HDF\r\n\x1a\n" and d[8] == 0 and d[13] == 8 and d[14] == 8, "unexpected HDF5 superblock"
    heap = d.index(b"HEAP")
    heap_data = struct.unpack_from("<Q", d, heap + 24)[0]
    snod = d.index(b"SNOD")
    nsym = struct.unpack_from("<H", d, snod + 6)[0]
    for k in range(nsym):
        name_off, ohdr = struct.unpack_from("<QQ", d, snod + 8 + 40 * k)
        end = d.index(b"\0", heap_data + name_off)
        if d[heap_data + name_off:end].decode() != name:
            continue
        version, _, nmsg = struct.unpack_from("<BBH", d, ohdr)
        assert version == 1
        p = ohdr + 16
        shape = dtype_ok = addr = size = None
        for _ in range(nmsg):
            mtype, msize = struct.unpack_from("<HH", d, p)
            body = d[p + 8:p + 8 + msize]
            if mtype == 0x1:
                rank = body[1]
                shape = list(struct.unpack_from(f"<{rank}Q", body, 8))
            elif mtype == 0x3:
                cls, bits0 = body[0] & 0x0F, body[1]
                dtype_ok = cls == 1 and (bits0 & 1) == 0 and struct.unpack_from("<I", body, 4)[0] == 4
            elif mtype == 0x8:
                assert body[0] == 3 and body[1] == 1, "expected a version-3 contiguous layout"
                addr, size = struct.unpack_from("<QQ", body, 2)
            p += 8 + msize
        assert shape and dtype_ok and addr is not None
        arr = np.frombuffer(d[addr:addr + size], dtype="<f4").reshape(shape)
        return arr
    raise KeyError(name)


if __name__ == "__main__":
    kk = read_dataset(SRC, "Kk")
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "matinv_kk.json")
    with open(out, "w") as f:
        json.dump({"source": "Tensor/Tensor.Test/TestData/MatInv.h5 dataset Kk (used by Tensor.Test/BaseTests.fs:214-233)",
                   "dtype": "float32", "shape": list(kk.shape),
                   "data_hex": kk.astype("<f4").tobytes().hex(),
                   "check": {"abs_tol": 1e-5, "rel_tol": 1e-5, "property": "invert(Kk) . Kk == identity"}}, f, indent=1)
    print("wrote", out, kk.shape, float(np.abs(kk).max()), file=sys.stderr)
