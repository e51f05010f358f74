"""CPU: the C-ABI library loads, exports every symbol include/tensor_hip.h declares, its descriptor layout matches the header
as compiled by gcc, and — with no GPU in the machine — the product path fails loudly instead of falling back."""
import ctypes as C
import os
import re
import subprocess
import tempfile

import numpy as np
import pytest

from deepnet_amd import abi, native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tensor_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    return sorted(set(re.findall(r"^int32_t\s+(dnh_\w+)\s*\(", text, flags=re.M)))


def test_library_exports_every_declared_symbol():
    lib = native.load()
    names = declared_symbols()
    assert len(names) >= 39
    for n in names:
        assert hasattr(lib, n), f"libtensor_hip.so lacks {n}"
    assert sorted(abi.EXPORTED_SYMBOLS) == names, "deepnet_amd/abi.py and include/tensor_hip.h disagree"


def test_descriptor_layout_matches_the_header():
    src = r'''
#include <stdio.h>
#include <stddef.h>
#include "tensor_hip.h"
int main(void) {
  printf("%zu %zu %zu %zu %zu %zu %zu %zu\n", sizeof(DnhTensor), offsetof(DnhTensor, base), offsetof(DnhTensor, offset),
         offsetof(DnhTensor, ndims), offsetof(DnhTensor, dtype), offsetof(DnhTensor, shape), offsetof(DnhTensor, stride), sizeof(DnhDeviceInfo));
  printf("%d %d %d %d %d %d %d %lld\n", DNH_F64, DNH_I16, DNH_U16, DNH_NEGATE, DNH_XOR, DNH_GREATER_OR_EQUAL, DNH_COUNT_TRUE, (long long)DNH_NOT_FOUND);
  return 0; }'''
    with tempfile.TemporaryDirectory() as d:
        c = os.path.join(d, "t.c")
        open(c, "w").write(src)
        exe = os.path.join(d, "t")
        subprocess.check_call(["gcc", "-std=c99", "-I", os.path.join(ROOT, "include"), c, "-o", exe])
        out = subprocess.check_output([exe]).decode().split()
    vals = [int(x) for x in out]
    T = abi.DnhTensor
    assert vals[:8] == [C.sizeof(T), T.base.offset, T.offset.offset, T.ndims.offset, T.dtype.offset, T.shape.offset, T.stride.offset,
                        C.sizeof(abi.DnhDeviceInfo)]
    assert vals[8:] == [abi.DNH_F64, abi.DNH_I16, abi.DNH_U16, abi.DNH_NEGATE, abi.DNH_XOR, abi.DNH_GREATER_OR_EQUAL, abi.DNH_COUNT_TRUE, abi.NOT_FOUND]


def test_oracle_exports_the_same_operator_set():
    from oracle import hostref
    lib = hostref.load()
    for name in abi.OP_SIGNATURES:
        assert hasattr(lib, "href_" + name)


def _have_gpu():
    return os.path.exists("/dev/kfd") and os.access("/dev/kfd", os.R_OK | os.W_OK)


@pytest.mark.skipif(_have_gpu(), reason="a GPU is present; this test pins the no-GPU failure mode")
def test_product_path_fails_loudly_without_a_gpu():
    from deepnet_amd import hip
    with pytest.raises(native.HipError):
        hip.ofNumpy(np.zeros(4, np.float32))
    assert "HIP" in native.last_error() or "hip" in native.last_error()
    # argument validation happens before any device work and reports through the same channel
    lib = native.load()
    assert lib.dnh_last_error(None, 0) == abi.DNH_ERR_INVALID_ARG


def test_status_codes_map_to_reference_exception_kinds():
    assert native._EXC[abi.DNH_ERR_INVALID_ARG] is ValueError
    assert native._EXC[abi.DNH_ERR_NOT_SUPPORTED] is NotImplementedError
    assert native._EXC[abi.DNH_ERR_INDEX_OUT_OF_RANGE] is IndexError
    assert native._EXC[abi.DNH_ERR_OUT_OF_MEMORY] is MemoryError


def test_options_are_set_and_read_without_a_device():
    """dnh_set_option / dnh_get_option touch no GPU: defaults, round trip, refusal of unknown names and of values out of range."""
    defaults = {"dot_bf16x3": 1, "dot_f64_pinned": 1, "dot_big": -1, "dot_splits": 0, "dot_int_mfma": 1, "tr4": 1,
                "scatter_fp_atomic": 0, "compact_one_pass": 0, "count_one_launch": 1, "lookback_spins": 1 << 18,
                "invert_tournament": -1}
    header = open(HEADER).read()
    for name, value in defaults.items():
        assert f'"{name}"' in header, f"include/tensor_hip.h does not document option {name}"
        if os.environ.get("DNH_" + name.upper()) is None:
            assert native.get_option(name) == value
        with native.option(name, 0):
            assert native.get_option(name) == 0
        assert native.get_option(name) == (value if os.environ.get("DNH_" + name.upper()) is None else native.get_option(name))
    with pytest.raises(ValueError):
        native.set_option("dot_big", 2)
    with pytest.raises(ValueError):
        native.set_option("dot_bf16x3", -1)
    with pytest.raises(ValueError):
        native.get_option("nonexistent")
    assert "nonexistent" in native.last_error()


def test_scatter_workspace_sizes():
    """The workspace a scatter asks for, against the formulas restated here: the binned form for 32-bit integers (per-workgroup
    bucket counts, bucket totals, 8 bytes per pair; taken only when its cost model beats 40 ps per direct update and the workspace
    stays within 1 GiB), the ordered form for floats (cells, counts, totals and starts, sorted cells and values)."""
    lib = native.load()

    def ask(dtype, m, n):
        b = C.c_size_t()
        native.check(lib.dnh_scatter_workspace_bytes(dtype, m, n, C.byref(b)))
        return b.value

    up = lambda x: (x + 255) // 256 * 256
    # 32-bit integers
    def binned(m, n):
        nb, nchunks = -(-n // 16384), -(-m // 8192)
        counts = up(nb * nchunks * 4)
        ws = counts + up(nb * 4) + 8 * m
        cheaper = (n * 8.0 + m * 36.0 + counts * 4.0) / 5.5e6 + 10.0 < m * 40e-6
        return ws if (m >= 1 << 20 and m <= 2 ** 31 - 1 and 1 <= n <= 4096 * 16384 and cheaper and ws <= 1 << 30) else 0
    for m, n in ((1 << 22, 1 << 24), (1 << 20, 300_000), ((1 << 20) - 1, 1 << 24), (1 << 21, 1 << 26), (1 << 28, 1 << 26), (1 << 22, (1 << 26) + 1)):
        assert ask(abi.DNH_I32, m, n) == binned(m, n), (m, n)
        assert ask(abi.DNH_U32, m, n) == binned(m, n)
    assert ask(abi.DNH_I32, 1 << 22, 1 << 24) == 2 * 1024 * 1024 + 4096 + 8 * (1 << 22)
    assert ask(abi.DNH_I32, 1 << 28, 1 << 26) == 0        # 512 MB of counts + 2 GB of pairs: beyond the cap, the direct kernel is taken
    assert ask(abi.DNH_I64, 1 << 22, 1 << 24) == 0 and ask(abi.DNH_U8, 1 << 22, 1 << 24) == 0
    # floats
    def ordered(m, n, esize):
        lg = max(n - 1, 0).bit_length()
        shift = min(max(lg - 10, 4), 13)
        nb = min(-(-n // (1 << shift)), 4096)
        nchunks = -(-m // 8192)
        return up(8 * m) + up(nb * nchunks * 4) + 2 * up(nb * 4) + up(4 * m) + up(esize * m)
    for m, n in ((1 << 22, 1 << 24), (50_000, 777), (1, 1), (70_000, 1), (1 << 20, 40_000_000), (8191, 100_000)):
        assert ask(abi.DNH_F32, m, n) == ordered(m, n, 4), (m, n)
        assert ask(abi.DNH_F64, m, n) == ordered(m, n, 8), (m, n)
    with native.option("scatter_fp_atomic", 1):
        assert ask(abi.DNH_F32, 1 << 22, 1 << 24) == 0
    assert ask(abi.DNH_F32, 0, 100) == 0 and ask(abi.DNH_F32, 100, 0) == 0
    b = C.c_size_t()
    assert lib.dnh_scatter_workspace_bytes(99, 1, 1, C.byref(b)) == abi.DNH_ERR_INVALID_ARG
