"""Known-answer vectors for Convert of floats that do not fit the integer target, worked out by hand from the rule the backends
state (truncate toward zero; NaN and out-of-range values give the minimum of int32 / int64; the 8- and 16-bit types go through int32
and uint32 through int64, keeping the low bits; uint64 splits at 2^63).  Inputs are doubles that are exactly representable."""
import numpy as np

I32_MIN, I64_MIN = -2 ** 31, -2 ** 63
U64 = 2 ** 64

INPUTS = [float("nan"), float("inf"), float("-inf"), -1.0, -0.9, 255.9, 256.0, 300.7, -129.2, 2147483647.0, 2147483648.0,
          -2147483648.0, -2147483649.0, 4294967301.0, 1e10, -1e10, 9.3e18, 18446744073709551616.0, 1e20, -9.3e18]

EXPECTED = {
    np.int32: [I32_MIN, I32_MIN, I32_MIN, -1, 0, 255, 256, 300, -129, 2147483647, I32_MIN, I32_MIN, I32_MIN, I32_MIN, I32_MIN, I32_MIN,
               I32_MIN, I32_MIN, I32_MIN, I32_MIN],
    np.int64: [I64_MIN, I64_MIN, I64_MIN, -1, 0, 255, 256, 300, -129, 2147483647, 2147483648, -2147483648, -2147483649, 4294967301,
               10 ** 10, -10 ** 10, I64_MIN, I64_MIN, I64_MIN, I64_MIN],
    np.uint8: [0, 0, 0, 255, 0, 255, 0, 44, 127, 255, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0],
    np.int8: [0, 0, 0, -1, 0, -1, 0, 44, 127, -1, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0],
    np.uint16: [0, 0, 0, 65535, 0, 255, 256, 300, 65407, 65535, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0],
    np.int16: [0, 0, 0, -1, 0, 255, 256, 300, -129, -1, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0],
    np.uint32: [0, 0, 0, 4294967295, 0, 255, 256, 300, 4294967167, 2147483647, 2147483648, 2147483648, 2147483647, 5, 1410065408,
                2884901888, 0, 0, 0, 0],
    np.uint64: [0, 0, 2 ** 63, U64 - 1, 0, 255, 256, 300, U64 - 129, 2147483647, 2147483648, U64 - 2147483648, U64 - 2147483649,
                4294967301, 10 ** 10, U64 - 10 ** 10, 9300000000000000000, 0, 0, 2 ** 63],
}


def expected(dst):
    return np.array([int(v) for v in EXPECTED[dst]], dtype=object).astype(np.dtype(dst))
