"""Single-precision Dot on operands of different bit activity: the same launches of the same kernels, only the operand bits differ.

The bf16-parts kernels issue six bf16 matrix instructions per multiply-add; how fast the matrix pipes run them depends on how many
operand bits toggle (the shader clock is pulled down under load).  This program times the product on zeros, on ones and small
integers (only the leading part of each float is non-zero), on random floats that bf16 represents exactly (one live product of the
six) and on random normal floats (all six live), on the bf16-parts kernels and, behind the library's switch, on the fp32 matrix
instruction.  One JSON line per case; every case issues `--warmup` + `--reps` launches, in the order printed, so that a counter run
of this program can be split by dispatch number.

    python bench_dot_operands.py [--shapes 4000,64x512] [--reps 20] [--warmup 5]
"""
import argparse
import ctypes as C
import json

import numpy as np


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--shapes", default="4000,64x512")
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    args = ap.parse_args()
    from deepnet_amd import hip as G, native
    lib = native.load()
    rng = np.random.default_rng(7)

    def timed(fn):
        e0, e1 = C.c_void_p(), C.c_void_p()
        native.check(lib.dnh_event_create(C.byref(e0)))
        native.check(lib.dnh_event_create(C.byref(e1)))
        for _ in range(args.warmup):
            fn()
        native.check(lib.dnh_event_record(e0, None))
        for _ in range(args.reps):
            fn()
        native.check(lib.dnh_event_record(e1, None))
        native.check(lib.dnh_event_sync(e1))
        ms = C.c_float()
        native.check(lib.dnh_event_elapsed_ms(e0, e1, C.byref(ms)))
        return ms.value / args.reps * 1e3

    def fills(shape):
        yield "zeros", np.zeros(shape, np.float32)
        yield "ones", np.ones(shape, np.float32)
        yield "integers -3..3", rng.integers(-3, 4, shape).astype(np.float32)
        yield "random, exact in bf16", (rng.standard_normal(shape).astype(np.float32).view(np.uint32) & 0xFFFF0000).view(np.float32)
        yield "random normal", rng.standard_normal(shape).astype(np.float32)

    for spec in args.shapes.split(","):
        if "x" in spec:
            nb, n = (int(v) for v in spec.split("x"))
            shape, label, mnk = (nb, n, n), "%dx%d^3" % (nb, n), nb * n ** 3
        else:
            n = int(spec)
            shape, label, mnk = (n, n), "%d^3" % n, n ** 3
        out = G.zeros(shape, np.float32)
        for name, host in fills(shape):
            a, b = G.ofNumpy(host), G.ofNumpy(host)
            for parts in (1, 0):
                with native.option("dot_bf16x3", parts):
                    us = timed(lambda: out.FillDot(a, b))
                print(json.dumps({"shape": label, "operands": name, "kernel": "bf16 parts" if parts else "fp32 instruction",
                                  "us": round(us, 1), "effective_tflops": round(2 * mnk / us / 1e6, 1),
                                  "launches": args.warmup + args.reps}), flush=True)


if __name__ == "__main__":
    main()
