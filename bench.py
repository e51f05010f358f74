#!/usr/bin/env python3
"""bench.py — headline benchmark of the HIP tensor backend on one MI355X.

Metric: achieved HBM GB/s (% of peak) for fp32 element-wise + axis-reduce at 64 Mi elements.

A "step" is one pass of the hot path over one batch of synthetic fp32 tensors of 8192 x 8192 = 67 108 864 elements
already resident in HBM: Add and Tanh (element-wise) and Sum / Max / ArgMax along the last axis and along the first
axis plus a full-tensor Sum (reductions) — nine backend calls through the C ABI, each into a preallocated target.
`value` = algorithmic bytes of the step (each distinct input read once + output written once) / step time.
Every op's launches are bracketed by HIP events on the stream they run on; the `roofline` object is the op that takes
the largest share of the step.  Consecutive ops read different 256 MiB tensors so the 256 MB Infinity Cache cannot
serve re-reads.  `cpu_baseline` times the CPU oracle (oracle/hostref.cpp, the HostTensor restatement) on the same step.
`configs` carries the other benchmark configurations (element-wise chain, permuted + broadcast add, double-precision
folds, integer / bool indexing, batched dot + softmax pieces): one entry per backend call with its algorithmic bytes or
FLOPs, the mean of >= 20 event-timed launches over rotated buffer sets and the fraction of 8 TB/s or, for a product, the flop
its kernel issues over the dense peak of the matrix instruction it issues them on (single-precision products are timed on both
of their kernels: bf16 matrix instruction with three parts per float, and fp32 matrix instruction); `config_summary` aggregates
them per configuration.  They are measured after the timed region.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-configs] [--all] [--no-cpu]
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, vendor figure
FP32_MFMA_PEAK_TFLOPS = 157.3
# HBM bytes per launch of the dominant kernel are not measured by this program: they come from two rocprofv3 --pmc runs of it
# (FETCH_SIZE, WRITE_SIZE), whose committed summary carries a line
#   traffic_bytes_per_launch <op> <bytes> kernel=<kernel symbol without blanks> sources=<sha256[:16] of the kernel's source files>
# The figure is reported only while it still describes the kernel this program times: same kernel symbol, same source text.
TRAFFIC_PROFILE = os.path.join("profiles", "bench_headline_fp32_8192x8192.txt")
KERNEL_SOURCES = {   # op -> the files whose text makes up its kernel
    "Add": ["deepnet_amd/csrc/map_kernels.h", "deepnet_amd/csrc/ops.h", "deepnet_amd/csrc/elemwise_binary.hip"],
}


def kernel_source_hash(op_name):
    import hashlib
    h = hashlib.sha256()
    for rel in KERNEL_SOURCES.get(op_name, []):
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def profiled_traffic(op_name, kernel_symbol):
    """(bytes, source file, note) of the committed counter summary for `op_name`; bytes is None when there is no summary or when
    it was taken from another kernel or another version of the kernel's sources (the note then says which)."""
    try:
        with open(os.path.join(ROOT, TRAFFIC_PROFILE)) as f:
            for line in f:
                parts = line.split()
                if len(parts) >= 3 and parts[0] == "traffic_bytes_per_launch" and parts[1] == op_name:
                    tags = dict(p.split("=", 1) for p in parts[3:] if "=" in p)
                    if tags.get("kernel") != kernel_symbol.replace(" ", ""):
                        return None, TRAFFIC_PROFILE, f"stale: profiled kernel {tags.get('kernel')} is not {kernel_symbol}"
                    if tags.get("sources") != kernel_source_hash(op_name):
                        return None, TRAFFIC_PROFILE, "stale: the kernel's source files changed after the counters were read"
                    return int(parts[2]), TRAFFIC_PROFILE, None
    except OSError:
        pass
    return None, None, "no committed counter summary"


def log(*a):
    print(*a, file=sys.stderr, flush=True)


class Op:
    """One backend call with prebuilt descriptors: fn(lib_or_oracle) issues it; `bytes` is its algorithmic traffic."""

    def __init__(self, name, kernel, entry, args, nbytes, flops=0, symbol=None):
        self.name, self.kernel, self.entry, self.args, self.bytes, self.flops = name, kernel, entry, args, nbytes, flops
        self.symbol = symbol or kernel   # the kernel's symbol as rocprofv3 prints it
        self.ms = []
        self.timed_ms = []


def desc_of(t):
    from deepnet_amd.backend import CAbiTensorBackend
    return CAbiTensorBackend._desc(t)


def make_ops(mod, rng_seed=123, n=8192):
    """Builds the step's tensors on device module `mod` (hip or hostref) and the list of backend calls."""
    from deepnet_amd import abi
    from deepnet_amd.tensor import Tensor
    rng = np.random.default_rng(rng_seed)
    N = n * n
    host = [rng.standard_normal((n, n), dtype=np.float32) for _ in range(3)]
    a, b, x = (mod.ofNumpy(h) for h in host)
    del host
    dev = a.Dev
    f32 = np.float32
    out_add = Tensor.new([n, n], dev, f32)
    out_tanh = Tensor.new([n, n], dev, f32)
    vec = [Tensor.new([n], dev, f32) for _ in range(4)]
    ivec = [Tensor.new([n], dev, np.int64) for _ in range(2)]
    scal = Tensor.new([], dev, f32)
    keep = [a, b, x, out_add, out_tanh, vec, ivec, scal]

    def D(t):
        d = desc_of(t)
        keep.append(d)
        return C.byref(d)

    def col(t):  # "along the first axis": the frontend permutes the reduced axis last as a view
        return t.permuteAxes([1, 0])

    s4 = 4
    ops = [
        Op("Add", "map_flat", "binary", (abi.DNH_ADD, D(out_add), D(a), D(b)), 3 * N * s4, symbol="map_flat_kernel<OpAdd<float>, 4, 1>"),
        Op("Tanh", "map_flat", "unary", (abi.DNH_TANH, D(out_tanh), D(x)), 2 * N * s4),
        Op("SumLastAxis(rows)", "reduce_rows", "reduce_last_axis", (abi.DNH_SUM, D(vec[0]), D(a)), N * s4 + n * s4),
        Op("MaxLastAxis(rows)", "reduce_rows", "reduce_last_axis", (abi.DNH_MAX, D(vec[1]), D(b)), N * s4 + n * s4),
        Op("ArgMaxLastAxis(rows)", "reduce_rows", "arg_reduce_last_axis", (abi.DNH_ARG_MAX, D(ivec[0]), D(x)), N * s4 + n * 8),
        Op("SumFirstAxis(cols)", "reduce_cols", "reduce_last_axis", (abi.DNH_SUM, D(vec[2]), D(col(a))), N * s4 + n * s4),
        Op("MaxFirstAxis(cols)", "reduce_cols", "reduce_last_axis", (abi.DNH_MAX, D(vec[3]), D(col(b))), N * s4 + n * s4),
        Op("ArgMaxFirstAxis(cols)", "reduce_cols", "arg_reduce_last_axis", (abi.DNH_ARG_MAX, D(ivec[1]), D(col(x))), N * s4 + n * 8),
        Op("Sum(full)", "reduce_rows", "reduce_last_axis", (abi.DNH_SUM, D(scal), D(a.flatten())), N * s4 + s4),
    ]
    return ops, keep


def run_gpu(steps, warmup):
    from deepnet_amd import hip as G, native
    lib = native.load()
    native.check(lib.dnh_init(0))
    info = G.Dev.Info()
    log(f"[bench] device: {info.name.decode()} ({info.arch.decode()}), {info.compute_units} CUs, "
        f"{info.total_memory_bytes / 2**30:.0f} GiB")
    ops, keep = make_ops(G)
    stream = C.c_void_p(0)

    def issue(op):
        native.check(getattr(lib, "dnh_" + op.entry)(*op.args, stream))

    def new_event():
        e = C.c_void_p()
        native.check(lib.dnh_event_create(C.byref(e)))
        return e

    def elapsed(e0, e1):
        ms = C.c_float()
        native.check(lib.dnh_event_elapsed_ms(e0, e1, C.byref(ms)))
        return ms.value

    # one plain contiguous copy of a known size (2 x 256 MiB of traffic): the reference kernel hardware-counter runs
    # (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE) are scaled by; it is outside the timed region
    native.check(lib.dnh_copy(ops[0].args[1], ops[0].args[2], stream))
    for _ in range(warmup):
        for op in ops:
            issue(op)

    # The timed region: K steps between two synchronisations.  Only the dominant kernel (Add: the most bytes of the step)
    # is bracketed by events inside it; an event pair costs a few microseconds of GPU idle time, which would otherwise
    # be charged once per op to a step of ~0.55 ms.
    dom = max(range(len(ops)), key=lambda i: ops[i].bytes)
    ev = [(new_event(), new_event()) for _ in range(steps)]
    native.check(lib.dnh_device_sync())
    t0 = time.perf_counter()
    for s in range(steps):
        for i, op in enumerate(ops):
            if i == dom:
                native.check(lib.dnh_event_record(ev[s][0], stream))
                issue(op)
                native.check(lib.dnh_event_record(ev[s][1], stream))
            else:
                issue(op)
    native.check(lib.dnh_device_sync())
    wall = time.perf_counter() - t0
    ops[dom].timed_ms = [elapsed(e0, e1) for e0, e1 in ev]

    # Per-op pass (outside the timed region): the same steps with every op bracketed, for the per-kernel table.
    nev = len(ops) + 1
    pev = [[new_event() for _ in range(nev)] for _ in range(steps)]
    for s in range(steps):
        native.check(lib.dnh_event_record(pev[s][0], stream))
        for i, op in enumerate(ops):
            issue(op)
            native.check(lib.dnh_event_record(pev[s][i + 1], stream))
    native.check(lib.dnh_device_sync())
    for s in range(steps):
        for i, op in enumerate(ops):
            op.ms.append(elapsed(pev[s][i], pev[s][i + 1]))
    for pair in ev:
        for e in pair:
            lib.dnh_event_destroy(e)
    for row in pev:
        for e in row:
            lib.dnh_event_destroy(e)
    del keep
    return ops, wall, info, dom


def run_cpu(repeats=1):
    """The oracle on the host cores: the same nine calls, once (plus one warm-up of the cheap ones)."""
    from oracle import hostref as H
    lib = H.load()
    ops, keep = make_ops(H)
    t_total = 0.0
    per = {}
    for op in ops:
        fn = getattr(lib, "href_" + op.entry)
        best = None
        for _ in range(repeats):
            t0 = time.perf_counter()
            st = fn(*op.args)
            dt = time.perf_counter() - t0
            assert st == 0, (op.name, st)
            best = dt if best is None else min(best, dt)
        per[op.name] = best
        t_total += best
    total_bytes = sum(op.bytes for op in ops)
    del keep
    return total_bytes / t_total / 1e9, H.get_threads(), per


def run_configs(everything):
    """The other benchmark configurations (not the headline): per-call lines and per-configuration sums."""
    import bench_configs
    if everything:
        res = bench_configs.run_all(log, (1, 2, 3, 4, 5, 6, 7))
    else:
        res = bench_configs.run_all(log, (1, 2, 3, 4, 5), fp32_folds=False, reference_dot_shapes=False)
    return res, bench_configs.summarise([r for r in res if r["cfg"] <= 5])


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-configs", action="store_true", help="skip the per-configuration lines (`configs` in the JSON)")
    ap.add_argument("--all", action="store_true", help="configurations: also the fp32 folds again, the reference's square products, "
                                                       "the vector forms of dot and host transfers")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this backend is single-GPU (the reference has no multi-device path); run with --gpus 1")
        sys.exit(2)

    ops, wall, info, dom_i = run_gpu(args.steps, args.warmup)
    total_bytes = sum(op.bytes for op in ops)
    ms_per_step = wall / args.steps * 1e3
    value = total_bytes / (wall / args.steps) / 1e9

    per_kernel = []
    for op in ops:
        avg = float(np.mean(op.ms))
        per_kernel.append({"op": op.name, "kernel": op.kernel, "avg_ms": round(avg, 5), "min_ms": round(float(np.min(op.ms)), 5),
                           "bytes": op.bytes, "GBps": round(op.bytes / (avg * 1e-3) / 1e9, 1),
                           "frac_of_peak": round(op.bytes / (avg * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)})
        log(f"[bench] {op.name:24s} {avg * 1e3:9.1f} us  {per_kernel[-1]['GBps']:8.1f} GB/s  {100 * per_kernel[-1]['frac_of_peak']:5.1f}% of HBM peak")
    dop = ops[dom_i]
    dom_ms = float(np.mean(dop.timed_ms))
    dom_gbs = dop.bytes / (dom_ms * 1e-3) / 1e9
    traffic, traffic_src, traffic_note = profiled_traffic(dop.name, dop.symbol)
    roofline = {"bound": "hbm", "kernel": dop.symbol, "op": dop.name, "achieved": round(dom_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(dom_gbs / HBM_PEAK_GBS, 4), "traffic": traffic, "traffic_source": traffic_src,
                "avg_launch_ms": round(dom_ms, 5), "algorithmic_bytes": dop.bytes}
    if traffic_note:
        roofline["traffic_note"] = traffic_note
        log(f"[bench] roofline.traffic withheld ({traffic_note})")
    ev_sum = sum(k["avg_ms"] for k in per_kernel)
    log(f"[bench] step: {ms_per_step:.3f} ms wall, {ev_sum:.3f} ms sum of event intervals, {value:.1f} GB/s = {100 * value / HBM_PEAK_GBS:.1f}% of HBM peak")

    cpu = None
    if not args.no_cpu:
        v, cores, per = run_cpu()
        cpu = {"value": round(v, 2), "unit": "GB/s", "cores": cores, "kind": "port",
               "sample": "the same nine calls at the full 8192x8192 fp32 size, each run once on the HostTensor-equivalent C++ oracle "
                         "(SIMD-list ops single-threaded, others threaded over dimension 0, folds sequential)"}
        for k, t in per.items():
            log(f"[bench] cpu {k:24s} {t * 1e3:9.1f} ms")

    configs, config_summary = (None, None) if args.no_configs else run_configs(args.all)

    print(json.dumps({
        "metric": "achieved HBM GB/s for fp32 elementwise + axis-reduce at 64M elems",
        "value": round(value, 1), "unit": "GB/s", "pct_of_peak": round(100 * value / HBM_PEAK_GBS, 2),
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "fp32 8192x8192 (64Mi elems): Add, Tanh, Sum/Max/ArgMax along last axis and along first axis, full Sum; "
                               "inputs resident in HBM, targets preallocated, seed 123",
                   "bytes_per_step": total_bytes, "device": info.name.decode() or info.arch.decode()},
        "roofline": roofline, "cpu_baseline": cpu, "per_kernel": per_kernel,
        "config_summary": config_summary, "configs": configs,
    }))


if __name__ == "__main__":
    main()
