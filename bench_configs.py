"""Per-configuration timings of the HIP backend (used by `bench.py`, which puts them into its JSON line): the five synthetic workloads of the
benchmark definition, one line per backend call with its algorithmic bytes (or FLOPs), HIP-event time and fraction of
the roofline that bounds it.  Inputs come from seed 123; an op whose working set is below ~600 MB is launched over
several independent buffer sets in rotation so that the 256 MB Infinity Cache cannot serve re-reads."""
import ctypes as C
import math

import numpy as np

HBM_PEAK_GBS = 8000.0
FP32_MFMA_PEAK_TFLOPS = 157.3
FP64_MFMA_PEAK_TFLOPS = 78.6
BF16_MFMA_PEAK_TFLOPS = 2500.0


class Timer:
    def __init__(self):
        from deepnet_amd import native
        self.native = native
        self.lib = native.load()
        self.stream = C.c_void_p(0)
        self.e0, self.e1 = C.c_void_p(), C.c_void_p()
        native.check(self.lib.dnh_event_create(C.byref(self.e0)))
        native.check(self.lib.dnh_event_create(C.byref(self.e1)))

    def issue(self, call):
        entry, args = call
        self.native.check(getattr(self.lib, "dnh_" + entry)(*args, self.stream))

    def time(self, sets, reps=20, warm=10):
        """sets: list of call lists (one list of (entry, args) per buffer set).  Returns average ms per pass over one set."""
        lib, check = self.lib, self.native.check
        for i in range(warm):
            for call in sets[i % len(sets)]:
                self.issue(call)
        check(lib.dnh_device_sync())
        check(lib.dnh_event_record(self.e0, self.stream))
        for i in range(reps):
            for call in sets[i % len(sets)]:
                self.issue(call)
        check(lib.dnh_event_record(self.e1, self.stream))
        check(lib.dnh_event_sync(self.e1))
        ms = C.c_float()
        check(lib.dnh_event_elapsed_ms(self.e0, self.e1, C.byref(ms)))
        return ms.value / reps


def nsets_for(nbytes):
    return max(1, min(40, math.ceil(600e6 / max(nbytes, 1))))


def profiled_call_traffic(tag):
    """HBM bytes one call moves according to the committed hardware-counter summary (`traffic_bytes_per_call <tag> <bytes>` lines of
    profiles/configs_all_kernels.txt), or None.  Used for the calls whose traffic is far from their algorithmic bytes."""
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "configs_all_kernels.txt")
    try:
        with open(path) as f:
            for line in f:
                parts = line.split()
                if len(parts) == 3 and parts[0] == "traffic_bytes_per_call" and parts[1] == tag:
                    return int(parts[2])
    except OSError:
        pass
    return None


# The matrix pipes a dot kernel can run on: MI355X's dense peak of the instruction the kernel issues, and how many flop it issues
# per algorithmic flop (the bf16-parts kernels form six bf16 products per multiply-add of the fp32 product).
MFMA_PIPES = {
    "bf16x3": {"kernel": "gemm_bf16x3_kernel / gemm_bf16x3_big_kernel", "instruction": "v_mfma_f32_32x32x16_bf16", "peak_TFLOPs": BF16_MFMA_PEAK_TFLOPS, "issue": 6},
    "fp32": {"kernel": "gemm_kernel<float>", "instruction": "v_mfma_f32_32x32x2_f32", "peak_TFLOPs": FP32_MFMA_PEAK_TFLOPS, "issue": 1},
    "fp64": {"kernel": "gemm_f64_kernel", "instruction": "v_mfma_f64_16x16x4_f64", "peak_TFLOPs": FP64_MFMA_PEAK_TFLOPS, "issue": 1},
}


def report(log, cfg, name, ms, nbytes=None, flops=None, pipe=None):
    """One line of the per-configuration table.  `frac` is the fraction of the roofline that bounds the call: 8 TB/s of HBM for
    algorithmic bytes, or, for a product, the flop its kernel issues over the dense peak of the matrix instruction it issues them on
    (`pipe`).  The product's own rate (2 M N K over time) is reported beside it, with its ratio to the fp32 matrix peak for
    single-precision products whatever instruction computed them."""
    if flops:
        p = MFMA_PIPES[pipe]
        tf = flops / (ms * 1e-3) / 1e12
        issued = flops * p["issue"]
        tf_issued = issued / (ms * 1e-3) / 1e12
        frac = tf_issued / p["peak_TFLOPs"]
        row = {"cfg": cfg, "op": name, "us": round(ms * 1e3, 2), "flops": int(flops), "TFLOPs": round(tf, 2), "bound": "mfma",
               "kernel": p["kernel"], "instruction": p["instruction"], "flops_issued": int(issued), "issued_TFLOPs": round(tf_issued, 1),
               "peak_TFLOPs": p["peak_TFLOPs"], "frac": round(frac, 4)}
        extra = ""
        if pipe in ("bf16x3", "fp32"):
            row["x_fp32_mfma_peak"] = round(tf / FP32_MFMA_PEAK_TFLOPS, 4)   # a speed figure, not a roofline fraction
            extra = f"  (product rate = {tf / FP32_MFMA_PEAK_TFLOPS:4.2f} x fp32 MFMA peak)"
        log(f"[cfg{cfg}] {name:38s} {ms * 1e3:9.1f} us  {tf:7.2f} TFLOP/s  issues {tf_issued:7.1f} TFLOP/s on {p['instruction']} = "
            f"{100 * frac:5.1f}% of its {p['peak_TFLOPs']:.1f} peak{extra}")
        return row
    gb = nbytes / (ms * 1e-3) / 1e9
    log(f"[cfg{cfg}] {name:34s} {ms * 1e3:9.1f} us  {gb:8.1f} GB/s  {100 * gb / HBM_PEAK_GBS:5.1f}% of HBM peak  ({nbytes / 1e6:.1f} MB)")
    row = {"cfg": cfg, "op": name, "us": round(ms * 1e3, 2), "bytes": int(nbytes), "GBps": round(gb, 1), "bound": "hbm", "frac": round(gb / HBM_PEAK_GBS, 4)}
    # gather / scatter move far more than their algorithmic bytes (a cache line per random 4-byte access): the counter-measured
    # traffic of the call and the rate it stands for are reported beside the algorithmic figures
    tag = ("Gather" if name.startswith("Gather") else "Scatter" if "Scatter" in name else None) if cfg == 4 else None
    traffic = profiled_call_traffic(tag) if tag else None
    if traffic:
        row.update({"traffic_bytes": traffic, "traffic_GBps": round(traffic / (ms * 1e-3) / 1e9, 1),
                    "traffic_frac": round(traffic / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "traffic_source": "profiles/configs_all_kernels.txt"})
        log(f"       (counter-measured traffic of this call {traffic / 1e6:.1f} MB = {traffic / (ms * 1e-3) / 1e9:.0f} GB/s = {100 * traffic / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS:.1f}% of HBM peak)")
    return row


def summarise(results):
    """Per configuration: sum of algorithmic bytes over sum of time of its memory-bound calls (the composite lines — the eager
    chain, which repeats the six calls above it — are left out), and the lowest fraction among all of its calls."""
    out = []
    for cfg in sorted({r["cfg"] for r in results}):
        rows = [r for r in results if r["cfg"] == cfg and "frac" in r]
        mem = [r for r in rows if r.get("bound") == "hbm" and not r.get("composite")]
        entry = {"cfg": cfg, "calls": len(rows), "min_frac": min(r["frac"] for r in rows) if rows else None}
        if mem:
            gb = sum(r["bytes"] for r in mem) / sum(r["us"] for r in mem) / 1e3
            entry.update({"hbm_bytes": sum(r["bytes"] for r in mem), "hbm_us": round(sum(r["us"] for r in mem), 1), "GBps": round(gb, 1),
                          "frac": round(gb / HBM_PEAK_GBS, 4)})
        out.append(entry)
    return out


def run_all(log, which=(1, 2, 3, 4, 5, 6), fp32_folds=True, reference_dot_shapes=True):
    """fp32_folds=False leaves configuration 3's single-precision folds out (bench.py's headline step times those);
    reference_dot_shapes=False leaves out the 1000 / 2000 / 4000 square products of the reference's own benchmark."""
    from deepnet_amd import abi, hip as G
    from deepnet_amd.backend import CAbiTensorBackend
    from deepnet_amd.tensor import Tensor
    T = Timer()
    rng = np.random.default_rng(123)
    keep = []
    results = []

    def D(t):
        d = CAbiTensorBackend._desc(t)
        keep.append((t, d))
        return C.byref(d)

    def new(shape, dt):
        return Tensor.new(shape, G.Dev, dt)

    def timed(cfg, name, nbytes, build, flops=None, reps=20, pipe=None):
        ns = nsets_for(nbytes)
        sets = [build(i) for i in range(ns)]
        ms = T.time(sets, reps=max(reps, ns))
        results.append(report(log, cfg, name, ms, nbytes, flops, pipe))
        keep.clear()

    def timed_dot(cfg, name, nbytes, build, flops, dt):
        """A product of single-precision operands is timed on both of its kernels: the default (bf16 matrix instruction, three parts
        per float) and, behind the library's switch, the fp32 matrix instruction."""
        if dt is np.float64:
            timed(cfg, name, nbytes, build, flops=flops, pipe="fp64")
            return
        timed(cfg, name + " [bf16 parts]", nbytes, build, flops=flops, pipe="bf16x3")
        with T.native.option("dot_bf16x3", 0):
            timed(cfg, name + " [fp32 instr]", nbytes, build, flops=flops, pipe="fp32")

    f32 = np.float32
    if 1 in which:
        n = 4096
        N = n * n
        base = [rng.uniform(-1, 1, (n, n)).astype(f32) for _ in range(3)]

        def chain_set(i):
            a, b, c = (G.ofNumpy(x) for x in base)
            t1, t2, y, t3, t4, out = (new([n, n], f32) for _ in range(6))
            return [("binary", (abi.DNH_MULTIPLY, D(t1), D(a), D(b))), ("binary", (abi.DNH_ADD, D(t2), D(t1), D(c))),
                    ("unary", (abi.DNH_TANH, D(y), D(t2))), ("binary", (abi.DNH_MULTIPLY, D(t3), D(y), D(y))),
                    ("unary", (abi.DNH_UNARY_MINUS, D(t4), D(t3))), ("unary", (abi.DNH_EXP, D(out), D(t4)))]
        names = [("Multiply a*b", 3), ("Add t1+c", 3), ("Tanh", 2), ("Multiply y*y", 2), ("UnaryMinus", 2), ("Exp", 2)]
        sets = [chain_set(i) for i in range(4)]
        for k, (nm, mult) in enumerate(names):
            ms = T.time([[s[k]] for s in sets], reps=20)
            results.append(report(log, 1, nm + " 4096x4096", ms, mult * N * 4))
        ms = T.time(sets, reps=12)
        results.append(dict(report(log, 1, "chain of 6 calls (eager)", ms, 14 * N * 4), composite=True))
        keep.clear()
        del sets

    if 2 in which:
        x = G.ofNumpy(rng.standard_normal((256, 512, 1024), dtype=f32))
        v = G.ofNumpy(rng.random(1024, dtype=f32))
        N = 256 * 512 * 1024
        xp = x.permuteAxes([2, 0, 1])                       # shape [512, 1024, 256], strides [1024, 1, 524288]
        vb = v[None, :, None].broadcastTo(xp.Shape)         # strides [0, 1, 0]
        y = new(xp.Shape, f32)
        timed(2, "Add permuted x + broadcast v", 2 * N * 4 + 4096, lambda i: [("binary", (abi.DNH_ADD, D(y), D(xp), D(vb)))], reps=10)
        timed(2, "Copy permuted x -> contiguous", 2 * N * 4, lambda i: [("copy", (D(y), D(xp)))], reps=10)
        # the NumPy reading of "axes (2,0,1)": shape [1024, 256, 512], strides [1, 524288, 1024]
        xq = x.permuteAxes([1, 2, 0])
        vq = v[:, None, None].broadcastTo(xq.Shape)
        yq = new(xq.Shape, f32)
        timed(2, "Add (NumPy-convention permute)", 2 * N * 4 + 4096, lambda i: [("binary", (abi.DNH_ADD, D(yq), D(xq), D(vq)))], reps=10)
        del x, v, xp, vb, y, xq, vq, yq

    if 3 in which:
        n = 8192
        N = n * n
        for dt, s in ((np.float32, 4), (np.float64, 8)):
            if dt == np.float32 and not fp32_folds:
                continue
            a = G.ofNumpy(rng.standard_normal((n, n)).astype(dt) if dt == np.float32 else rng.uniform(-1, 1, (n, n)))
            b = G.ofNumpy(G.toNumpy(a) * dt(0.5))
            srcs = [a, b]
            vec = new([n], dt)
            ivec = new([n], np.int64)
            sc = new([], dt)
            nm = np.dtype(dt).name
            for label, view in (("last axis", lambda t: t), ("first axis", lambda t: t.permuteAxes([1, 0]))):
                timed(3, f"Sum {label} {nm}", N * s + n * s, lambda i: [("reduce_last_axis", (abi.DNH_SUM, D(vec), D(view(srcs[i % 2]))))])
                timed(3, f"Max {label} {nm}", N * s + n * s, lambda i: [("reduce_last_axis", (abi.DNH_MAX, D(vec), D(view(srcs[i % 2]))))])
                timed(3, f"ArgMax {label} {nm}", N * s + n * 8, lambda i: [("arg_reduce_last_axis", (abi.DNH_ARG_MAX, D(ivec), D(view(srcs[i % 2]))))])
            timed(3, f"Sum full {nm}", N * s + s, lambda i: [("reduce_last_axis", (abi.DNH_SUM, D(sc), D(srcs[i % 2].flatten())))])
            del a, b, srcs

    if 4 in which:
        N, M = 1 << 24, 1 << 22
        ha = rng.integers(-1000, 1001, N).astype(np.int32)
        hb = rng.integers(-1000, 1001, N).astype(np.int32)
        hidx = rng.integers(0, N, M).astype(np.int64)
        hidxu = rng.permutation(N)[:M].astype(np.int64)
        K = int((ha > 0).sum())
        zero = G.scalar(0, np.int32)

        def mk():
            a, b = G.ofNumpy(ha), G.ofNumpy(hb)
            m = new([N], np.bool_)
            m.Backend.Greater(m, a, zero.broadcastTo([N]))
            return a, b, m
        timed(4, "Greater int32 > 0 -> bool", N * 4 + N + 4,
              lambda i: (lambda a, b, m: [("compare", (abi.DNH_GREATER, D(m), D(a), D(zero.broadcastTo([N]))))])(*mk()))
        timed(4, "IfThenElse bool,int32,int32", N + 3 * N * 4,
              lambda i: (lambda a, b, m: [("if_then_else", (D(new([N], np.int32)), D(m), D(a), D(b)))])(*mk()))
        cnt = new([], np.int64)
        timed(4, "CountTrue bool[16Mi]", N + 8,
              lambda i: (lambda a, b, m: [("reduce_last_axis", (abi.DNH_COUNT_TRUE, D(cnt), D(m)))])(*mk()))

        def mget(i):
            a, b, m = mk()
            arr = (C.POINTER(abi.DnhTensor) * 1)()
            dm = CAbiTensorBackend._desc(m)
            keep.append((m, dm, arr))
            arr[0] = C.pointer(dm)
            return [("masked_get", (D(new([K], np.int32)), D(a), arr, 1))]
        timed(4, "MaskedGet int32 by bool mask", 2 * N + N * 4 + K * 4, mget)

        def mset(i):
            a, b, m = mk()
            arr = (C.POINTER(abi.DnhTensor) * 1)()
            dm = CAbiTensorBackend._desc(m)
            keep.append((m, dm, arr))
            arr[0] = C.pointer(dm)
            return [("masked_set", (D(a), arr, 1, D(b[0:K])))]
        timed(4, "MaskedSet int32 by bool mask", 2 * N + K * 4 + K * 4, mset)
        timed(4, "TrueIndices bool[16Mi] -> [K,1]", 2 * N + K * 8,
              lambda i: (lambda a, b, m: [("true_indices", (D(new([K, 1], np.int64)), D(m)))])(*mk()))

        def gat(i):
            a = G.ofNumpy(ha)
            idx = G.ofNumpy(hidx)
            arr = (C.POINTER(abi.DnhTensor) * 1)()
            di = CAbiTensorBackend._desc(idx)
            keep.append((idx, di, arr))
            arr[0] = C.pointer(di)
            return [("gather", (D(new([M], np.int32)), arr, 1, D(a)))]
        timed(4, "Gather 4Mi int64 idx from 16Mi", M * 8 + M * 4 + M * 4, gat)

        def sca(i):
            src = G.ofNumpy(ha[:M])
            idx = G.ofNumpy(hidxu)
            t = new([N], np.int32)
            arr = (C.POINTER(abi.DnhTensor) * 1)()
            di = CAbiTensorBackend._desc(idx)
            z = np.zeros(1, np.int32)
            keep.append((idx, di, arr, z))
            arr[0] = C.pointer(di)
            return [("fill_const", (D(t), z.ctypes.data_as(C.c_void_p))), ("scatter", (D(t), arr, 1, D(src)))]
        timed(4, "FillConst 0 + Scatter (unique idx)", N * 4 + M * 8 + M * 4 + M * 4, sca)

    if 5 in which:
        Bn, n = 64, 512
        N = Bn * n * n
        R = Bn * n
        sd = 1.0 / math.sqrt(512.0)
        ha = (rng.standard_normal((Bn, n, n)) * sd).astype(f32)
        hb = (rng.standard_normal((Bn, n, n)) * sd).astype(f32)

        def mk5():
            return G.ofNumpy(ha), G.ofNumpy(hb), new([Bn, n, n], f32)
        timed_dot(5, "BatchedMatMatDot 64x512^3 fp32", 3 * N * 4, lambda i: (lambda a, b, c: [("dot", (D(c), D(a), D(b)))])(*mk5()),
                  2.0 * Bn * n ** 3, f32)
        timed(5, "Tanh [64,512,512]", 2 * N * 4, lambda i: (lambda a, b, c: [("unary", (abi.DNH_TANH, D(c), D(a)))])(*mk5()))
        timed(5, "MaxAxis 2 (rows of 512)", N * 4 + R * 4,
              lambda i: (lambda a, b, c: [("reduce_last_axis", (abi.DNH_MAX, D(new([Bn, n], f32)), D(a)))])(*mk5()))

        def sub5(i):
            a, b, c = mk5()
            mx = new([Bn, n], f32)
            mx.Backend.MaxLastAxis(mx, a)
            return [("binary", (abi.DNH_SUBTRACT, D(c), D(a), D(mx[:, :, None].broadcastTo([Bn, n, n]))))]
        timed(5, "Subtract t - rowmax (broadcast)", 2 * N * 4 + R * 4, sub5)
        timed(5, "Exp [64,512,512]", 2 * N * 4, lambda i: (lambda a, b, c: [("unary", (abi.DNH_EXP, D(c), D(a)))])(*mk5()))
        timed(5, "SumAxis 2 (rows of 512)", N * 4 + R * 4,
              lambda i: (lambda a, b, c: [("reduce_last_axis", (abi.DNH_SUM, D(new([Bn, n], f32)), D(a)))])(*mk5()))

        def div5(i):
            a, b, c = mk5()
            sm = new([Bn, n], f32)
            sm.Backend.SumLastAxis(sm, a)
            return [("binary", (abi.DNH_DIVIDE, D(c), D(a), D(sm[:, :, None].broadcastTo([Bn, n, n]))))]
        timed(5, "Divide e / rowsum (broadcast)", 2 * N * 4 + R * 4, div5)
        # the matrix sizes of the reference's own benchmark (Tensor.Benchmark/Benchmark.fs:216): few output tiles, K is split
        for sq in ((1000, 2000, 4000) if reference_dot_shapes else (4000,)):
            for dt, sz in ((np.float32, 4), (np.float64, 8)):
                sa = G.ofNumpy(rng.standard_normal((sq, sq)).astype(dt))
                sb = G.ofNumpy(rng.standard_normal((sq, sq)).astype(dt))
                sc = new([sq, sq], dt)
                timed_dot(5, f"MatMatDot {sq}^3 {np.dtype(dt).name}", 3 * sq * sq * sz, lambda i: [("dot", (D(sc), D(sa), D(sb)))],
                          2.0 * sq ** 3, dt)
                del sa, sb, sc
    if 6 in which:
        # the vector forms of dot (not one of the five configurations; bandwidth-bound)
        n = 8192
        for dt, sz in ((np.float32, 4), (np.float64, 8)):
            nm = np.dtype(dt).name
            mats = [G.ofNumpy(rng.standard_normal((n, n)).astype(dt)) for _ in range(3)]
            x = G.ofNumpy(rng.standard_normal(n).astype(dt))
            y = new([n], dt)
            timed(6, f"MatVecDot 8192x8192 {nm}", n * n * sz + 2 * n * sz, lambda i: [("dot", (D(y), D(mats[i % 3]), D(x)))])
            timed(6, f"MatVecDot transposed view {nm}", n * n * sz + 2 * n * sz, lambda i: [("dot", (D(y), D(mats[i % 3].T), D(x)))])
            u, v = (G.ofNumpy(rng.standard_normal(1 << 26).astype(dt)) for _ in range(2))
            r = new([], dt)
            timed(6, f"VecVecDot 64Mi {nm}", 2 * (1 << 26) * sz, lambda i: [("dot", (D(r), D(u), D(v)))])
            del mats, u, v
    if 7 in which:
        # the step either side of every benchmark: host <-> device copies of 256 MiB (wall clock, synchronous calls)
        import time
        lib, check = T.lib, T.native.check
        nbytes = 256 << 20
        dev = new([nbytes], np.uint8)
        dptr = dev.Storage.Pointer()
        pinned = C.c_void_p()
        check(lib.dnh_host_alloc(nbytes, C.byref(pinned)))
        C.memset(pinned, 1, nbytes)
        pageable = np.ones(nbytes, np.uint8)
        for kind, hptr in (("pinned", pinned.value), ("pageable", pageable.ctypes.data)):
            for name, call in (("H2D", lambda: lib.dnh_memcpy_h2d(dptr, hptr, nbytes, T.stream, 1)),
                               ("D2H", lambda: lib.dnh_memcpy_d2h(hptr, dptr, nbytes, T.stream, 1))):
                for _ in range(2):
                    check(call())
                t0 = time.perf_counter()
                for _ in range(5):
                    check(call())
                ms = (time.perf_counter() - t0) / 5 * 1e3
                log(f"[cfg7] {name} 256 MiB {kind:8s} host memory {ms:9.2f} ms  {nbytes / ms / 1e6:8.1f} GB/s")
                results.append({"cfg": 7, "op": f"{name} {kind}", "us": round(ms * 1e3, 1), "GBps": round(nbytes / ms / 1e6, 1)})
        check(lib.dnh_host_free(pinned))
    if 8 in which:
        # floating-point scatter with repeated indices (not one of the five configurations): the ordered form, which adds a cell's
        # sources in the reference's order, beside float atomics; 4 Mi sources into 16 Mi cells, uniform random indices
        N, M = 1 << 24, 1 << 22
        hidx = rng.integers(0, N, M).astype(np.int64)
        for dt, sz in ((np.float32, 4), (np.float64, 8)):
            hsrc = rng.standard_normal(M).astype(dt)

            def sca8(i):
                src = G.ofNumpy(hsrc)
                idx = G.ofNumpy(hidx)
                t = new([N], dt)
                arr = (C.POINTER(abi.DnhTensor) * 1)()
                di = CAbiTensorBackend._desc(idx)
                z = np.zeros(1, dt)
                keep.append((idx, di, arr, z))
                arr[0] = C.pointer(di)
                return [("fill_const", (D(t), z.ctypes.data_as(C.c_void_p))), ("scatter", (D(t), arr, 1, D(src)))]
            nm = np.dtype(dt).name
            timed(8, f"FillConst 0 + Scatter {nm} ordered", N * sz + M * 8 + M * sz + M * sz, sca8, reps=6)
            with T.native.option("scatter_fp_atomic", 1):
                timed(8, f"FillConst 0 + Scatter {nm} atomics", N * sz + M * 8 + M * sz + M * sz, sca8, reps=6)
    return results


if __name__ == "__main__":
    import sys
    which = tuple(int(x) for x in sys.argv[1:]) or (1, 2, 3, 4, 5, 6)
    run_all(lambda *a: print(*a, flush=True), which)
