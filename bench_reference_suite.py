"""The reference's own operation benchmark on the HIP device.

Re-expresses Tensor/Tensor.Benchmark/Benchmark.fs:95-203 (Worker) and :205-317 (TensorBenchmark): every listed operation on
tensors of shape 1000x1000, 2000x2000 and 4000x4000 for bool, int32, int64, single and double, inputs drawn uniformly from
[-50, 50) and converted to the element type, each measurement = the frontend call (result allocation included) followed by a
device synchronisation, timed on the host clock.  The output is a CSV with the reference report's columns
(Method, Shape, Type, Dev, Mean [ms], StdDev [ms]) so that it can be laid beside
Tensor.Benchmark/Results/*/TensorBenchmark-report.csv; operations a device does not support are reported as NA, as there.

    python bench_reference_suite.py [--out FILE.csv] [--shapes 1000x1000,4000x4000] [--types single,int32] [--iters 10]
"""
import argparse
import sys
import time

import numpy as np

TYPES = {"bool": np.bool_, "int32": np.int32, "int64": np.int64, "single": np.float32, "double": np.float64}
METHODS = ["Zeros", "Ones", "Identity", "Arange", "Copy", "Negate", "Add", "Subtract", "Multiply", "Divide", "Power", "Modulo", "Dot",
           "Sgn", "Log", "Log10", "Exp", "Sin", "Cos", "Tan", "Asin", "Acos", "Atan", "Sinh", "Cosh", "Tanh", "Sqrt", "Ceiling", "Floor",
           "Round", "Truncate", "MaxElemwise", "MinElemwise", "SumAxis", "ProductAxis", "MaxAxis", "MinAxis", "ArgMaxAxis", "ArgMinAxis",
           "FindAxis", "MaskedGet", "MaskedSet", "Invert", "PseudoInvert", "SVD", "SymEigDec", "Equal", "NotEqual", "Less", "LessOrEqual",
           "Greater", "GreaterOrEqual", "Not", "And", "Or", "Xor", "CountTrueAxis", "AllAxis", "AnyAxis", "TrueIndices", "IfThenElse"]


class Worker:
    """Benchmark.fs:95-203: the operands are created once, every method creates (and drops) its result."""

    def __init__(self, G, dtype, shape):
        from deepnet_amd.tensor import Tensor
        self.T, self.G, self.dev, self.dtype, self.shape = Tensor, G, G.Dev, np.dtype(dtype), list(shape)
        self.lastAxis = len(shape) - 1
        self.nElems = int(np.prod(shape))
        rng = np.random.default_rng(123)

        def numbers():
            return (rng.random(shape) * 100.0 - 50.0).astype(self.dtype)

        def bools():
            return rng.random(shape) >= 0.5

        self.is_bool = self.dtype == np.bool_
        self.a = G.ofNumpy(bools() if self.is_bool else numbers())
        self.b = G.ofNumpy(bools() if self.is_bool else numbers())
        self.p = G.ofNumpy(bools())
        self.q = G.ofNumpy(bools())
        self.maskedSetTarget = Tensor.zeros(self.shape, self.dev, self.dtype)
        self.maskedSetElems = self.a.M(self.p)

    def _ensure_bool(self):
        if not self.is_bool:
            raise NotImplementedError("Operation only supported for boolean data type.")

    def Zeros(self): self.T.zeros(self.shape, self.dev, self.dtype)
    def Ones(self): self.T.ones(self.shape, self.dev, self.dtype)
    def Identity(self): self.T.identity(self.shape[0], self.dev, self.dtype)
    def Arange(self): self.T.arange(0, 1, self.nElems, self.dev, self.dtype)
    def Copy(self): self.a.Copy()
    def Negate(self): -self.a
    def Add(self): self.a + self.b
    def Subtract(self): self.a - self.b
    def Multiply(self): self.a * self.b
    def Divide(self): self.a / self.b
    def Power(self): self.a ** self.b
    def Modulo(self): self.a % self.b
    def Dot(self): self.a @ self.b
    def Sgn(self): self.a.sgn()
    def Log(self): self.a.log()
    def Log10(self): self.a.log10()
    def Exp(self): self.a.exp()
    def Sin(self): self.a.sin()
    def Cos(self): self.a.cos()
    def Tan(self): self.a.tan()
    def Asin(self): self.a.asin()
    def Acos(self): self.a.acos()
    def Atan(self): self.a.atan()
    def Sinh(self): self.a.sinh()
    def Cosh(self): self.a.cosh()
    def Tanh(self): self.a.tanh()
    def Sqrt(self): self.a.sqrt()
    def Ceiling(self): self.a.ceiling()
    def Floor(self): self.a.floor()
    def Round(self): self.a.round()
    def Truncate(self): self.a.truncate()
    def MaxElemwise(self): self.T.maxElemwise(self.a, self.b)
    def MinElemwise(self): self.T.minElemwise(self.a, self.b)
    def Equal(self): self.a == self.b
    def NotEqual(self): self.a != self.b
    def Less(self): self.a < self.b
    def LessOrEqual(self): self.a <= self.b
    def Greater(self): self.a > self.b
    def GreaterOrEqual(self): self.a >= self.b
    def IfThenElse(self): self.T.ifThenElse(self.p, self.a, self.b)
    def SumAxis(self): self.a.sumAxis(self.lastAxis)
    def ProductAxis(self): self.a.productAxis(self.lastAxis)
    def MaxAxis(self): self.a.maxAxis(self.lastAxis)
    def MinAxis(self): self.a.minAxis(self.lastAxis)
    def ArgMaxAxis(self): self.a.argMaxAxis(self.lastAxis)
    def ArgMinAxis(self): self.a.argMinAxis(self.lastAxis)
    def FindAxis(self): self.a.findAxis(self.dtype.type(0), self.lastAxis)
    def MaskedGet(self): self.a.M(self.p)
    def MaskedSet(self): self.maskedSetTarget.setM([self.p], self.maskedSetElems)
    def Invert(self): self.T.invert(self.a)
    def PseudoInvert(self): self.T.pseudoInvert(self.a)
    def SVD(self): self.T.SVD(self.a)
    def SymEigDec(self): self.T.symmetricEigenDecomposition("Upper", self.a)
    def Not(self): self._ensure_bool(); ~self.p
    def And(self): self._ensure_bool(); self.p & self.q
    def Or(self): self._ensure_bool(); self.p | self.q
    def Xor(self): self._ensure_bool(); self.p ^ self.q
    def CountTrueAxis(self): self._ensure_bool(); self.p.countTrueAxis(self.lastAxis)
    def AllAxis(self): self._ensure_bool(); self.p.allAxis(self.lastAxis)
    def AnyAxis(self): self._ensure_bool(); self.p.anyAxis(self.lastAxis)
    def TrueIndices(self): self._ensure_bool(); self.p.trueIdx()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", default="-")
    ap.add_argument("--shapes", default="1000x1000,2000x2000,4000x4000")
    ap.add_argument("--types", default="bool,int32,int64,single,double")
    ap.add_argument("--methods", default=",".join(METHODS))
    ap.add_argument("--iters", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    args = ap.parse_args()

    from deepnet_amd import hip as G, native
    native.check(native.load().dnh_init(0))
    out = sys.stdout if args.out == "-" else open(args.out, "w")
    out.write("Method,Shape,Type,Dev,Mean [ms],StdDev [ms]\n")
    for shape_s in args.shapes.split(","):
        shape = [int(x) for x in shape_s.split("x")]
        for tname in args.types.split(","):
            w = Worker(G, TYPES[tname], shape)
            G.synchronize()
            for m in args.methods.split(","):
                fn = getattr(w, m)
                try:
                    for _ in range(args.warmup):
                        fn()
                    G.synchronize()
                    ts = []
                    for _ in range(args.iters):
                        t0 = time.perf_counter()
                        fn()
                        G.synchronize()
                        ts.append((time.perf_counter() - t0) * 1e3)
                    out.write(f"{m},{shape_s},{tname},Hip,{np.mean(ts):.4f},{np.std(ts):.4f}\n")
                except (NotImplementedError, ValueError, TypeError, ArithmeticError):
                    out.write(f"{m},{shape_s},{tname},Hip,NA,NA\n")
                    G.synchronize()
                out.flush()
            del w
    if out is not sys.stdout:
        out.close()


if __name__ == "__main__":
    main()
