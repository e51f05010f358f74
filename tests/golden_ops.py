"""Maps the `fn` names of tests/golden/reference_vectors.json to frontend call sequences (device-agnostic)."""
import json
import os

import numpy as np

from deepnet_amd import layout as L
from deepnet_amd.tensor import Tensor

HERE = os.path.dirname(os.path.abspath(__file__))


def load_vectors():
    with open(os.path.join(HERE, "golden", "reference_vectors.json")) as f:
        return json.load(f)["vectors"]


def to_array(spec):
    def conv(x):
        if isinstance(x, str):
            return float(x)
        if isinstance(x, list):
            return [conv(y) for y in x]
        return x
    return np.array(conv(spec["data"]), dtype=spec["dtype"])


def _fill_multiply_twice(f3, d, e):
    f3.FillMultiply(d, e)
    f3.FillMultiply(f3, e)
    return f3


def _mask_set(a, m, v):
    a.setM([m], v)
    return a


# tensor-valued ops: fn(*tensors_or_scalars)
OPS = {
    "add": lambda a, b: a + b, "sub": lambda a, b: a - b, "mul": lambda a, b: a * b, "div": lambda a, b: a / b,
    "mod": lambda a, b: a % b, "pow": lambda a, b: a ** b, "mul_scalar": lambda a, s: a * s,
    "fill_multiply_twice": _fill_multiply_twice, "dot": lambda a, b: a @ b,
    "sin": lambda a: a.sin(), "cos": lambda a: a.cos(), "tan": lambda a: a.tan(), "asin": lambda a: a.asin(), "acos": lambda a: a.acos(),
    "atan": lambda a: a.atan(), "sinh": lambda a: a.sinh(), "cosh": lambda a: a.cosh(), "tanh": lambda a: a.tanh(), "log": lambda a: a.log(),
    "log10": lambda a: a.log10(), "exp": lambda a: a.exp(), "sqrt": lambda a: a.sqrt(), "ceiling": lambda a: a.ceiling(),
    "floor": lambda a: a.floor(), "round": lambda a: a.round(), "truncate": lambda a: a.truncate(), "isFinite": lambda a: a.isFinite(),
    "pos": lambda a: +a, "neg": lambda a: -a, "abs": lambda a: abs(a), "sgn": lambda a: a.sgn(), "convert_f64": lambda a: a.convert(np.float64),
    "eq": lambda a, b: a == b, "ne": lambda a, b: a != b, "lt": lambda a, b: a < b, "le": lambda a, b: a <= b, "gt": lambda a, b: a > b,
    "ge": lambda a, b: a >= b, "not": lambda a: ~a, "and_not_self": lambda a: a & ~a, "and": lambda a, b: a & b, "or": lambda a, b: a | b,
    "xor": lambda a, b: a ^ b, "maxElemwise": lambda a, b: Tensor.maxElemwise(a, b), "minElemwise": lambda a, b: Tensor.minElemwise(a, b),
    "ifThenElse": lambda c, a, b: Tensor.ifThenElse(c, a, b),
    "sum": lambda a: a.sum(), "product": lambda a: a.product(), "min": lambda a: a.min(), "max": lambda a: a.max(),
    "sumAxis": lambda a, ax: a.sumAxis(ax), "productAxis": lambda a, ax: a.productAxis(ax), "minAxis": lambda a, ax: a.minAxis(ax),
    "maxAxis": lambda a, ax: a.maxAxis(ax), "allAxis": lambda a, ax: a.allAxis(ax), "all": lambda a: a.all(),
    "countTrueAxis": lambda a, ax: a.countTrueAxis(ax), "countTrue": lambda a: a.countTrue(), "trueIdx": lambda a: a.trueIdx(),
    "argMax": lambda a: a.argMax(), "argMaxAxis": lambda a, ax: a.argMaxAxis(ax), "argMinAxis": lambda a, ax: a.argMinAxis(ax),
    "tryFind": lambda a, v: a.tryFind(v), "findAxis": lambda a, v, ax: a.findAxis(v, ax),
    "gather2": lambda s, i0, i1: Tensor.gather([i0, i1], s), "gather_none_first": lambda s, j1: Tensor.gather([None, j1], s),
    "scatter2": lambda s, i0, i1, shp: Tensor.scatter([i0, i1], shp, s),
    "mask_get": lambda a, m: a.M(m), "mask_get_rows": lambda a, m0: a.M(m0, None), "mask_set": _mask_set,
    "reverse0": lambda a: a.reverseAxis(0).Copy(),
}

# pure layout algebra: fn(*plain args) -> plain value
LAYOUT_OPS = {
    "permute_shape": lambda shp, perm: list(L.permuteAxes(perm, L.newC(shp)).Shape),
    "swap_shape": lambda shp, a, b: list(L.swapDim(a, b, L.newC(shp)).Shape),
    "reshape_shape": lambda shp, new: list(L.reshape(new, L.newC(shp)).Shape),
    "broadcast_in_dims": lambda sa, sb, dims: [list(x.Shape) for x in L.broadcastToSameInDimsMany(dims, [L.newC(sa), L.newC(sb)])],
    "broadcast_to": lambda sa, shp: list(L.broadcastToShape(shp, L.newC(sa)).Shape),
    "pad_to_same": lambda sa, sb: [list(x.Shape) for x in L.padToSame(L.newC(sa), L.newC(sb))],
}


def run_vector(mod, vec):
    """Evaluates one vector on device module `mod`; returns (result, expected) as NumPy arrays or plain values."""
    fn = vec["fn"]
    if fn in LAYOUT_OPS:
        return LAYOUT_OPS[fn](*vec["args"]), vec["expect"]
    args = [mod.ofNumpy(to_array(a)) if isinstance(a, dict) else a for a in vec["args"]]
    out = OPS[fn](*args)
    if hasattr(out, "Layout"):
        out = mod.toNumpy(out)
    exp = vec["expect"]
    if isinstance(exp, dict):
        exp = to_array(exp)
    return out, exp


def check_vector(mod, vec):
    out, exp = run_vector(mod, vec)
    atol, rtol = vec.get("atol", 0.0), vec.get("rtol", 0.0)
    if isinstance(exp, np.ndarray):
        assert isinstance(out, np.ndarray), (vec["id"], type(out))
        assert out.dtype == exp.dtype, (vec["id"], out.dtype, exp.dtype)
        assert out.shape == exp.shape, (vec["id"], out.shape, exp.shape)
        if atol == 0 and rtol == 0:
            assert np.array_equal(out, exp), (vec["id"], out, exp)
        else:
            assert np.allclose(out, exp, rtol=rtol, atol=atol), (vec["id"], out, exp)
    elif isinstance(exp, (list, bool)) or exp is None:
        assert out == exp, (vec["id"], out, exp)
    else:
        assert abs(float(out) - float(exp)) <= atol + rtol * abs(float(exp)), (vec["id"], out, exp)
