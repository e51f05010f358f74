"""Helpers shared by the parity tests: run one frontend call sequence on the oracle device and on the HIP device."""
import numpy as np


def run_on(mod, fn, arrays):
    """Uploads `arrays` to device module `mod`, applies fn(*tensors) and downloads the result(s) as NumPy."""
    ts = [mod.ofNumpy(a) for a in arrays]
    out = fn(*ts)
    if isinstance(out, (tuple, list)):
        return [mod.toNumpy(o) if hasattr(o, "Layout") else o for o in out]
    return mod.toNumpy(out) if hasattr(out, "Layout") else out


def both(H, G, fn, *arrays):
    return run_on(H, fn, arrays), run_on(G, fn, arrays)


def assert_exact(ref, got):
    ref, got = np.asarray(ref), np.asarray(got)
    assert ref.dtype == got.dtype, (ref.dtype, got.dtype)
    assert ref.shape == got.shape, (ref.shape, got.shape)
    if ref.dtype.kind == "f":
        # bit-exact including signed zeros; NaNs compare by payload-insensitive position
        assert np.array_equal(np.isnan(ref), np.isnan(got))
        m = ~np.isnan(ref)
        assert np.array_equal(ref[m].view(np.uint32 if ref.dtype == np.float32 else np.uint64),
                              got[m].view(np.uint32 if ref.dtype == np.float32 else np.uint64)), \
            f"max abs diff {np.max(np.abs(ref[m].astype(np.float64) - got[m].astype(np.float64)))}"
    else:
        assert np.array_equal(ref, got)


def assert_rel(ref, got, rel=1e-6):
    """|got - ref| <= rel * |ref| (+ one denormal step); infinities and NaNs must coincide."""
    ref, got = np.asarray(ref), np.asarray(got)
    assert ref.dtype == got.dtype and ref.shape == got.shape
    assert np.array_equal(np.isnan(ref), np.isnan(got))
    inf = np.isinf(ref)
    assert np.array_equal(ref[inf], got[inf])
    m = np.isfinite(ref)
    tiny = np.finfo(ref.dtype).smallest_subnormal
    err = np.abs(got[m].astype(np.float64) - ref[m].astype(np.float64))
    bound = rel * np.abs(ref[m].astype(np.float64)) + float(tiny)
    bad = err > bound
    assert not bad.any(), f"{bad.sum()} elements exceed rel {rel}: worst {np.max(err / np.maximum(np.abs(ref[m].astype(np.float64)), 1e-300))}"
