"""The reference's own device tests (Tensor/Tensor.Test/CudaTests.fs:28-177) with the HIP device in place of CudaTensor and the
oracle device in place of HostTensor: host <-> device transfers of row-major and other layouts, single and double matrix dot
against the host result, and the mixed copy / fill / diagonal / invert / element-wise / reduction sequence."""
import numpy as np
import pytest

from deepnet_amd.tensor import Tensor

pytestmark = pytest.mark.gpu


def almost_equal(a, b, abs_tol=1e-5, rel_tol=1e-5):
    """Tensor.almostEqual on downloaded arrays (Tensor.fs isClose: |a - b| <= absTol + relTol |b|)."""
    return a.shape == b.shape and bool(np.all(np.abs(a - b) <= abs_tol + rel_tol * np.abs(b)))


def test_tensor_transfer_to_device(H, G):
    """CudaTests.fs:28-37: counting 30 -> float -> [3; 10], to the device and back."""
    data = H.Dev and Tensor.counting(30, H.Dev).convert(np.float64).reshape([3, 10])
    dev = G.transfer(data)
    assert dev.Dev.Id == "Hip" and dev.Shape == [3, 10]
    back = H.transfer(dev)
    assert back.Dev.Id == H.Dev.Id
    np.testing.assert_array_equal(H.toNumpy(back), H.toNumpy(data))


def test_tensor_transfer_to_device_custom_order(H, G):
    """CudaTests.fs:39-51: a [3; 2; 5] tensor stored in the order [1; 0; 2] (not row-major) survives the round trip."""
    data = Tensor.counting(30, H.Dev).convert(np.float64).reshape([3, 2, 5])
    # the copy with order=CustomOrder [1; 0; 2]: dimension 1 is the fastest, then 0, then 2
    storage_view = Tensor.new([5, 3, 2], H.Dev, np.float64).permuteAxes([2, 0, 1])       # shape [3; 2; 5], strides [2; 1; 6]
    assert storage_view.Shape == [3, 2, 5] and storage_view.Stride == [2, 1, 6]
    storage_view.CopyFrom(data)
    dev = G.transfer(storage_view)
    back = H.transfer(dev)
    np.testing.assert_array_equal(H.toNumpy(back), H.toNumpy(data))
    # and a non-row-major device tensor transfers back correctly as well
    dev_t = dev.T
    np.testing.assert_array_equal(H.toNumpy(H.transfer(dev_t)), H.toNumpy(data).transpose(0, 2, 1))
    # transfer into a non-row-major device target goes through a temporary (CudaBackend.fs:260-270)
    trgt = Tensor.new([5, 2, 3], G.Dev, np.float64).permuteAxes([2, 1, 0])               # shape [3; 2; 5], not row-major
    assert trgt.Backend.Transfer(trgt, data)
    np.testing.assert_array_equal(G.toNumpy(trgt), H.toNumpy(data))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_matrix_dot_against_host(H, G, dtype):
    """CudaTests.fs:53-75: h = init [5; 3] (3 i + j), i = 0.1 + identity 3; device h .* i almost equals host h .* i."""
    h_np = np.fromfunction(lambda i, j: 3.0 * i + j, (5, 3)).astype(dtype)
    h = H.ofNumpy(h_np)
    i = Tensor.identity(3, H.Dev, dtype) + dtype(0.1)
    hi = h @ i
    h_gpu, i_gpu = G.transfer(h), G.transfer(i)
    hi_gpu = h_gpu @ i_gpu
    assert almost_equal(H.toNumpy(H.transfer(hi_gpu)), H.toNumpy(hi))


def test_mixed_device_sequence(H, G):
    """CudaTests.fs:77-177: ones -> device -> host; device copy; FillConst; 3 * identity; its inverse; element-wise and axis ops."""
    shape = [5, 5]
    a = Tensor.ones(shape, H.Dev, np.float32)
    ca = G.transfer(a)
    ha = H.transfer(ca)
    np.testing.assert_array_equal(H.toNumpy(ha), np.ones(shape, np.float32))
    cb = ca.Copy()
    cb.FillConst(np.float32(-5.5))
    np.testing.assert_array_equal(G.toNumpy(cb), np.full(shape, -5.5, np.float32))
    np.testing.assert_array_equal(G.toNumpy(ca), np.ones(shape, np.float32))            # the copy owns its storage
    cdiag = Tensor.identity(3, G.Dev, np.float32) * np.float32(3.0)
    cinv = Tensor.invert(cdiag)
    np.testing.assert_allclose(G.toNumpy(cinv), np.eye(3, dtype=np.float32) / 3, rtol=1e-6)
    # element-wise and reductions on device operands against the same calls on the host
    x = np.arange(25, dtype=np.float32).reshape(5, 5) / 7
    hx, cx = H.ofNumpy(x), G.ofNumpy(x)
    for f in (lambda t: t + t, lambda t: t * t - t, lambda t: (t + 1.0).log(), lambda t: t.sumAxis(0), lambda t: t.maxAxis(1),
              lambda t: t.T.Copy(), lambda t: t > 1.5, lambda t: t.argMaxAxis(0)):
        ref, got = H.toNumpy(f(hx)), G.toNumpy(f(cx))
        assert ref.dtype == got.dtype
        if ref.dtype.kind == "f":
            assert almost_equal(got, ref, 1e-6, 1e-6)
        else:
            np.testing.assert_array_equal(got, ref)


def test_operands_on_different_devices_are_rejected(H, G):
    """Tensor.fs:4507-4512 CheckSameStorage."""
    with pytest.raises(ValueError):
        H.ofNumpy(np.ones(3, np.float32)) + G.ofNumpy(np.ones(3, np.float32))
