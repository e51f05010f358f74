"""deepnet_amd — MI355X (gfx950) tensor backend for Deep.Net's Tensor<'T> plugin surface.

`deepnet_amd.hip` is the HipTensor device (loads libtensor_hip.so on first use); `deepnet_amd.tensor.Tensor` is the
device-agnostic frontend mirror; `deepnet_amd.layout` the TensorLayout algebra; `deepnet_amd.abi` the C ABI declarations.
"""
from . import abi, layout  # noqa: F401
from .tensor import Tensor  # noqa: F401
