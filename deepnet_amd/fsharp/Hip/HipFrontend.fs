namespace Tensor

// The HipTensor module: creation functions on the HIP device, mirroring Tensor/Tensor/Cuda/CudaFrontend.fs:30-149.
// Source only (no .NET SDK on this repository's build machine).

open Tensor.Backend
open Tensor.Hip

module HipTensor =
    /// the HIP tensor device
    let Dev = TensorHipDevice.Instance :> ITensorDevice

    /// copies a tensor (normally a HostTensor) to the HIP device
    let transfer x = Tensor.transfer Dev x

    let empty<'T> = Tensor<'T>.empty Dev
    let zeros<'T> = Tensor<'T>.zeros Dev
    let ones<'T> = Tensor<'T>.ones Dev
    let falses = Tensor.falses Dev
    let trues = Tensor.trues Dev
    let scalar<'T> = Tensor<'T>.scalar Dev
    let filled<'T> = Tensor<'T>.filled Dev
    let identity<'T> = Tensor<'T>.identity Dev
    let counting = Tensor.counting Dev
    let arange<'T> = Tensor<'T>.arange Dev
    let linspace<'T> = Tensor<'T>.linspace Dev
