namespace Tensor

// The HipTensor module: creation functions on the HIP device, mirroring Tensor/Tensor/Cuda/CudaFrontend.fs:30-149.
// Source only (no .NET SDK on this repository's build machine).

open System
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

    /// <summary>Creates a tensor from the given device pointer, allocation size in bytes, type and layout
    /// (the counterpart of CudaTensor.usingPtrAndType, Tensor/Tensor/Cuda/CudaFrontend.fs:129-137).</summary>
    /// <remarks>The data is referenced, not copied, and is never freed by the tensor: changing values within the tensor changes
    /// the original data, and the memory must outlive the tensor.</remarks>
    let usingPtrAndType (ptr: nativeint) (sizeInBytes: int64) (typ: Type) (layout: TensorLayout) =
        let elemSize = int64 (System.Runtime.InteropServices.Marshal.SizeOf typ)
        let storType = typedefof<TensorHipStorage<_>>.MakeGenericType [|typ|]
        let ofPointer = storType.GetMethod "OfPointer"
        let stor = ofPointer.Invoke (null, [|box ptr; box (sizeInBytes / elemSize)|])
        let tensorType = typedefof<Tensor<_>>.MakeGenericType [|typ|]
        Activator.CreateInstance (tensorType, [|box layout; stor|]) :?> ITensor

    /// <summary>Creates a tensor from the given device pointer, allocation size in bytes and layout
    /// (the counterpart of CudaTensor.usingPtr, Tensor/Tensor/Cuda/CudaFrontend.fs:139-149).</summary>
    let usingPtr<'T> (ptr: nativeint) (sizeInBytes: int64) (layout: TensorLayout) =
        usingPtrAndType ptr sizeInBytes typeof<'T> layout :?> Tensor<'T>
