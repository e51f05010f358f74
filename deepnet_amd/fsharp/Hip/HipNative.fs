namespace Tensor.Hip

// P/Invoke surface of libtensor_hip.so (include/tensor_hip.h).  Source only: this repository's build machine has no
// .NET SDK, so these files are compiled where Deep.Net is (add them to Tensor/Tensor/Tensor.fsproj after the Cuda/ group
// and ship libtensor_hip.so under runtimes/linux-x64/native, the location Tensor/Tensor/NativeLib.fs:146-161 probes).

open System
open System.Runtime.InteropServices

/// DnhStatus
type internal Status =
    | OK = 0
    | InvalidArg = 1
    | NotSupported = 2
    | OutOfMemory = 3
    | Hip = 4
    | IndexOutOfRange = 5
    | NotInitialized = 6
    | SingularMatrix = 7
    | NoConvergence = 8

/// DnhDType — the element types the reference marshals to kernels (Cuda/NativeTensor.fs:22-34).
type internal DType =
    | Bool = 0 | U8 = 1 | I8 = 2 | I32 = 3 | U32 = 4 | I64 = 5 | U64 = 6 | F32 = 7 | F64 = 8 | I16 = 9 | U16 = 10

/// DnhTensor: descriptor passed by reference (replaces the Reflection.Emit structs of Cuda/NativeTensor.fs:96-208).
/// Blittable: the two extents arrays of the C struct are spelled out as sixteen int64 fields (a managed int64[] marked ByValArray
/// would make the struct non-blittable: it could not be pinned, and `byref` marshalling would copy it on every call).
[<Struct; StructLayout(LayoutKind.Sequential)>]
type internal DnhTensor =
    val mutable Base:   nativeint
    val mutable Offset: int64
    val mutable NDims:  int32
    val mutable DType:  int32
    val mutable Shape0: int64
    val mutable Shape1: int64
    val mutable Shape2: int64
    val mutable Shape3: int64
    val mutable Shape4: int64
    val mutable Shape5: int64
    val mutable Shape6: int64
    val mutable Shape7: int64
    val mutable Stride0: int64
    val mutable Stride1: int64
    val mutable Stride2: int64
    val mutable Stride3: int64
    val mutable Stride4: int64
    val mutable Stride5: int64
    val mutable Stride6: int64
    val mutable Stride7: int64

    member this.SetShape (i: int, v: int64) =
        match i with
        | 0 -> this.Shape0 <- v | 1 -> this.Shape1 <- v | 2 -> this.Shape2 <- v | 3 -> this.Shape3 <- v
        | 4 -> this.Shape4 <- v | 5 -> this.Shape5 <- v | 6 -> this.Shape6 <- v | 7 -> this.Shape7 <- v
        | _ -> invalidArg "i" "a descriptor holds at most 8 dimensions"
    member this.SetStride (i: int, v: int64) =
        match i with
        | 0 -> this.Stride0 <- v | 1 -> this.Stride1 <- v | 2 -> this.Stride2 <- v | 3 -> this.Stride3 <- v
        | 4 -> this.Stride4 <- v | 5 -> this.Stride5 <- v | 6 -> this.Stride6 <- v | 7 -> this.Stride7 <- v
        | _ -> invalidArg "i" "a descriptor holds at most 8 dimensions"

module internal Native =
    [<Literal>]
    let Lib = "tensor_hip"
    let private cc = CallingConvention.Cdecl

    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_init (int device)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_last_error (byte[] buf, unativeint n)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_async_error (nativeint stream, int& code)
    // option names cross as NUL-terminated ASCII bytes
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_set_option (byte[] name, int value)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_get_option (byte[] name, int& value)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_scatter_workspace_bytes (int dtype, int64 sources, int64 cells, unativeint& bytes)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_alloc (unativeint bytes, nativeint& ptr)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_free (nativeint ptr)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_alloc_async (unativeint bytes, nativeint stream, nativeint& ptr)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_free_async (nativeint ptr, nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_pool_trim ()
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_memcpy_h2d (nativeint dst, nativeint src, unativeint bytes, nativeint stream, int sync)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_memcpy_d2h (nativeint dst, nativeint src, unativeint bytes, nativeint stream, int sync)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_stream_sync (nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_fill_const (DnhTensor& t, nativeint value, nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_fill_incrementing (DnhTensor& t, nativeint start, nativeint incr, nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_copy (DnhTensor& t, DnhTensor& src, nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_convert (DnhTensor& t, DnhTensor& src, nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_unary (int op, DnhTensor& t, DnhTensor& a, nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_is_finite (DnhTensor& t, DnhTensor& a, nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_binary (int op, DnhTensor& t, DnhTensor& a, DnhTensor& b, nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_compare (int op, DnhTensor& t, DnhTensor& a, DnhTensor& b, nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_if_then_else (DnhTensor& t, DnhTensor& c, DnhTensor& a, DnhTensor& b, nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_reduce_last_axis (int op, DnhTensor& t, DnhTensor& src, nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_arg_reduce_last_axis (int op, DnhTensor& t, DnhTensor& src, nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_find_last_axis (nativeint value, DnhTensor& t, DnhTensor& src, nativeint stream)
    // index tensors and masks: arrays of pointers to pinned descriptors, IntPtr.Zero where the reference passes None
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_gather (DnhTensor& t, nativeint[] idx, int nIdx, DnhTensor& src, nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_scatter (DnhTensor& t, nativeint[] idx, int nIdx, DnhTensor& src, nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_masked_get (DnhTensor& t, DnhTensor& src, nativeint[] masks, int nMasks, nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_masked_set (DnhTensor& t, nativeint[] masks, int nMasks, DnhTensor& src, nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_true_indices (DnhTensor& t, DnhTensor& src, nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_dot (DnhTensor& t, DnhTensor& a, DnhTensor& b, nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_batched_invert (DnhTensor& t, DnhTensor& src, nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_batched_svd (DnhTensor& s, DnhTensor& u, DnhTensor& v, DnhTensor& src, nativeint stream)
    // the same entry point with u = v = NULL: singular values only
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl, EntryPoint="dnh_batched_svd")>] extern int dnh_batched_svd_values (DnhTensor& s, nativeint u, nativeint v, DnhTensor& src, nativeint stream)
    [<DllImport(Lib, CallingConvention=CallingConvention.Cdecl)>] extern int dnh_symmetric_eig (int part, DnhTensor& eigVals, DnhTensor& eigVecs, DnhTensor& src, nativeint stream)

    /// Maps a status to the exception type the reference's backends raise for the same condition.
    let check (status: int) =
        if status <> 0 then
            let buf = Array.zeroCreate<byte> 1024
            dnh_last_error (buf, unativeint buf.Length) |> ignore
            let msg = System.Text.Encoding.UTF8.GetString(buf).TrimEnd('\000')
            match enum<Status> status with
            | Status.InvalidArg -> raise (InvalidOperationException msg)
            | Status.NotSupported -> raise (NotSupportedException msg)
            | Status.OutOfMemory -> raise (OutOfMemoryException msg)
            | Status.IndexOutOfRange -> raise (IndexOutOfRangeException msg)
            | Status.SingularMatrix -> raise (Tensor.SingularMatrixException msg)
            | Status.NoConvergence -> failwith msg      // "SVD did not converge" (Host/HostBackend.fs:598)
            | _ -> failwithf "HIP tensor backend error %d: %s" status msg
