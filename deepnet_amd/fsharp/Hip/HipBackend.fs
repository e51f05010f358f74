namespace Tensor.Hip

// TensorHipStorage / TensorHipBackend / TensorHipDevice: the HIP counterpart of Tensor/Tensor/Cuda/CudaBackend.fs behind the
// unchanged plugin interfaces of Tensor/Tensor/TensorBackend.fs.  Every ITensorBackend member is one call into
// libtensor_hip.so; nothing is computed on the managed side.  Source only (no .NET SDK on this repository's build machine).

open System
open System.Runtime.InteropServices
open Tensor
open Tensor.Utils
open Tensor.Backend

/// Thread-local options (mirror of Tensor.Cuda.Cfg, Cuda/CudaCfg.fs:14-60).
type Cfg private () =
    static let stream = new System.Threading.ThreadLocal<nativeint> (fun () -> IntPtr.Zero)
    static let stacktrace = new System.Threading.ThreadLocal<bool> (fun () -> true)

    /// hipStream_t all operations of this thread are issued on (IntPtr.Zero = default stream)
    static member Stream
        with get () = stream.Value
        and set v = stream.Value <- v

    /// Read the device index-error flag after every Gather/Scatter so that a bad index raises at the faulting call, as on
    /// the host backend.  Defaults to true (a device never traps on a bad index, so this is the only way the error surfaces).
    static member Stacktrace
        with get () = stacktrace.Value
        and set v = stacktrace.Value <- v

    /// Tuning switches of the native library (dnh_set_option: which kernel computes a result, never its contract), e.g.
    /// Cfg.SetOption ("dot_bf16x3", 0) keeps single-precision products on the fp32 matrix instruction.
    static member SetOption (name: string, value: int) =
        Native.check (Native.dnh_set_option (System.Text.Encoding.ASCII.GetBytes (name + "\000"), value))
    static member GetOption (name: string) : int =
        let mutable v = 0
        Native.check (Native.dnh_get_option (System.Text.Encoding.ASCII.GetBytes (name + "\000"), &v))
        v

module internal Desc =
    let dtypeOf (t: Type) =
        if   t = typeof<bool>   then DType.Bool elif t = typeof<byte>   then DType.U8  elif t = typeof<sbyte>  then DType.I8
        elif t = typeof<int32>  then DType.I32  elif t = typeof<uint32> then DType.U32 elif t = typeof<int64>  then DType.I64
        elif t = typeof<uint64> then DType.U64  elif t = typeof<single> then DType.F32 elif t = typeof<double> then DType.F64
        elif t = typeof<int16>  then DType.I16  elif t = typeof<uint16> then DType.U16
        else raise (NotSupportedException (sprintf "element type %s is not supported by the HIP backend" t.Name))

    let make (basePtr: nativeint) (dataType: Type) (layout: TensorLayout) =
        if layout.NDims > 8 then raise (NotSupportedException "the HIP backend supports at most 8 dimensions")
        let mutable d = DnhTensor()
        d.Base <- basePtr
        d.Offset <- layout.Offset
        d.NDims <- layout.NDims
        d.DType <- int (dtypeOf dataType)
        layout.Shape |> List.iteri (fun i s -> d.SetShape (i, s))
        layout.Stride |> List.iteri (fun i s -> d.SetStride (i, s))
        d

    /// Calls f with the address of one host element holding `value`.  bool crosses as one byte 0/1 (a bool[] is not blittable
    /// and cannot be pinned); every other element type is pinned as a one-element array.
    let withScalar (value: 'T) (f: nativeint -> unit) =
        let arr : Array =
            if typeof<'T> = typeof<bool> then [| (if (box value :?> bool) then 1uy else 0uy) |] :> Array
            else [| value |] :> Array
        let h = GCHandle.Alloc (arr, GCHandleType.Pinned)
        try f (h.AddrOfPinnedObject ()) finally h.Free ()

    /// Reads one element back: `f` receives the address of a one-element buffer to fill.
    let readScalar<'T> (f: nativeint -> unit) : 'T =
        if typeof<'T> = typeof<bool> then
            let v = [| 0uy |]
            let h = GCHandle.Alloc (v, GCHandleType.Pinned)
            try f (h.AddrOfPinnedObject ()) finally h.Free ()
            box (v.[0] <> 0uy) :?> 'T
        else
            let v = [| Unchecked.defaultof<'T> |]
            let h = GCHandle.Alloc (v, GCHandleType.Pinned)
            try f (h.AddrOfPinnedObject ()) finally h.Free ()
            v.[0]

/// What the library reports without touching the device.
type Planning private () =
    /// Bytes of the stream's workspace a Scatter of `sources` elements of type 'T into a target of `cells` elements takes
    /// (0 where atomics do the work), so that pools can be sized before the first call.
    static member ScatterWorkspaceBytes<'T> (sources: int64, cells: int64) : uint64 =
        let mutable bytes = 0un
        Native.check (Native.dnh_scatter_workspace_bytes (int (Desc.dtypeOf typeof<'T>), sources, cells, &bytes))
        uint64 bytes

/// Device memory owned by one tensor storage (CudaBackend.fs:54-93).
/// The block comes from the library's stream-ordered cache under the stream current at creation.  While every use was
/// issued on that stream the finalizer hands it back without waiting for the device (the finalizer runs after the last
/// operation on the storage was queued, whichever thread it runs on); otherwise it uses the synchronising free.
/// A storage made from an existing device pointer (HipTensor.usingPtr) references that memory and never frees it.
type TensorHipStorage<'T when 'T: (new: unit -> 'T) and 'T: struct and 'T :> ValueType> private (nElems: int64, external: nativeint) =
    let bytes = unativeint (max nElems 1L) * unativeint sizeof<'T>
    let stream = Cfg.Stream
    let owned = external = IntPtr.Zero
    let mutable singleStream = true
    let mutable ptr = external
    do if owned then Native.check (Native.dnh_alloc_async (bytes, stream, &ptr))

    /// allocates nElems elements on the device
    new (nElems: int64) = TensorHipStorage<'T> (nElems, IntPtr.Zero)
    /// references nElems elements of existing device memory; the caller keeps ownership
    static member OfPointer (devPtr: nativeint, nElems: int64) =
        if devPtr = IntPtr.Zero then invalidArg "devPtr" "null device pointer"
        TensorHipStorage<'T> (nElems, devPtr)

    member this.Ptr =
        if Cfg.Stream <> stream then singleStream <- false
        ptr
    member this.NElems = nElems
    override this.Finalize () =
        if owned && ptr <> IntPtr.Zero then
            (if singleStream then Native.dnh_free_async (ptr, stream) else Native.dnh_free ptr) |> ignore

    interface ITensorStorage<'T> with
        member this.Backend layout = TensorHipBackend<'T> (layout, this) :> ITensorBackend<_>
        member this.Dev = TensorHipDevice.Instance :> ITensorDevice

and TensorHipBackend<'T when 'T: (new: unit -> 'T) and 'T: struct and 'T :> ValueType>
        (layout: TensorLayout, storage: TensorHipStorage<'T>) =

    static let desc (t: ITensorFrontend<'A>) =
        let st = t.Storage :?> TensorHipStorage<'A>
        Desc.make st.Ptr typeof<'A> t.Layout

    // Every helper ends with GC.KeepAlive of the tensors it was given: `desc` copies the raw device pointer out of the storage, and
    // without a later use of the storage object its finalizer could release the block while the native call is still running.
    static let unary op (trgt: ITensorFrontend<'R>) (a: ITensorFrontend<'A>) =
        let mutable t, ad = desc trgt, desc a
        Native.check (Native.dnh_unary (op, &t, &ad, Cfg.Stream))
        GC.KeepAlive trgt; GC.KeepAlive a
    static let binary op (trgt: ITensorFrontend<'R>) (a: ITensorFrontend<'A>) (b: ITensorFrontend<'A>) =
        let mutable t, ad, bd = desc trgt, desc a, desc b
        Native.check (Native.dnh_binary (op, &t, &ad, &bd, Cfg.Stream))
        GC.KeepAlive trgt; GC.KeepAlive a; GC.KeepAlive b
    static let compare op (trgt: ITensorFrontend<bool>) (a: ITensorFrontend<'A>) (b: ITensorFrontend<'A>) =
        let mutable t, ad, bd = desc trgt, desc a, desc b
        Native.check (Native.dnh_compare (op, &t, &ad, &bd, Cfg.Stream))
        GC.KeepAlive trgt; GC.KeepAlive a; GC.KeepAlive b
    static let reduce op (trgt: ITensorFrontend<'R>) (src: ITensorFrontend<'A>) =
        let mutable t, sd = desc trgt, desc src
        Native.check (Native.dnh_reduce_last_axis (op, &t, &sd, Cfg.Stream))
        GC.KeepAlive trgt; GC.KeepAlive src
    static let argReduce op (trgt: ITensorFrontend<int64>) (src: ITensorFrontend<'A>) =
        let mutable t, sd = desc trgt, desc src
        Native.check (Native.dnh_arg_reduce_last_axis (op, &t, &sd, Cfg.Stream))
        GC.KeepAlive trgt; GC.KeepAlive src
    static let dot (trgt: ITensorFrontend<'T>) (a: ITensorFrontend<'T>) (b: ITensorFrontend<'T>) =
        let mutable t, ad, bd = desc trgt, desc a, desc b
        Native.check (Native.dnh_dot (&t, &ad, &bd, Cfg.Stream))
        GC.KeepAlive trgt; GC.KeepAlive a; GC.KeepAlive b

    /// Copies optional descriptors into unmanaged memory and calls f with the array of their addresses (IntPtr.Zero for None);
    /// the library copies the descriptors before it returns.
    static let withDescs (ts: ITensorFrontend<'A> option list) (f: nativeint[] -> unit) =
        let size = Marshal.SizeOf (typeof<DnhTensor>)
        let n = List.length ts
        let block = Marshal.AllocHGlobal (max 1 (size * n))
        try
            let ptrs =
                ts |> List.mapi (fun i t ->
                    match t with
                    | Some t ->
                        let p = block + nativeint (i * size)
                        Marshal.StructureToPtr (desc t, p, false)
                        p
                    | None -> IntPtr.Zero)
                |> Array.ofList
            f ptrs
        finally
            Marshal.FreeHGlobal block
            ts |> List.iter (Option.iter (fun t -> GC.KeepAlive t))

    static let checkIndexError () =
        if Cfg.Stacktrace then
            let mutable code = 0
            Native.check (Native.dnh_async_error (Cfg.Stream, &code))
            Native.check code

    let itemAddr (idx: int64[]) = storage.Ptr + nativeint (TensorLayout.addr (List.ofArray idx) layout) * nativeint sizeof<'T>

    interface ITensorBackend<'T> with
        member this.Item
            with get idx =                                              // CudaBackend.fs:77-87: synchronous 1-element copy
                let v = Desc.readScalar<'T> (fun p -> Native.check (Native.dnh_memcpy_d2h (p, itemAddr idx, unativeint sizeof<'T>, Cfg.Stream, 1)))
                GC.KeepAlive storage
                v
            and set idx value =
                Desc.withScalar value (fun p -> Native.check (Native.dnh_memcpy_h2d (itemAddr idx, p, unativeint sizeof<'T>, Cfg.Stream, 1)))
                GC.KeepAlive storage

        member this.Copy (trgt, src) =
            let mutable t, s = desc trgt, desc src
            Native.check (Native.dnh_copy (&t, &s, Cfg.Stream))
            GC.KeepAlive trgt; GC.KeepAlive src
        member this.Convert (trgt: ITensorFrontend<'T>, src: ITensorFrontend<'S>) =
            let mutable t, s = desc trgt, desc src
            Native.check (Native.dnh_convert (&t, &s, Cfg.Stream))
            GC.KeepAlive trgt; GC.KeepAlive src
        member this.Transfer (trgt, src) = HipTransfer.transfer (trgt, src)   // host <-> device, as CudaBackend.fs:206-270
        member this.FillConst (value, trgt) =
            let mutable t = desc trgt
            Desc.withScalar value (fun p -> Native.check (Native.dnh_fill_const (&t, p, Cfg.Stream)))
            GC.KeepAlive trgt
        member this.FillIncrementing (start, incr, trgt) =               // numeric element types only, so the array is blittable
            let mutable t = desc trgt
            let h = GCHandle.Alloc ([| start; incr |], GCHandleType.Pinned)
            try
                let p = h.AddrOfPinnedObject ()
                Native.check (Native.dnh_fill_incrementing (&t, p, p + nativeint sizeof<'T>, Cfg.Stream))
            finally h.Free ()
            GC.KeepAlive trgt

        member this.UnaryPlus (t, a) = unary 0 t a
        member this.UnaryMinus (t, a) = unary 1 t a
        member this.Abs (t, a) = unary 2 t a
        member this.Sgn (t, a) = unary 3 t a
        member this.Log (t, a) = unary 4 t a
        member this.Log10 (t, a) = unary 5 t a
        member this.Exp (t, a) = unary 6 t a
        member this.Sin (t, a) = unary 7 t a
        member this.Cos (t, a) = unary 8 t a
        member this.Tan (t, a) = unary 9 t a
        member this.Asin (t, a) = unary 10 t a
        member this.Acos (t, a) = unary 11 t a
        member this.Atan (t, a) = unary 12 t a
        member this.Sinh (t, a) = unary 13 t a
        member this.Cosh (t, a) = unary 14 t a
        member this.Tanh (t, a) = unary 15 t a
        member this.Sqrt (t, a) = unary 16 t a
        member this.Ceiling (t, a) = unary 17 t a
        member this.Floor (t, a) = unary 18 t a
        member this.Round (t, a) = unary 19 t a
        member this.Truncate (t, a) = unary 20 t a
        member this.Negate (t, a) = unary 21 t a
        member this.IsFinite (trgt, src) =
            let mutable t, a = desc trgt, desc src
            Native.check (Native.dnh_is_finite (&t, &a, Cfg.Stream))
            GC.KeepAlive trgt; GC.KeepAlive src

        member this.Add (t, a, b) = binary 0 t a b
        member this.Subtract (t, a, b) = binary 1 t a b
        member this.Multiply (t, a, b) = binary 2 t a b
        member this.Divide (t, a, b) = binary 3 t a b
        member this.Modulo (t, a, b) = binary 4 t a b
        member this.Power (t, a, b) = binary 5 t a b
        member this.MaxElemwise (t, a, b) = binary 6 t a b
        member this.MinElemwise (t, a, b) = binary 7 t a b
        member this.And (t, a, b) = binary 8 t a b
        member this.Or (t, a, b) = binary 9 t a b
        member this.Xor (t, a, b) = binary 10 t a b

        member this.Equal (t, a, b) = compare 0 t a b
        member this.NotEqual (t, a, b) = compare 1 t a b
        member this.Less (t, a, b) = compare 2 t a b
        member this.LessOrEqual (t, a, b) = compare 3 t a b
        member this.Greater (t, a, b) = compare 4 t a b
        member this.GreaterOrEqual (t, a, b) = compare 5 t a b

        member this.IfThenElse (trgt, cond, ifTrue, ifFalse) =
            let mutable t, c, a, b = desc trgt, desc cond, desc ifTrue, desc ifFalse
            Native.check (Native.dnh_if_then_else (&t, &c, &a, &b, Cfg.Stream))
            GC.KeepAlive trgt; GC.KeepAlive cond; GC.KeepAlive ifTrue; GC.KeepAlive ifFalse

        member this.Gather (trgt, srcIdxs, src) =
            let mutable t, s = desc trgt, desc src
            withDescs srcIdxs (fun p -> Native.check (Native.dnh_gather (&t, p, p.Length, &s, Cfg.Stream)))
            GC.KeepAlive trgt; GC.KeepAlive src
            checkIndexError ()
        member this.Scatter (trgt, trgtIdxs, src) =
            let mutable t, s = desc trgt, desc src
            withDescs trgtIdxs (fun p -> Native.check (Native.dnh_scatter (&t, p, p.Length, &s, Cfg.Stream)))
            GC.KeepAlive trgt; GC.KeepAlive src
            checkIndexError ()
        member this.MaskedGet (trgt, src, masks) =
            let mutable t, s = desc trgt, desc src
            withDescs (List.ofArray masks) (fun p -> Native.check (Native.dnh_masked_get (&t, &s, p, p.Length, Cfg.Stream)))
            GC.KeepAlive trgt; GC.KeepAlive src
        member this.MaskedSet (trgt, masks, src) =
            let mutable t, s = desc trgt, desc src
            withDescs (List.ofArray masks) (fun p -> Native.check (Native.dnh_masked_set (&t, p, p.Length, &s, Cfg.Stream)))
            GC.KeepAlive trgt; GC.KeepAlive src
        member this.TrueIndices (trgt, src) =
            let mutable t, s = desc trgt, desc src
            Native.check (Native.dnh_true_indices (&t, &s, Cfg.Stream))
            GC.KeepAlive trgt; GC.KeepAlive src

        member this.SumLastAxis (t, s) = reduce 0 t s
        member this.ProductLastAxis (t, s) = reduce 1 t s
        member this.MinLastAxis (t, s) = reduce 2 t s
        member this.MaxLastAxis (t, s) = reduce 3 t s
        member this.AllLastAxis (t, s) = reduce 4 t s
        member this.AnyLastAxis (t, s) = reduce 5 t s
        member this.CountTrueLastAxis (t, s) = reduce 6 t s
        member this.ArgMinLastAxis (t, s) = argReduce 0 t s
        member this.ArgMaxLastAxis (t, s) = argReduce 1 t s
        member this.FindLastAxis (value, trgt, src) =
            let mutable t, s = desc trgt, desc src
            Desc.withScalar value (fun p -> Native.check (Native.dnh_find_last_axis (p, &t, &s, Cfg.Stream)))
            GC.KeepAlive trgt; GC.KeepAlive src

        member this.VecVecDot (t, a, b) = dot t a b
        member this.MatVecDot (t, a, b) = dot t a b
        member this.MatMatDot (t, a, b) = dot t a b
        member this.BatchedMatMatDot (t, a, b) = dot t a b

        // LAPACK-type members; the CUDA backend leaves SVD and the eigen-decomposition unsupported (CudaBackend.fs:486-492)
        member this.BatchedInvert (trgt, src) =
            let mutable t, s = desc trgt, desc src
            Native.check (Native.dnh_batched_invert (&t, &s, Cfg.Stream))
            GC.KeepAlive trgt; GC.KeepAlive src
        member this.BatchedSVD (trgtS, trgtUV, src) =
            let mutable s, a = desc trgtS, desc src
            match trgtUV with
            | Some (trgtU, trgtV) ->
                let mutable u, v = desc trgtU, desc trgtV
                Native.check (Native.dnh_batched_svd (&s, &u, &v, &a, Cfg.Stream))
            | None ->
                Native.check (Native.dnh_batched_svd_values (&s, IntPtr.Zero, IntPtr.Zero, &a, Cfg.Stream))
            GC.KeepAlive trgtS; GC.KeepAlive trgtUV; GC.KeepAlive src
        member this.SymmetricEigenDecomposition (part, eigVals, eigVecs, src) =
            let mutable w, v, a = desc eigVals, desc eigVecs, desc src
            let part = match part with | MatrixPart.Upper -> 0 | MatrixPart.Lower -> 1
            Native.check (Native.dnh_symmetric_eig (part, &w, &v, &a, Cfg.Stream))
            GC.KeepAlive eigVals; GC.KeepAlive eigVecs; GC.KeepAlive src

/// Host <-> device copies: the source is made row-major first, a non-row-major target goes through a device temporary
/// (CudaBackend.fs:206-270).  Returns false for pairs this backend does not handle so the frontend can try the other side
/// (Tensor.fs:704-711).
and internal HipTransfer =
    static member transfer (trgt: ITensorFrontend<'T>, src: ITensorFrontend<'T>) : bool =
        match box trgt.Storage, box src.Storage with
        | (:? TensorHipStorage<'T> as ts), (:? Tensor.Host.TensorHostStorage<'T> as hs) ->
            let src = if TensorLayout.isC src.Layout then src else src.Copy (order=RowMajor)
            let hs = src.Storage :?> Tensor.Host.TensorHostStorage<'T>
            use pin = hs.Pin ()
            let bytes = unativeint (src.NElems * int64 sizeof<'T>)
            let hostPtr = pin.Ptr + nativeint (src.Layout.Offset * int64 sizeof<'T>)
            if TensorLayout.isC trgt.Layout then
                let dst = ts.Ptr + nativeint (trgt.Layout.Offset * int64 sizeof<'T>)
                Native.check (Native.dnh_memcpy_h2d (dst, hostPtr, bytes, Cfg.Stream, 1))
            else
                let tmp = trgt.Copy (order=RowMajor)
                let tmpSt = tmp.Storage :?> TensorHipStorage<'T>
                Native.check (Native.dnh_memcpy_h2d (tmpSt.Ptr, hostPtr, bytes, Cfg.Stream, 1))
                trgt.CopyFrom tmp
            true
        | (:? Tensor.Host.TensorHostStorage<'T> as hs), (:? TensorHipStorage<'T>) ->
            let src = if TensorLayout.isC src.Layout then src else src.Copy (order=RowMajor)
            let ss = src.Storage :?> TensorHipStorage<'T>
            let tmpHost = if TensorLayout.isC trgt.Layout then trgt else trgt.Copy (order=RowMajor)
            let ths = tmpHost.Storage :?> Tensor.Host.TensorHostStorage<'T>
            use pin = ths.Pin ()
            let bytes = unativeint (src.NElems * int64 sizeof<'T>)
            let srcPtr = ss.Ptr + nativeint (src.Layout.Offset * int64 sizeof<'T>)
            Native.check (Native.dnh_memcpy_d2h (pin.Ptr + nativeint (tmpHost.Layout.Offset * int64 sizeof<'T>), srcPtr, bytes, Cfg.Stream, 1))
            if not (obj.ReferenceEquals (tmpHost, trgt)) then trgt.CopyFrom tmpHost
            true
        | _ -> false

/// The device (CudaBackend.fs:497-507): new storage is uninitialised, so Zeroed = false and `zeros` launches FillConst.
and TensorHipDevice private () =
    inherit BaseTensorDevice ()
    static let instance = TensorHipDevice ()
    static member Instance = instance
    override this.Id = "Hip"
    override this.Create nElems = TensorHipStorage<'T> nElems :> ITensorStorage<'T>
    override this.Zeroed = false
