/*
 * tensor_hip.h — C ABI of libtensor_hip.so, the MI355X (gfx950) tensor backend that a Deep.Net
 * `TensorHipBackend<'T>` binds through P/Invoke (cdecl, blittable arguments only).
 *
 * Every entry point replaces one member (or a family of members) of the reference plugin interface
 * `ITensorBackend<'T>` (Tensor/Tensor/TensorBackend.fs:64-146) or one facility the reference's CUDA
 * storage/device objects obtain from the CUDA driver (Tensor/Tensor/Cuda/CudaBackend.fs,
 * Tensor/Tensor/Cuda/CudaUtils.fs).  The citation beside each declaration names what it replaces.
 *
 * Conventions
 *  - every function returns a DnhStatus (0 = OK); a human-readable message for the calling thread's
 *    last failure is available from dnh_last_error();
 *  - tensors are passed as pointers to DnhTensor descriptors, which the library copies before it returns;
 *    `base` is a DEVICE pointer to element 0 of the storage, `offset` and `stride` are in ELEMENTS and
 *    may be zero (broadcast) or negative, exactly as in TensorLayout (Tensor/Tensor/TensorLayout.fs:12-24);
 *  - operands arrive already broadcast to the target's shape by the frontend
 *    (Tensor/Tensor/Tensor.fs:4520-4540); the library checks shapes and dtypes and reports
 *    DNH_ERR_INVALID_ARG on a mismatch;
 *  - `stream` is a hipStream_t passed as void* (NULL = the default stream); all ops are asynchronous with
 *    respect to the host unless stated otherwise;
 *  - all entry points may be called from any thread, also several threads on one stream at once: scratch memory
 *    the library keeps per stream is held by one call until the kernels that use it are queued.
 */
#ifndef TENSOR_HIP_H
#define TENSOR_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DNH_MAX_DIMS 8

typedef enum DnhStatus {
    DNH_OK = 0,
    DNH_ERR_INVALID_ARG = 1,      /* -> ArgumentException / InvalidOperationException          */
    DNH_ERR_NOT_SUPPORTED = 2,    /* -> NotSupportedException (CudaBackend.fs:486-492)          */
    DNH_ERR_OUT_OF_MEMORY = 3,    /* -> OutOfCudaMemoryException analogue (CudaUtils.fs:183-210) */
    DNH_ERR_HIP = 4,              /* -> CudaException analogue                                  */
    DNH_ERR_INDEX_OUT_OF_RANGE = 5, /* -> IndexOutOfRangeException (Host/FastAccess.fs:51-61)   */
    DNH_ERR_NOT_INITIALIZED = 6,
    DNH_ERR_SINGULAR_MATRIX = 7,  /* -> SingularMatrixException (Tensor.fs:2831-2834)               */
    DNH_ERR_NO_CONVERGENCE = 8    /* -> "SVD did not converge" (Host/HostBackend.fs:598)             */
} DnhStatus;

/* Element types: the set the reference marshals to kernels (Cuda/NativeTensor.fs:22-34) plus the 16-bit integers its host device
 * also handles (Sgn.fs:11-15, Host/ScalarOps.fs).  bool is one byte 0/1.  Values are part of the ABI: new types are appended. */
typedef enum DnhDType {
    DNH_BOOL = 0,
    DNH_U8 = 1,
    DNH_I8 = 2,
    DNH_I32 = 3,
    DNH_U32 = 4,
    DNH_I64 = 5,
    DNH_U64 = 6,
    DNH_F32 = 7,
    DNH_F64 = 8,
    DNH_I16 = 9,
    DNH_U16 = 10,
    DNH_DTYPE_COUNT = 11
} DnhDType;

/* Replaces the by-value kernel argument struct Tensor<T,N> (Cuda/Kernels/Tensor.cuh:7-16,
 * Cuda/NativeTensor.fs:96-112): one rank-agnostic, blittable descriptor. */
typedef struct DnhTensor {
    void*   base;                  /* device pointer to element 0 of the storage, aligned to the
                                    * element size (no more is asked for: offsets, pitches and
                                    * extents are free, odd ones included)                        */
    int64_t offset;                /* TensorLayout.Offset (elements)                             */
    int32_t ndims;                 /* 0..DNH_MAX_DIMS                                            */
    int32_t dtype;                 /* DnhDType                                                   */
    int64_t shape[DNH_MAX_DIMS];   /* TensorLayout.Shape                                         */
    int64_t stride[DNH_MAX_DIMS];  /* TensorLayout.Stride (elements)                             */
} DnhTensor;

typedef struct DnhDeviceInfo {
    int32_t device;
    int32_t compute_units;
    int32_t wavefront_size;
    int32_t max_threads_per_block;
    int64_t lds_bytes_per_block;
    int64_t total_memory_bytes;
    int64_t l2_bytes;
    int32_t clock_khz;
    int32_t memory_clock_khz;
    char    name[128];
    char    arch[64];
} DnhDeviceInfo;

/* State of the block cache behind dnh_alloc_async / dnh_free_async. */
typedef struct DnhPoolStats {
    int64_t live_bytes;    /* handed out and not yet released                      */
    int64_t cached_bytes;  /* released and kept for reuse                          */
    int64_t limit_bytes;   /* cap on cached_bytes, 0 = none                        */
    int64_t hits;          /* allocations served from the cache                    */
    int64_t misses;        /* allocations that went to the driver                  */
} DnhPoolStats;

/* Unary element ops: ITensorBackend UnaryPlus..Truncate (TensorBackend.fs:74-94), Negate (:113);
 * scalar semantics Host/ScalarOps.fs:381-493, ScalarPrimitives.fs:54-150, Sgn.fs:11-15.
 * Round is ties-to-even (F# `round`), unlike the reference CUDA kernel (Cuda/Kernels/Elemwise.cuh:128). */
typedef enum DnhUnaryOp {
    DNH_UNARY_PLUS = 0, DNH_UNARY_MINUS, DNH_ABS, DNH_SGN, DNH_LOG, DNH_LOG10, DNH_EXP, DNH_SIN, DNH_COS,
    DNH_TAN, DNH_ASIN, DNH_ACOS, DNH_ATAN, DNH_SINH, DNH_COSH, DNH_TANH, DNH_SQRT, DNH_CEILING, DNH_FLOOR,
    DNH_ROUND, DNH_TRUNCATE, DNH_NEGATE, DNH_UNARY_COUNT
} DnhUnaryOp;

/* Binary element ops: ITensorBackend Add..MinElemwise (TensorBackend.fs:97-104), And/Or/Xor (:114-116);
 * Host/ScalarOps.fs:495-575.  Max/Min are `if a>b then a else b` / `if a<b then a else b`. */
typedef enum DnhBinaryOp {
    DNH_ADD = 0, DNH_SUBTRACT, DNH_MULTIPLY, DNH_DIVIDE, DNH_MODULO, DNH_POWER, DNH_MAX_ELEMWISE,
    DNH_MIN_ELEMWISE, DNH_AND, DNH_OR, DNH_XOR, DNH_BINARY_COUNT
} DnhBinaryOp;

/* Comparisons into a bool target: ITensorBackend Equal..GreaterOrEqual (TensorBackend.fs:106-111);
 * Host/ScalarOps.fs:535-563. */
typedef enum DnhCompareOp {
    DNH_EQUAL = 0, DNH_NOT_EQUAL, DNH_LESS, DNH_LESS_OR_EQUAL, DNH_GREATER, DNH_GREATER_OR_EQUAL,
    DNH_COMPARE_COUNT
} DnhCompareOp;

/* Last-axis folds: ITensorBackend SumLastAxis..CountTrueLastAxis (TensorBackend.fs:125-131);
 * Host/ScalarOps.fs:299-361 (ApplyAxisFold), :606-636.
 * NaN in Min / Max: the reference's fold is the sequential `if res > v then res else v` from minValue (ScalarOps.fs:620-628), whose
 * result with NaNs depends on their positions: a NaN replaces the running value and is itself replaced by the next element, so the
 * result is the fold of what follows the last NaN, or NaN when it comes last.  The folds here give exactly that for every input (a
 * result that met a NaN is recomputed in the reference's order by the thread that stores it).  The element-wise MaxElemwise /
 * MinElemwise are the same comparison, `a > b ? a : b` (ScalarOps.fs:525-533; the reference's SIMD path for contiguous single and
 * double data, Host/VectorOps.fs:234-240, leaves the NaN case to the platform).  ArgMin / ArgMax never select a NaN, as
 * in the reference.  Sum / Product are re-associated: |result - reference| <= (n + 64) u sum|x_i| (u = unit roundoff). */
typedef enum DnhReduceOp {
    DNH_SUM = 0, DNH_PRODUCT, DNH_MIN, DNH_MAX, DNH_ALL, DNH_ANY, DNH_COUNT_TRUE, DNH_REDUCE_COUNT
} DnhReduceOp;

/* Index-valued last-axis folds: ArgMinLastAxis / ArgMaxLastAxis (TensorBackend.fs:133-134);
 * Host/ScalarOps.fs:638-654. */
typedef enum DnhArgReduceOp { DNH_ARG_MIN = 0, DNH_ARG_MAX = 1 } DnhArgReduceOp;

/* "value was not found": SpecialIdx.NotFound = Int64.MinValue + 4 (Tensor/Tensor/TensorRng.fs:24). */
#define DNH_NOT_FOUND ((int64_t)(-9223372036854775807LL - 1LL + 4LL))

/* ---------------------------------------------------------------------------------------------------
 * Device, errors                                     (replaces Cuda/CudaUtils.fs:36-60 context creation)
 * ------------------------------------------------------------------------------------------------- */
/* Selects the device every later call of this process runs on (the reference likewise creates one context on the
 * first device it finds, Cuda/CudaUtils.fs:36-60).  Optional: the first other call initialises device 0.  Calling it
 * again with the same device is a no-op; another device is refused with DNH_ERR_INVALID_ARG, since buffers, cached
 * blocks and workspaces already belong to the first one. */
int32_t dnh_init(int32_t device);
int32_t dnh_device_info(DnhDeviceInfo* info);
/* Copies the calling thread's last error message (NUL terminated, truncated to n). */
int32_t dnh_last_error(char* buf, size_t n);
/* Tuning switches (no counterpart in the reference, whose backends take theirs from Tensor.Cfg statics): process-wide integers that
 * select which kernel computes a result, never its contract; a change applies to the calls issued after it.  Each starts from the
 * environment variable DNH_<NAME IN UPPER CASE> when the process has one.
 *   "dot_bf16x3"        1 (default): single-precision products on the bf16 matrix instruction, three parts per float; 0: fp32 instruction
 *   "dot_f64_pinned"    1 (default): double-precision products on the kernel with a pinned instruction order where the layout allows
 *   "dot_big"           -1 (default): the library picks the tile form of the bf16-parts kernel; 0 / 1: 128 x 128 / 256 x 256 tiles
 *   "dot_splits"        0 (default): the library picks the number of chunks along K; n > 0: that many
 *   "dot_int_mfma"      1 (default): 32- and 64-bit integer products on the int8 matrix instruction
 *   "tr4"               1 (default): transposing copies of 4-byte elements through LDS
 *   "scatter_fp_atomic" 0 (default): floating-point scatter adds duplicates in source order; 1: float atomics (faster, order varies)
 *   "compact_one_pass"  0 (default): compactions of contiguous masks by a counting and a moving launch; 1: one launch whose
 *                       workgroups pass their counts on through device memory (measured slower on MI355X: the counts cross XCDs)
 *   "count_one_launch"  1 (default): CountTrue of a whole contiguous mask in one launch
 *   "lookback_spins"    262144 (default): how often a tile of a one-pass compaction polls for the counts of the tiles before it
 *                       before it counts them itself (0: at once; for tests of that path)
 *   "invert_tournament" -1 (default): BatchedInvert of matrices with more than 32 rows chooses the 32 pivot rows of a panel by
 *                       tournament (wavefronts elect candidates among 128 rows each, further games among the candidates) and
 *                       updates the columns the next panel does not need on a stream of the library's own, beside that panel's
 *                       tournament; 0: every size eliminates its panels column by column with partial pivoting in one
 *                       workgroup; 1: tournament for every size
 * Unknown names and values outside an option's range: DNH_ERR_INVALID_ARG. */
int32_t dnh_set_option(const char* name, int32_t value);
int32_t dnh_get_option(const char* name, int32_t* value);
/* Reads and clears the device-side index error flag set by gather/scatter kernels on `stream`
 * (synchronises the stream; every stream has its own flag, so concurrent streams do not see each other's errors).  *code = DNH_OK or DNH_ERR_INDEX_OUT_OF_RANGE.
 * Replaces the error word + `Cfg.Stacktrace` read-back of Cuda/CudaKernels.fs:323-342, 385-398. */
int32_t dnh_async_error(void* stream, int32_t* code);

/* ---------------------------------------------------------------------------------------------------
 * Memory and streams        (replaces TensorCudaStorage / CudaDeviceVariable, Cuda/CudaBackend.fs:54-93,
 *                            transfers :206-270, pinned host memory Cuda/CudaRegMem.fs, stream Cuda/CudaCfg.fs:16-27)
 * ------------------------------------------------------------------------------------------------- */
int32_t dnh_alloc(size_t bytes, void** out);          /* at least one byte is allocated (CudaBackend.fs:56-58) */
int32_t dnh_free(void* ptr);                          /* waits for in-flight work; callable from any thread    */
/* Stream-ordered storage for tensors created inside a chain of operations (every Tensor op allocates its result,
 * Tensor.fs:317-325, and the reference pays a driver allocation plus GC pressure handling for each one,
 * Cuda/CudaUtils.fs:179-210).  A block released with dnh_free_async(ptr, stream) is handed out again only to
 * dnh_alloc_async calls that name the same stream, so neither call waits for the device.  `stream` must be the one
 * stream all work on the block was queued on; a block used from several streams is released with dnh_free.
 * When the driver is out of memory the cache is emptied and the allocation retried once (the reference's GC retry).
 * dnh_free accepts blocks from either allocator. */
int32_t dnh_alloc_async(size_t bytes, void* stream, void** out);
int32_t dnh_free_async(void* ptr, void* stream);
int32_t dnh_pool_trim(void);                          /* waits for the device, returns every cached block to the driver */
int32_t dnh_pool_set_limit(size_t bytes);             /* cap on cached bytes; 0 (default) = no cap                      */
int32_t dnh_pool_stats(DnhPoolStats* stats);
int32_t dnh_host_alloc(size_t bytes, void** out);     /* pinned host memory for transfers                      */
int32_t dnh_host_free(void* ptr);
int32_t dnh_memset(void* dst, int32_t byte_value, size_t bytes, void* stream);
/* sync != 0: the call returns when the bytes have arrived.  Synchronous copies of 16 MiB and more between the device and host
 * memory that did not come from dnh_host_alloc are staged through pinned chunks on several host threads (callers take turns). */
int32_t dnh_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream, int32_t sync);
int32_t dnh_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream, int32_t sync);
int32_t dnh_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream, int32_t sync);
int32_t dnh_stream_create(void** stream);
int32_t dnh_stream_destroy(void* stream);
int32_t dnh_stream_sync(void* stream);
int32_t dnh_device_sync(void);
/* Events, for timing kernels on the stream they run on. */
int32_t dnh_event_create(void** event);
int32_t dnh_event_destroy(void* event);
int32_t dnh_event_record(void* event, void* stream);
int32_t dnh_event_sync(void* event);
int32_t dnh_event_elapsed_ms(void* start, void* stop, float* ms);

/* ---------------------------------------------------------------------------------------------------
 * Element-wise ops
 * ------------------------------------------------------------------------------------------------- */
/* ITensorBackend.FillConst (TensorBackend.fs:71; Host/ScalarOps.fs:363-365). `value` points to one host element of t's dtype. */
int32_t dnh_fill_const(const DnhTensor* t, const void* value, void* stream);
/* ITensorBackend.FillIncrementing (TensorBackend.fs:72; Host/ScalarOps.fs:367-370): t[pos] = start + incr * T(pos[0]). */
int32_t dnh_fill_incrementing(const DnhTensor* t, const void* start, const void* incr, void* stream);
/* ITensorBackend.Copy (TensorBackend.fs:67; Host/HostBackend.fs:196-208). Same dtype, any layouts. */
int32_t dnh_copy(const DnhTensor* t, const DnhTensor* src, void* stream);
/* ITensorBackend.Convert (TensorBackend.fs:69; Host/ScalarOps.fs:376-379): C# explicit numeric conversion. */
int32_t dnh_convert(const DnhTensor* t, const DnhTensor* src, void* stream);
/* Unary ops, DnhUnaryOp. */
int32_t dnh_unary(int32_t op, const DnhTensor* t, const DnhTensor* a, void* stream);
/* ITensorBackend.IsFinite (TensorBackend.fs:95; ScalarPrimitives.fs:181-188): bool target; true for every integer. */
int32_t dnh_is_finite(const DnhTensor* t_bool, const DnhTensor* a, void* stream);
/* Binary ops, DnhBinaryOp (And/Or/Xor take bool operands). */
int32_t dnh_binary(int32_t op, const DnhTensor* t, const DnhTensor* a, const DnhTensor* b, void* stream);
/* Comparisons, DnhCompareOp, into a bool target. */
int32_t dnh_compare(int32_t op, const DnhTensor* t_bool, const DnhTensor* a, const DnhTensor* b, void* stream);
/* ITensorBackend.IfThenElse (TensorBackend.fs:118; Host/ScalarOps.fs:577-581). */
int32_t dnh_if_then_else(const DnhTensor* t, const DnhTensor* cond_bool, const DnhTensor* if_true,
                         const DnhTensor* if_false, void* stream);

/* ---------------------------------------------------------------------------------------------------
 * Reductions along the LAST axis of `src` (src.ndims == t.ndims + 1, t.shape == src.shape[0..n-2]);
 * the frontend permutes the reduced axis to the last position as a view (Tensor.fs:4544-4567), so the
 * strides of `src` are arbitrary and select the kernel strategy.
 * ------------------------------------------------------------------------------------------------- */
int32_t dnh_reduce_last_axis(int32_t op, const DnhTensor* t, const DnhTensor* src, void* stream);
/* The folds of dnh_reduce_last_axis for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid it).  No counterpart in the reference.  Same arguments, same kernels and bit-identical results;
 * the partial results of two-pass folds are kept in an array of DNH_STATIC_SCRATCH_BYTES that is part of the library's device
 * image, so the call never allocates or frees.  A fold whose partials do not fit returns DNH_ERR_NOT_SUPPORTED: folds with a state
 * as wide as their elements need at most about 4 MiB whatever the shape; only CountTrue down the columns of a bool matrix (an
 * int64 per column and chunk of 512 rows, for up to 1024 chunks x column tiles) can need more.  Every call on one GPU shares that
 * GPU's array and leaves its partials there: calls that overlap on one GPU, on any streams, race; issue them on one stream or
 * order them yourself. */
#define DNH_STATIC_SCRATCH_BYTES (8u << 20)
int32_t dnh_reduce_last_axis_noalloc(int32_t op, const DnhTensor* t, const DnhTensor* src, void* stream);
int32_t dnh_arg_reduce_last_axis(int32_t op, const DnhTensor* t_i64, const DnhTensor* src, void* stream);
/* ITensorBackend.FindLastAxis (TensorBackend.fs:135; Host/ScalarOps.fs:656-665): first index equal to *value, else DNH_NOT_FOUND. */
int32_t dnh_find_last_axis(const void* value, const DnhTensor* t_i64, const DnhTensor* src, void* stream);

/* ---------------------------------------------------------------------------------------------------
 * Indexing
 * ------------------------------------------------------------------------------------------------- */
/* ITensorBackend.Gather (TensorBackend.fs:119; Host/ScalarOps.fs:583-591).  idx has src->ndims entries, each NULL
 * (identity on that dimension) or an int64 tensor already broadcast to t's shape.  An out-of-range index sets the
 * stream's error flag (dnh_async_error) and leaves the target element unwritten; it never faults the device. */
int32_t dnh_gather(const DnhTensor* t, const DnhTensor* const* idx, int32_t n_idx, const DnhTensor* src, void* stream);
/* ITensorBackend.Scatter (TensorBackend.fs:120; Host/ScalarOps.fs:593-604): t[idx[s]] += src[s]; the frontend
 * zero-fills t first (Tensor.fs:2159).  idx has t->ndims entries broadcast to src's shape.
 * Repeated indices: integer sums wrap and are the same in any order.  Single and double: every target element receives its sources
 * one after the other in the row-major order of src, which is the order of the reference's loop, so the result has the reference's
 * bits and is the same on every run (the sources are sorted by target element first; workspace of about 20 bytes per source element,
 * DNH_ERR_OUT_OF_MEMORY when it cannot be had).  dnh_set_option("scatter_fp_atomic", 1) selects float atomics instead: no workspace,
 * faster for few repeats, but the order of a cell's additions then varies from run to run; either way a target element that m_j
 * sources name is within m_j u sum|src_s| of the exact sum (u = unit roundoff). */
int32_t dnh_scatter(const DnhTensor* t, const DnhTensor* const* idx, int32_t n_idx, const DnhTensor* src, void* stream);
/* How much of the stream's workspace a dnh_scatter of `sources` elements into a target of `cells` elements asks for (no counterpart in
 * the reference; for hosts that plan device memory): 0 for the forms that need none (atomics), the sorted pairs and counters of the
 * binned form for 32-bit integers on rank-1 contiguous tensors when that form is chosen, about 20 bytes per source for the ordered
 * floating-point form.  Touches no device. */
int32_t dnh_scatter_workspace_bytes(int32_t dtype, int64_t sources, int64_t cells, size_t* bytes);
/* ITensorBackend.CountTrue is dnh_reduce_last_axis(DNH_COUNT_TRUE).
 * ITensorBackend.MaskedGet (TensorBackend.fs:121; Host/ScalarOps.fs:667-681): masks has src->ndims entries, each NULL
 * or a rank-1 bool tensor of length src->shape[d]; selected elements are written to t in row-major order. */
int32_t dnh_masked_get(const DnhTensor* t, const DnhTensor* src, const DnhTensor* const* masks, int32_t n_masks, void* stream);
/* ITensorBackend.MaskedSet (TensorBackend.fs:122; Host/ScalarOps.fs:683-697). */
int32_t dnh_masked_set(const DnhTensor* t, const DnhTensor* const* masks, int32_t n_masks, const DnhTensor* src, void* stream);
/* ITensorBackend.TrueIndices (TensorBackend.fs:123; Host/ScalarOps.fs:699-707): t is [nTrue; src.ndims] int64. */
int32_t dnh_true_indices(const DnhTensor* t_i64, const DnhTensor* src_bool, void* stream);

/* ---------------------------------------------------------------------------------------------------
 * Dot: ITensorBackend VecVecDot / MatVecDot / MatMatDot / BatchedMatMatDot (TensorBackend.fs:137-140;
 * Host/HostBackend.fs:463-546).  The ranks of (t, a, b) select the variant exactly as Tensor.FillDot does
 * (Tensor.fs:2714-2730): (0,1,1) (1,2,1) (2,2,2) or (n,n,n) with n>2.  fp32 and fp64 on the matrix cores.  Single-precision
 * operands that are contiguous along one of their two dimensions, with K >= 16, run on the bf16 instructions with every float cut
 * into three bf16 parts (six of the nine partial products; error within 16 u S of the exact product like an fp32 sgemm, u = 2^-24,
 * S = sum_k |a_ik||b_kj|); tiles whose operands hold an infinite element or a nonzero element below 2^-109, which cannot be cut
 * exactly, are computed with the fp32 instruction, so infinities and NaNs come out as IEEE arithmetic (the reference's sgemm) gives
 * them.  dnh_set_option("dot_bf16x3", 0) keeps every product on the fp32 instruction (a tuning switch, same results contract).
 * Denormal operands are honoured, but the single-precision matrix instruction flushes products and partial sums below 2^-126 to
 * zero: results carry an absolute error of up to K x 2^-126 on top of the bound.  The integer types wrap like the host backend's
 * multiply + sumAxis (HostBackend.fs:544-546); bool: status 2.
 * ------------------------------------------------------------------------------------------------- */
int32_t dnh_dot(const DnhTensor* t, const DnhTensor* a, const DnhTensor* b, void* stream);

/* ITensorBackend.BatchedInvert (TensorBackend.fs:144; Host/HostBackend.fs:548-576 LAPACK getrf + getri;
 * Cuda/CudaBackend.fs:451-484 getrfBatched + getriBatched).  t and src have shape [b_1..b_k; n; n] (src broadcast to
 * t's shape by the frontend, Tensor.fs:2811-2815), single or double; any strides; t may be src.  Gauss-Jordan with row pivoting:
 * partial pivoting for matrices of up to 32 rows, tournament pivoting (the 32 pivot rows of a block of columns elected by games of
 * partial pivoting among groups of rows) above, see the option "invert_tournament"; either way the result is an inverse computed
 * by a backward-stable elimination (in the tests within 8 n eps cond(A) max|inv(A)| of the exact inverse, as LAPACK's is), not
 * LAPACK's bits.  A pivot that is
 * exactly zero gives DNH_ERR_SINGULAR_MATRIX (LAPACK info > 0).  Synchronises the stream to read that flag. */
int32_t dnh_batched_invert(const DnhTensor* t, const DnhTensor* src, void* stream);

/* ITensorBackend.BatchedSVD (TensorBackend.fs:143; Host/HostBackend.fs:579-606 LAPACK gesdd with job 'A' or 'N'; not implemented
 * by the reference's CUDA backend, Cuda/CudaBackend.fs:486-488).  src [b_1..b_k; M; N], single or double, any strides.
 * s [b..; min(M, N)] receives the singular values in descending order.  u [b..; M; M] and v [b..; N; N] are both given (then
 * src = u diag(s) v^T with u, v orthogonal) or both NULL (singular values only).  One-sided Jacobi rotations; synchronises
 * the stream once per sweep; DNH_ERR_NO_CONVERGENCE if a matrix is not diagonal after 60 sweeps. */
int32_t dnh_batched_svd(const DnhTensor* s, const DnhTensor* u, const DnhTensor* v, const DnhTensor* src, void* stream);

/* ITensorBackend.SymmetricEigenDecomposition (TensorBackend.fs:145; Host/HostBackend.fs:608-628 LAPACK syevd 'V'; not implemented
 * by the reference's CUDA backend, Cuda/CudaBackend.fs:490-492).  src [n; n]; only the triangle named by part (0 = upper,
 * 1 = lower, MatrixPart in Tensor/Tensor/TensorBackend.fs) is read.  eigvals [n] receives the eigenvalues in ascending order,
 * column k of eigvecs [n; n] the unit eigenvector of eigenvalue k.  eigvecs may be src. */
int32_t dnh_symmetric_eig(int32_t part, const DnhTensor* eigvals, const DnhTensor* eigvecs, const DnhTensor* src, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TENSOR_HIP_H */
