// Shared host-side helpers of libtensor_hip: status/error plumbing, dtype utilities, descriptor validation and the
// dimension-collapsing planner that turns n-d strided operands into the few shapes the kernels specialise on.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>

#include "../../include/tensor_hip.h"

namespace dnh {

// ---- errors -----------------------------------------------------------------------------------------------------------

std::string& last_error();  // thread-local message (runtime.hip)

inline int32_t fail(int32_t code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    last_error() = buf;
    return code;
}

#define DNH_HIP(expr)                                                                                          \
    do {                                                                                                       \
        hipError_t _e = (expr);                                                                                \
        if (_e != hipSuccess)                                                                                  \
            return ::dnh::fail(_e == hipErrorOutOfMemory ? DNH_ERR_OUT_OF_MEMORY : DNH_ERR_HIP, "%s failed: %s", \
                               #expr, hipGetErrorString(_e));                                                  \
    } while (0)

#define DNH_TRY(expr)                  \
    do {                               \
        int32_t _s = (expr);           \
        if (_s != DNH_OK) return _s;   \
    } while (0)

// Checks the launch that was just issued.
#define DNH_LAUNCH_CHECK() DNH_HIP(hipGetLastError())

int32_t ensure_init();                       // DNH_ERR_NOT_INITIALIZED-free lazy init on the current device
int device_cus();                            // compute units of the active device
int32_t error_flag_ptr(hipStream_t stream, int32_t** out);   // the stream's device int32 set by gather/scatter kernels on a bad index
// Per-stream scratch buffer owned by the library (partials of two-pass reductions and split products, block counts of
// compactions); it grows on demand.  Kernels of one stream run in order, so the buffer is free again as soon as the kernels that
// use it are queued; the lease keeps other host threads that enqueue on the same stream out until then.  Declare the lease in the
// scope that issues every launch touching the buffer; asking twice with one lease is fine.
class WorkspaceLease {
public:
    WorkspaceLease() = default;
    WorkspaceLease(const WorkspaceLease&) = delete;
    WorkspaceLease& operator=(const WorkspaceLease&) = delete;
    ~WorkspaceLease() { release(); }
    void release() {
        if (held_) held_->unlock();
        held_ = nullptr;
    }

private:
    friend int32_t workspace(hipStream_t stream, size_t bytes, void** out, WorkspaceLease& lease);
    friend int32_t sync_words(hipStream_t stream, size_t bytes, void** out, uint32_t* epoch, WorkspaceLease& lease);
    std::mutex* held_ = nullptr;
};
int32_t workspace(hipStream_t stream, size_t bytes, void** out, WorkspaceLease& lease);
// A second per-stream buffer, for the words through which the workgroups of ONE launch meet (arrival counters, tile descriptors).  It is zero when first handed out and is used for nothing else, so kernels may leave it in the state the next
// launch expects (counters back at zero) and tag what they cannot reset with `epoch`, a number no earlier launch on the stream used
// (30 bits; the buffer is cleared when it wraps).  Same lease discipline as workspace().
int32_t sync_words(hipStream_t stream, size_t bytes, void** out, uint32_t* epoch, WorkspaceLease& lease);
// Layout of that buffer: counters that every launch leaves at zero in front, epoch-tagged words behind them.
constexpr size_t kSyncCountTop = 64;       // uint64: arrival word of the one-launch CountTrue
constexpr size_t kSyncCountGroups = 128;   // uint64 x up to kSyncMaxCountGroups: its per-group arrival words
constexpr size_t kSyncMaxCountGroups = 496;
constexpr size_t kSyncTileWords = 4096;    // uint64 per tile, epoch-tagged

// ---- tuning switches --------------------------------------------------------------------------------------------------
// Process-wide integers behind dnh_set_option / dnh_get_option.  Each starts from an environment variable of the same name in
// upper case with a DNH_ prefix (dot_bf16x3 <- DNH_DOT_BF16X3) or, without one, from the default below; a change applies to the
// calls issued after it.  None of them changes a result's contract, only which kernel computes it.
enum Option {
    OPT_DOT_BF16X3 = 0,      // 1: single-precision products on the bf16 matrix instructions (three parts per float); 0: fp32 instruction
    OPT_DOT_F64_PINNED,      // 1: double-precision products on gemm_f64_kernel where the layout allows; 0: gemm_kernel<double>
    OPT_DOT_BIG,             // -1: the cost model picks the tile form of the bf16-parts kernel; 0 / 1: 128 x 128 / 256 x 256 tiles
    OPT_DOT_SPLITS,          // 0: the cost model picks the number of chunks along K; n > 0: that many
    OPT_DOT_INT_MFMA,        // 1: 32 / 64-bit integer products on the int8 matrix instruction; 0: gemm_int_kernel
    OPT_TR4,                 // 1: 4-byte transposing copies through LDS where the layout asks for them; 0: the general n-d kernel
    OPT_SCATTER_FP_ATOMIC,   // 0: floating-point scatter adds duplicates in source order (reproducible); 1: float atomics
    OPT_COMPACT_ONE_PASS,    // 1: maskedGet / maskedSet / trueIndices of contiguous masks in one launch; 0: count + move launches
    OPT_COUNT_ONE_LAUNCH,    // 1: countTrue of a whole contiguous mask in one launch (arrival counters); 0: the general two-pass fold
    OPT_LOOKBACK_SPINS,      // polls a one-pass compaction's tile spends on predecessors that have not published before it counts for itself
    OPT_INVERT_TOURNAMENT,   // -1: matrices of more than 32 rows pick a panel's pivots by tournament; 0: never; 1: always
    OPT_COUNT
};
int option(Option o);

// ---- dtypes -----------------------------------------------------------------------------------------------------------

inline int dtype_size(int dt) {
    switch (dt) {
        case DNH_BOOL: case DNH_U8: case DNH_I8: return 1;
        case DNH_I16: case DNH_U16: return 2;
        case DNH_I32: case DNH_U32: case DNH_F32: return 4;
        case DNH_I64: case DNH_U64: case DNH_F64: return 8;
    }
    return 0;
}
inline bool dtype_is_fp(int dt) { return dt == DNH_F32 || dt == DNH_F64; }
inline bool dtype_is_signed(int dt) { return dt == DNH_I8 || dt == DNH_I16 || dt == DNH_I32 || dt == DNH_I64 || dtype_is_fp(dt); }
inline bool dtype_is_numeric(int dt) { return dt > DNH_BOOL && dt < DNH_DTYPE_COUNT; }
inline const char* dtype_name(int dt) {
    static const char* n[] = {"bool", "uint8", "int8", "int32", "uint32", "int64", "uint64", "single", "double", "int16", "uint16"};
    return (dt >= 0 && dt < DNH_DTYPE_COUNT) ? n[dt] : "?";
}

// ---- descriptors ------------------------------------------------------------------------------------------------------

inline int32_t check_tensor(const DnhTensor* t, const char* what) {
    if (!t) return fail(DNH_ERR_INVALID_ARG, "%s: null tensor descriptor", what);
    if (t->ndims < 0 || t->ndims > DNH_MAX_DIMS) return fail(DNH_ERR_INVALID_ARG, "%s: rank %d outside 0..%d", what, t->ndims, DNH_MAX_DIMS);
    if (t->dtype < 0 || t->dtype >= DNH_DTYPE_COUNT) return fail(DNH_ERR_INVALID_ARG, "%s: unknown dtype %d", what, t->dtype);
    int64_t n = 1;
    for (int d = 0; d < t->ndims; d++) {
        if (t->shape[d] < 0) return fail(DNH_ERR_INVALID_ARG, "%s: negative extent", what);
        n *= t->shape[d];
    }
    if (n > 0 && !t->base) return fail(DNH_ERR_INVALID_ARG, "%s: null base pointer", what);
    return DNH_OK;
}

inline int64_t nelems(const DnhTensor* t) {
    int64_t n = 1;
    for (int d = 0; d < t->ndims; d++) n *= t->shape[d];
    return n;
}

inline bool same_shape(const DnhTensor* a, const DnhTensor* b) {
    if (a->ndims != b->ndims) return false;
    for (int d = 0; d < a->ndims; d++)
        if (a->shape[d] != b->shape[d]) return false;
    return true;
}

inline char* elem_ptr(const DnhTensor* t) { return (char*)t->base + t->offset * (int64_t)dtype_size(t->dtype); }

// ---- element-wise plan ------------------------------------------------------------------------------------------------

constexpr int kMaxOperands = 4;  // target + up to three sources

// Operands of one element-wise launch over a common (collapsed) index space.  Operand 0 is the target.
struct MapPlan {
    int nd;                                       // collapsed rank, 0 for a single element
    int nops;
    int64_t total;                                // number of elements
    int64_t shape[DNH_MAX_DIMS];
    int64_t stride[kMaxOperands][DNH_MAX_DIMS];   // elements
    char* ptr[kMaxOperands];                      // element 0 of each operand
    int esize[kMaxOperands];
};

// Builds the plan: drops extent-1 dimensions, orders dimensions so the target's strides decrease (its fastest dimension
// last, which makes stores coalesced whatever the logical order was — the same freedom the reference's host backend uses
// when it swaps the best dimension last, Host/HostBackend.fs:139-153) and merges neighbours that chain for every operand.
inline int32_t make_map_plan(MapPlan* p, int nops, const DnhTensor* const* ops, const char* what) {
    for (int k = 0; k < nops; k++) DNH_TRY(check_tensor(ops[k], what));
    for (int k = 1; k < nops; k++)
        if (!same_shape(ops[0], ops[k])) return fail(DNH_ERR_INVALID_ARG, "%s: operand %d does not have the target's shape", what, k);
    p->nops = nops;
    p->total = nelems(ops[0]);
    for (int k = 0; k < nops; k++) {
        p->ptr[k] = elem_ptr(ops[k]);
        p->esize[k] = dtype_size(ops[k]->dtype);
    }
    int nd = 0;
    int64_t shape[DNH_MAX_DIMS], stride[kMaxOperands][DNH_MAX_DIMS];
    for (int d = 0; d < ops[0]->ndims; d++) {
        if (ops[0]->shape[d] == 1) continue;
        shape[nd] = ops[0]->shape[d];
        for (int k = 0; k < nops; k++) stride[k][nd] = ops[k]->stride[d];
        nd++;
    }
    // normalise negative target strides away so ordering by magnitude is meaningful: flip the dimension for all operands
    for (int d = 0; d < nd; d++) {
        if (stride[0][d] < 0) {
            for (int k = 0; k < nops; k++) {
                p->ptr[k] += (shape[d] - 1) * stride[k][d] * (int64_t)p->esize[k];
                stride[k][d] = -stride[k][d];
            }
        }
    }
    // insertion sort by target stride, descending (stable)
    for (int i = 1; i < nd; i++) {
        for (int j = i; j > 0 && stride[0][j - 1] < stride[0][j]; j--) {
            std::swap(shape[j - 1], shape[j]);
            for (int k = 0; k < nops; k++) std::swap(stride[k][j - 1], stride[k][j]);
        }
    }
    // merge dimension d+1 into d when stride[d] == stride[d+1] * shape[d+1] for every operand
    int out = 0;
    for (int d = 0; d < nd; d++) {
        if (out > 0) {
            bool chain = true;
            for (int k = 0; k < nops; k++) chain = chain && stride[k][out - 1] == stride[k][d] * shape[d];
            if (chain) {
                shape[out - 1] *= shape[d];
                for (int k = 0; k < nops; k++) stride[k][out - 1] = stride[k][d];
                continue;
            }
        }
        shape[out] = shape[d];
        for (int k = 0; k < nops; k++) stride[k][out] = stride[k][d];
        out++;
    }
    p->nd = out;
    for (int d = 0; d < DNH_MAX_DIMS; d++) {
        p->shape[d] = d < out ? shape[d] : 1;
        for (int k = 0; k < kMaxOperands; k++) p->stride[k][d] = (d < out && k < nops) ? stride[k][d] : 0;
    }
    return DNH_OK;
}

inline unsigned cdiv(int64_t a, int64_t b) { return (unsigned)((a + b - 1) / b); }

}  // namespace dnh
