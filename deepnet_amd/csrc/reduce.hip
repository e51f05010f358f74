// dnh_reduce_last_axis, dnh_arg_reduce_last_axis, dnh_find_last_axis:
// ITensorBackend SumLastAxis..CountTrueLastAxis, ArgMin/ArgMaxLastAxis, FindLastAxis (Tensor/Tensor/TensorBackend.fs:125-135).
// Fold semantics follow Tensor/Tensor/Host/ScalarOps.fs:606-665: sum from zero, product from one, max from minValue<T>
// with `if res > v then res else v`, min from maxValue<T>, all from true, any from false, countTrue into int64; an empty
// axis yields the initial value.  Float sums and products are re-associated (tree order); Max / Min of floats follow the sequential
// rule for NaNs as well (RMax); everything else is order-independent.
#include "reduce_kernels.h"
#include "ops.h"

#include <mutex>

using namespace dnh;

namespace {

template <class X> struct RSum {
    using In = X; using State = X; using Out = X;
    __device__ X init() const { return X(0); }
    __device__ X step(X s, X v, int64_t) const { return OpAdd<X>{}(s, v); }
    __device__ X combine(X a, X b) const { return OpAdd<X>{}(a, b); }
    __device__ X extract(X s) const { return s; }
};
template <class X> struct RProd {
    using In = X; using State = X; using Out = X;
    __device__ X init() const { return X(1); }
    __device__ X step(X s, X v, int64_t) const { return OpMul<X>{}(s, v); }
    __device__ X combine(X a, X b) const { return OpMul<X>{}(a, b); }
    __device__ X extract(X s) const { return s; }
};
// Max / Min follow the reference's sequential rule `if res > v then res else v` from minValue (Host/ScalarOps.fs:620-628).  Without
// NaNs any order gives the same value: the larger of minValue and the true maximum.  With a NaN the rule depends on the order: the NaN
// replaces the running value, and the next element replaces the NaN, so the result is the plain maximum of what follows the last NaN
// (NaN if it comes last; minValue plays no part any more).  The tree therefore starts from -inf, carries a NaN through every step and
// combination (a result that met one is a NaN) and applies minValue when it extracts; a NaN result is recomputed from the axis:
// the threads that share a row look for its last NaN and fold what follows (reduce_rows_kernel: fix_rows), a thread that owns a
// column walks it in order (sequential).  Partials of a two-pass fold are true maxima, so only the last chunk that holds a NaN is
// read again.  Faithful for every input, at one extra comparison per element for NaN-free data.
template <class X, bool MAX> struct RExtreme {
    using In = X; using State = X; using Out = X;
    static constexpr bool kFloat = std::is_floating_point<X>::value;
    static constexpr bool kSeqFix = kFloat;
    // where the reference's fold starts
    __device__ static X start() { return MAX ? std::numeric_limits<X>::lowest() : std::numeric_limits<X>::max(); }
    // neutral element of pick()
    __device__ static X identity() {
        if constexpr (kFloat) return MAX ? -std::numeric_limits<X>::infinity() : std::numeric_limits<X>::infinity();
        else return start();
    }
    __device__ static bool beats(X a, X b) { return MAX ? a > b : a < b; }
    __device__ static X pick(X a, X b) { return beats(a, b) ? a : b; }              // the reference's step; NaN-free operands commute
    __device__ X init() const { return identity(); }
    __device__ X step(X s, X v, int64_t) const { return (beats(s, v) || s != s) ? s : v; }
    __device__ X combine(X a, X b) const { return (beats(a, b) || a != a) ? a : b; }
    __device__ X extract(X s) const { return pick(start(), s); }
    __device__ bool needs_fix(X s) const { return s != s; }
    // the reference's fold over p[0], p[stride] .. p[(n - 1) stride] continued from s
    __device__ X sequential(X s, const X* p, int64_t n, int64_t stride) const {
        int64_t i = 0;
        for (; i + 16 <= n; i += 16) {   // sixteen fetches on their way at a time, applied in order
            X v[16];
#pragma unroll
            for (int u = 0; u < 16; u++) v[u] = p[(i + u) * stride];
#pragma unroll
            for (int u = 0; u < 16; u++) s = pick(s, v[u]);
        }
        for (; i < n; i++) s = pick(s, p[i * stride]);
        return s;
    }
};
template <class X> using RMax = RExtreme<X, true>;
template <class X> using RMin = RExtreme<X, false>;
struct RAll {
    using In = uint8_t; using State = uint8_t; using Out = uint8_t;
    __device__ uint8_t init() const { return 1; }
    __device__ uint8_t step(uint8_t s, uint8_t v, int64_t) const { return (uint8_t)(s & (v != 0)); }
    __device__ uint8_t combine(uint8_t a, uint8_t b) const { return (uint8_t)(a & b); }
    __device__ uint8_t extract(uint8_t s) const { return s; }
};
struct RAny {
    using In = uint8_t; using State = uint8_t; using Out = uint8_t;
    __device__ uint8_t init() const { return 0; }
    __device__ uint8_t step(uint8_t s, uint8_t v, int64_t) const { return (uint8_t)(s | (v != 0)); }
    __device__ uint8_t combine(uint8_t a, uint8_t b) const { return (uint8_t)(a | b); }
    __device__ uint8_t extract(uint8_t s) const { return s; }
};
struct RCountTrue {
    using In = uint8_t; using State = int64_t; using Out = int64_t;
    __device__ int64_t init() const { return 0; }
    __device__ int64_t step(int64_t s, uint8_t v, int64_t) const { return s + (v != 0); }
    __device__ int64_t combine(int64_t a, int64_t b) const { return a + b; }
    __device__ int64_t extract(int64_t s) const { return s; }
};

template <class X, class P> struct ArgState {
    X val;
    P pos;
};
// State starts at (NotFound, minValue|maxValue) and is replaced only by a strictly better value, so a position is set
// only together with a value better than the initial one; equal values therefore are either both unset or both set, and
// taking the smaller position on a tie reproduces "first index wins" under any combine order.
// P: the position's type inside the state.  int64, or uint32 (with 0xFFFFFFFF for NotFound) for 4-byte elements on axes shorter than
// 2^32 - 1: the state is then 8 bytes instead of 16, which halves the partial results of two-pass folds and lets the column kernel
// take its 256-lane form.
template <class X, bool MAX, class P> struct RArg {
    using In = X; using State = ArgState<X, P>; using Out = int64_t;
    static constexpr P kNone = std::is_same<P, int64_t>::value ? (P)DNH_NOT_FOUND : (P)0xFFFFFFFFu;
    __device__ static bool better(X a, X b) { return MAX ? a > b : a < b; }
    __device__ State init() const { return State{MAX ? std::numeric_limits<X>::lowest() : std::numeric_limits<X>::max(), kNone}; }
    __device__ State step(State s, X v, int64_t i) const { return better(v, s.val) ? State{v, (P)i} : s; }
    __device__ State combine(State a, State b) const {
        const bool takeb = better(b.val, a.val) || (b.val == a.val && b.pos < a.pos);
        return takeb ? b : a;
    }
    __device__ int64_t extract(State s) const { return s.pos == kNone ? DNH_NOT_FOUND : (int64_t)s.pos; }
};
template <class X> struct RFind {
    using In = X; using State = int64_t; using Out = int64_t;
    X value;
    __device__ int64_t init() const { return DNH_NOT_FOUND; }
    __device__ int64_t step(int64_t s, X v, int64_t i) const { return (s == DNH_NOT_FOUND && v == value) ? i : s; }
    __device__ int64_t combine(int64_t a, int64_t b) const {
        if (a == DNH_NOT_FOUND) return b;
        if (b == DNH_NOT_FOUND) return a;
        return a < b ? a : b;
    }
    __device__ int64_t extract(int64_t s) const { return s; }
};

template <template <class> class RT>
int32_t run_numeric(const DnhTensor* t, const DnhTensor* s, hipStream_t st, const char* what, const PartialStore& ps) {
    switch (s->dtype) {
        case DNH_U8: return launch_reduce(RT<uint8_t>{}, t, s, st, what, ps);
        case DNH_I8: return launch_reduce(RT<int8_t>{}, t, s, st, what, ps);
        case DNH_I16: return launch_reduce(RT<int16_t>{}, t, s, st, what, ps);
        case DNH_U16: return launch_reduce(RT<uint16_t>{}, t, s, st, what, ps);
        case DNH_I32: return launch_reduce(RT<int32_t>{}, t, s, st, what, ps);
        case DNH_U32: return launch_reduce(RT<uint32_t>{}, t, s, st, what, ps);
        case DNH_I64: return launch_reduce(RT<int64_t>{}, t, s, st, what, ps);
        case DNH_U64: return launch_reduce(RT<uint64_t>{}, t, s, st, what, ps);
        case DNH_F32: return launch_reduce(RT<float>{}, t, s, st, what, ps);
        case DNH_F64: return launch_reduce(RT<double>{}, t, s, st, what, ps);
    }
    return fail(DNH_ERR_NOT_SUPPORTED, "%s is not defined for %s", what, dtype_name(s->dtype));
}

template <bool MAX>
int32_t run_arg(const DnhTensor* t, const DnhTensor* s, hipStream_t st, const char* what) {
    const bool short_axis = s->ndims >= 1 && s->shape[s->ndims - 1] < 0xFFFFFFFFLL;
    switch (s->dtype) {
        case DNH_U8: return launch_reduce(RArg<uint8_t, MAX, int64_t>{}, t, s, st, what);
        case DNH_I8: return launch_reduce(RArg<int8_t, MAX, int64_t>{}, t, s, st, what);
        case DNH_I16: return launch_reduce(RArg<int16_t, MAX, int64_t>{}, t, s, st, what);
        case DNH_U16: return launch_reduce(RArg<uint16_t, MAX, int64_t>{}, t, s, st, what);
        case DNH_I32: return short_axis ? launch_reduce(RArg<int32_t, MAX, uint32_t>{}, t, s, st, what) : launch_reduce(RArg<int32_t, MAX, int64_t>{}, t, s, st, what);
        case DNH_U32: return short_axis ? launch_reduce(RArg<uint32_t, MAX, uint32_t>{}, t, s, st, what) : launch_reduce(RArg<uint32_t, MAX, int64_t>{}, t, s, st, what);
        case DNH_I64: return launch_reduce(RArg<int64_t, MAX, int64_t>{}, t, s, st, what);
        case DNH_U64: return launch_reduce(RArg<uint64_t, MAX, int64_t>{}, t, s, st, what);
        case DNH_F32: return short_axis ? launch_reduce(RArg<float, MAX, uint32_t>{}, t, s, st, what) : launch_reduce(RArg<float, MAX, int64_t>{}, t, s, st, what);
        case DNH_F64: return launch_reduce(RArg<double, MAX, int64_t>{}, t, s, st, what);
    }
    return fail(DNH_ERR_NOT_SUPPORTED, "%s is not defined for %s", what, dtype_name(s->dtype));
}

}  // namespace

// ---- CountTrue of a whole contiguous mask in one launch -----------------------------------------------------------------------------
// The general fold needs a second, dependent launch to add the workgroups' partial counts.  Integer counts can be added in any order,
// so here the workgroups meet through device-scope atomics instead: a workgroup adds (count | 1 << 48) to the word of its group of 16
// workgroups; the one that finds 15 arrivals before it carries the group's sum on to the top word in the same way, and the last
// arrival there stores the result.  One atomic carries count and arrival together, so no ordering between locations is relied on,
// and no more than 16 workgroups (or groups) ever meet on one address.  Each last arrival puts its word back to zero for the next launch.
namespace {
constexpr int kCountGroup = 16;
constexpr unsigned long long kCountArrival = 1ull << 48, kCountMask = kCountArrival - 1;

__global__ __launch_bounds__(kBlock) void count_true_kernel(const uint8_t* __restrict__ mask, int64_t n, int64_t per_block, uint32_t nblocks,
                                                            unsigned long long* top, unsigned long long* groups, int64_t* out) {
    const int64_t r0 = (int64_t)blockIdx.x * per_block;
    const int64_t r1 = r0 + per_block < n ? r0 + per_block : n;
    uint32_t c = 0;
    // per_block is a multiple of 16 x kBlock and the mask is 4-byte aligned: whole 16-byte pieces, then the last few bytes one by one
    constexpr int U = 4;
    int64_t i = r0 + (int64_t)threadIdx.x * 16;
    for (; i + (U - 1) * kBlock * 16 + 16 <= r1; i += (int64_t)U * kBlock * 16) {
        Pack<uint32_t, 4> v[U];
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = load_pack<uint32_t, 4>((const uint32_t*)(mask + i + (int64_t)u * kBlock * 16));
#pragma unroll
        for (int u = 0; u < U; u++)
#pragma unroll
            for (int w = 0; w < 4; w++) {
                const uint32_t x = v[u].v[w];
                c += ((x & 0xFFu) != 0) + ((x & 0xFF00u) != 0) + ((x & 0xFF0000u) != 0) + ((x & 0xFF000000u) != 0);
            }
    }
    for (; i < r1; i += (int64_t)kBlock * 16) {
        if (i + 16 <= r1) {
            const Pack<uint32_t, 4> v = load_pack<uint32_t, 4>((const uint32_t*)(mask + i));
#pragma unroll
            for (int w = 0; w < 4; w++) {
                const uint32_t x = v.v[w];
                c += ((x & 0xFFu) != 0) + ((x & 0xFF00u) != 0) + ((x & 0xFF0000u) != 0) + ((x & 0xFF000000u) != 0);
            }
        } else {
            for (int64_t j = i; j < r1; j++) c += mask[j] != 0;
        }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) c += (uint32_t)__shfl_xor((int)c, m, 64);
    __shared__ uint32_t part[kBlock / 64];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = c;
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned long long total = 0;
#pragma unroll
        for (int w = 0; w < kBlock / 64; w++) total += part[w];
        const uint32_t g = blockIdx.x / kCountGroup, ngroups = (nblocks + kCountGroup - 1) / kCountGroup;
        const uint32_t gsize = g + 1 < ngroups ? (uint32_t)kCountGroup : nblocks - g * kCountGroup;
        const unsigned long long was = __hip_atomic_fetch_add(groups + g, total | kCountArrival, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if ((was >> 48) == gsize - 1) {
            const unsigned long long gsum = (was & kCountMask) + total;
            __hip_atomic_store(groups + g, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const unsigned long long twas = __hip_atomic_fetch_add(top, gsum | kCountArrival, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if ((twas >> 48) == ngroups - 1) {
                out[0] = (int64_t)((twas & kCountMask) + gsum);
                __hip_atomic_store(top, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
}

// Takes CountTrue of one contiguous run of bools into a single int64 when that is worth a launch of its own shape.
bool try_count_true_one_launch(const DnhTensor* t, const DnhTensor* src, hipStream_t stream, int32_t* status) {
    if (option(OPT_COUNT_ONE_LAUNCH) == 0 || nelems(t) != 1 || src->ndims < 1) return false;
    const int64_t n = src->shape[src->ndims - 1];
    for (int d = 0; d + 1 < src->ndims; d++)
        if (src->shape[d] != 1) return false;
    const uint8_t* mask = (const uint8_t*)elem_ptr(src);
    if (src->stride[src->ndims - 1] != 1 || n < (1 << 20) || n >= ((int64_t)1 << 47) || ((uintptr_t)mask & 3) != 0) return false;
    const int64_t piece = (int64_t)16 * kBlock;   // bytes one round of a workgroup's loads covers
    int64_t nblocks = 2 * (int64_t)device_cus();
    int64_t per_block = ((n + nblocks - 1) / nblocks + piece - 1) / piece * piece;
    nblocks = (n + per_block - 1) / per_block;
    if (nblocks > (int64_t)kCountGroup * (int64_t)kSyncMaxCountGroups) return false;
    char* words = nullptr;
    uint32_t epoch = 0;
    WorkspaceLease lease;
    *status = sync_words(stream, kSyncTileWords, (void**)&words, &epoch, lease);
    if (*status != DNH_OK) return true;
    hipLaunchKernelGGL(count_true_kernel, dim3((unsigned)nblocks), dim3(kBlock), 0, stream, mask, n, per_block, (uint32_t)nblocks,
                       (unsigned long long*)(words + kSyncCountTop), (unsigned long long*)(words + kSyncCountGroups), (int64_t*)elem_ptr(t));
    *status = hipGetLastError() == hipSuccess ? DNH_OK : fail(DNH_ERR_HIP, "CountTrue: launch failed");
    return true;
}
}  // namespace

// The folds of dnh_reduce_last_axis; `ps` says where the partial results of a two-pass fold are kept.
static int32_t reduce_impl(const char* entry, int32_t op, const DnhTensor* t, const DnhTensor* src, hipStream_t st, const PartialStore& ps) {
    DNH_TRY(check_tensor(t, entry));
    DNH_TRY(check_tensor(src, entry));
    if (op == DNH_ALL || op == DNH_ANY) {
        if (src->dtype != DNH_BOOL || t->dtype != DNH_BOOL) return fail(DNH_ERR_INVALID_ARG, "All/Any need bool source and target");
        return op == DNH_ALL ? launch_reduce(RAll{}, t, src, st, "AllLastAxis", ps) : launch_reduce(RAny{}, t, src, st, "AnyLastAxis", ps);
    }
    if (op == DNH_COUNT_TRUE) {
        if (src->dtype != DNH_BOOL || t->dtype != DNH_I64) return fail(DNH_ERR_INVALID_ARG, "CountTrue needs a bool source and an int64 target");
        if (t->ndims + 1 == src->ndims && !ps.fixed) {   // (the entry point that may not allocate keeps the general fold: the arrival words
            int32_t cst = DNH_OK;                        //  live in a buffer the library allocates on a stream's first use)
            if (try_count_true_one_launch(t, src, st, &cst)) return cst;
        }
        return launch_reduce(RCountTrue{}, t, src, st, "CountTrueLastAxis", ps);
    }
    if (t->dtype != src->dtype) return fail(DNH_ERR_INVALID_ARG, "%s: target is %s but source is %s", entry, dtype_name(t->dtype), dtype_name(src->dtype));
    switch (op) {
        case DNH_SUM: return run_numeric<RSum>(t, src, st, "SumLastAxis", ps);
        case DNH_PRODUCT: return run_numeric<RProd>(t, src, st, "ProductLastAxis", ps);
        case DNH_MIN: return run_numeric<RMin>(t, src, st, "MinLastAxis", ps);
        case DNH_MAX: return run_numeric<RMax>(t, src, st, "MaxLastAxis", ps);
    }
    return fail(DNH_ERR_INVALID_ARG, "%s: unknown op %d", entry, op);
}

extern "C" int32_t dnh_reduce_last_axis(int32_t op, const DnhTensor* t, const DnhTensor* src, void* stream) {
    DNH_TRY(ensure_init());
    return reduce_impl("dnh_reduce_last_axis", op, t, src, (hipStream_t)stream, PartialStore());
}

// ---- the fold entry point that allocates nothing ---------------------------------------------------------------------------------
// Partial results of two-pass folds live in a file-scope device array instead of the stream's workspace.  Every GPU the library runs
// on holds its own copy of the array, at its own address, until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress: the device address is looked up once per device and that pointer is what the kernels receive.
static __device__ __align__(256) unsigned char scratch[DNH_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxScratchDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxScratchDevices] = {};

// Device address of `scratch` on the calling thread's current device (looked up on the first call per device).
int32_t static_scratch(void** out) {
    int dev = -1;
    DNH_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxScratchDevices) return fail(DNH_ERR_NOT_SUPPORTED, "static scratch: device %d outside 0..%d", dev, kMaxScratchDevices - 1);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        DNH_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fail(DNH_ERR_HIP, "static scratch: hipGetSymbolAddress returned a null address");
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return DNH_OK;
}
}  // namespace

extern "C" int32_t dnh_reduce_last_axis_noalloc(int32_t op, const DnhTensor* t, const DnhTensor* src, void* stream) {
    DNH_TRY(ensure_init());
    PartialStore ps;
    DNH_TRY(static_scratch(&ps.fixed));
    ps.fixed_bytes = DNH_STATIC_SCRATCH_BYTES;
    // Partials are written by the first pass before the second reads them, so nothing in the array has to start at zero.
    return reduce_impl("dnh_reduce_last_axis_noalloc", op, t, src, (hipStream_t)stream, ps);
}

extern "C" int32_t dnh_arg_reduce_last_axis(int32_t op, const DnhTensor* t, const DnhTensor* src, void* stream) {
    DNH_TRY(ensure_init());
    DNH_TRY(check_tensor(t, "dnh_arg_reduce_last_axis"));
    DNH_TRY(check_tensor(src, "dnh_arg_reduce_last_axis"));
    if (t->dtype != DNH_I64) return fail(DNH_ERR_INVALID_ARG, "dnh_arg_reduce_last_axis: target must be int64");
    hipStream_t st = (hipStream_t)stream;
    if (op == DNH_ARG_MAX) return run_arg<true>(t, src, st, "ArgMaxLastAxis");
    if (op == DNH_ARG_MIN) return run_arg<false>(t, src, st, "ArgMinLastAxis");
    return fail(DNH_ERR_INVALID_ARG, "dnh_arg_reduce_last_axis: unknown op %d", op);
}

extern "C" int32_t dnh_find_last_axis(const void* value, const DnhTensor* t, const DnhTensor* src, void* stream) {
    DNH_TRY(ensure_init());
    DNH_TRY(check_tensor(t, "dnh_find_last_axis"));
    DNH_TRY(check_tensor(src, "dnh_find_last_axis"));
    if (!value) return fail(DNH_ERR_INVALID_ARG, "dnh_find_last_axis: null value");
    if (t->dtype != DNH_I64) return fail(DNH_ERR_INVALID_ARG, "dnh_find_last_axis: target must be int64");
    hipStream_t st = (hipStream_t)stream;
#define CASE(DT, X) case DT: { X v; memcpy(&v, value, sizeof(X)); return launch_reduce(RFind<X>{v}, t, src, st, "FindLastAxis"); }
    switch (src->dtype) {
        CASE(DNH_BOOL, uint8_t) CASE(DNH_U8, uint8_t) CASE(DNH_I8, int8_t) CASE(DNH_I16, int16_t) CASE(DNH_U16, uint16_t) CASE(DNH_I32, int32_t) CASE(DNH_U32, uint32_t)
        CASE(DNH_I64, int64_t) CASE(DNH_U64, uint64_t) CASE(DNH_F32, float) CASE(DNH_F64, double)
    }
#undef CASE
    return fail(DNH_ERR_NOT_SUPPORTED, "FindLastAxis on unknown dtype");
}
