// Last-axis reduction kernels for gfx950.  A reducer R supplies
//   In / State / Out, init(), step(State, In, int64 index), combine(State, State), extract(State).
// Every combine below is commutative and associative (index-carrying states break value ties on the smaller index), so
// any tree order yields the reference's sequential result for order-independent folds and the first-index rule of
// ArgMin/ArgMax/Find (Tensor/Tensor/Host/ScalarOps.fs:638-665).
//
//   reduce_rows    : reduced axis has stride 1.  TPR threads (16, 64 = one wavefront, or 256 = the block) share a row,
//                    16-byte loads, several in flight, wavefront shuffle tree + one LDS step for the block variant.
//                    A long axis with few rows is split over gridDim.y into State partials (pass one of the two-pass tree).
//   reduce_cols    : a kept dimension has stride 1 instead (the frontend's "reduce along the first axis" view,
//                    Tensor.fs:4544-4567): lanes run along the kept dimension (coalesced), four wavefronts and
//                    gridDim.y splits share the reduced axis, LDS combine, partials when split.
//   reduce_rows<FROM_STATE> doubles as the finishing pass over partials.
//   reduce_generic : one thread per output, for axes too short or layouts too irregular for the above.
#pragma once

#include "map_kernels.h"

namespace dnh {

struct OuterArgs {
    int nd;
    uint32_t shape[DNH_MAX_DIMS];
    int64_t tstride[DNH_MAX_DIMS];
    int64_t sstride[DNH_MAX_DIMS];
};

__device__ __forceinline__ void outer_offsets(const OuterArgs& o, uint32_t idx, int64_t& toff, int64_t& soff) {
    toff = 0;
    soff = 0;
    for (int d = o.nd - 1; d >= 0; d--) {
        const uint32_t q = (d == 0) ? 0u : idx / o.shape[d];
        const uint32_t i = idx - q * o.shape[d];
        idx = q;
        toff += (int64_t)i * o.tstride[d];
        soff += (int64_t)i * o.sstride[d];
    }
}

template <class S>
__device__ __forceinline__ S shfl_xor_any(const S& s, int mask) {
    constexpr int W = (sizeof(S) + 3) / 4;
    uint32_t w[W] = {};
    __builtin_memcpy(w, &s, sizeof(S));
#pragma unroll
    for (int i = 0; i < W; i++) w[i] = (uint32_t)__shfl_xor((int)w[i], mask, 64);
    S r;
    __builtin_memcpy(&r, w, sizeof(S));
    return r;
}

template <class R, int GROUP>
__device__ __forceinline__ typename R::State group_reduce(const R& r, typename R::State s) {
#pragma unroll
    for (int m = (GROUP < 64 ? GROUP : 64) / 2; m >= 1; m >>= 1) s = r.combine(s, shfl_xor_any(s, m));
    return s;
}

// A fold may name results that the tree cannot produce faithfully (kSeqFix: Max / Min of floats that met a NaN, whose value under
// the reference's sequential rule depends on where the NaN stood).  Such a reducer also supplies start(), identity(), pick(),
// needs_fix() and sequential(); a result that needs_fix() is recomputed from the reduced axis (elements p[0], p[stride] ..
// p[(n - 1) stride]).  Rare by construction; every other result is extract(state).
template <class R, class = void> struct NeedsSeqFix : std::false_type {};
template <class R> struct NeedsSeqFix<R, std::void_t<decltype(R::kSeqFix)>> : std::integral_constant<bool, R::kSeqFix> {};

// By the one thread that owns the result (column and one-thread-per-output kernels): the whole axis in order.
template <class R>
__device__ __forceinline__ typename R::Out finish_value(const R& r, const typename R::State& s, const typename R::In* p, int64_t n, int64_t stride) {
    if constexpr (NeedsSeqFix<R>::value) {
        if (r.needs_fix(s)) return r.sequential(R::start(), p, n, stride);
    }
    return r.extract(s);
}

// The same for a two-pass fold whose partials q[0], q[qstride] .. q[(splits - 1) qstride] are true folds of chunks of `chunk`
// elements (NaN when the chunk holds one): only the last chunk with a NaN is walked, the partials behind it continue the fold.
template <class R>
__device__ __forceinline__ typename R::Out finish_value_chunked(const R& r, const typename R::State& s, const typename R::State* q, int64_t qstride,
                                                                uint32_t splits, const typename R::In* p, int64_t n, int64_t stride, int64_t chunk) {
    if constexpr (NeedsSeqFix<R>::value) {
        if (r.needs_fix(s)) {
            int64_t j = (int64_t)splits - 1;
            while (j > 0 && !r.needs_fix(q[j * qstride])) j--;
            const int64_t c0 = j * chunk, c1 = (c0 + chunk < n) ? c0 + chunk : n;
            typename R::State v = r.sequential(R::start(), p + c0 * stride, c1 - c0, stride);
            for (int64_t k = j + 1; k < (int64_t)splits; k++) v = R::pick(v, q[k * qstride]);
            return v;
        }
    }
    return r.extract(s);
}

// All-reduce of v over the G threads that share a row (threads `threadIdx.x % G` of a group are consecutive): shuffles inside a
// wavefront; G = kBlock: the wavefronts' values meet in `sh` (kBlock / 64 words of 8 bytes), every thread of the block calls.
template <int G, class V, class F>
__device__ __forceinline__ V group_all_reduce(V v, F f, uint64_t* sh) {
#pragma unroll
    for (int m = (G < 64 ? G : 64) / 2; m >= 1; m >>= 1) v = f(v, shfl_xor_any(v, m));
    if constexpr (G > 64) {
        static_assert(sizeof(V) <= 8, "group_all_reduce: value wider than a slot");
        __syncthreads();   // an earlier use of sh is over
        if ((threadIdx.x & 63) == 0) __builtin_memcpy(&sh[threadIdx.x / 64], &v, sizeof(V));
        __syncthreads();
        __builtin_memcpy(&v, &sh[0], sizeof(V));
#pragma unroll
        for (int w = 1; w < G / 64; w++) {
            V o;
            __builtin_memcpy(&o, &sh[w], sizeof(V));
            v = f(v, o);
        }
    }
    return v;
}

// The reference's sequential Max / Min over elements i0 .. i1 - 1 of an axis, for a range known to hold a NaN, by the G threads that
// share the row: the position of the last NaN, then the plain fold of what follows it (NaN when nothing does).
template <class R, int G>
__device__ __forceinline__ typename R::In fold_after_last_nan(const typename R::In* p, int64_t i0, int64_t i1, int64_t stride, uint32_t lane,
                                                              uint64_t* sh) {
    using X = typename R::In;
    int64_t q = i0 - 1;
#pragma unroll 4
    for (int64_t i = i0 + lane; i < i1; i += G) {
        const X v = p[i * stride];
        if (v != v) q = i;
    }
    q = group_all_reduce<G>(q, [](int64_t a, int64_t b) { return a > b ? a : b; }, sh);
    X m = R::identity();
#pragma unroll 4
    for (int64_t i = q + 1 + lane; i < i1; i += G) m = R::pick(m, p[i * stride]);
    m = group_all_reduce<G>(m, [](X a, X b) { return R::pick(a, b); }, sh);
    return q == i1 - 1 ? p[q * stride] : m;
}

// A NaN result of a row, recomputed by the G threads that share it (all of them call; the result is the same in each).
// FROM_STATE: part[0 .. splits - 1] are the chunks' partials (true folds, NaN where the chunk holds one) and `chunk` their length.
template <class R, int G, bool FROM_STATE>
__device__ __forceinline__ typename R::In fix_rows(const typename R::In* src, int64_t n, int64_t stride, const typename R::In* part,
                                                   int64_t splits, int64_t chunk, uint32_t lane, uint64_t* sh) {
    using X = typename R::In;
    if constexpr (!FROM_STATE) {
        return fold_after_last_nan<R, G>(src, 0, n, stride, lane, sh);
    } else {
        int64_t j = -1;
        for (int64_t i = lane; i < splits; i += G)
            if (part[i] != part[i]) j = i;
        j = group_all_reduce<G>(j, [](int64_t a, int64_t b) { return a > b ? a : b; }, sh);
        const int64_t c0 = j * chunk, c1 = (c0 + chunk < n) ? c0 + chunk : n;
        const X m = fold_after_last_nan<R, G>(src, c0, c1, stride, lane, sh);
        if (j + 1 >= splits) return m;
        X t = R::identity();
        for (int64_t i = j + 1 + lane; i < splits; i += G) t = R::pick(t, part[i]);
        t = group_all_reduce<G>(t, [](X a, X b) { return R::pick(a, b); }, sh);
        return R::pick(m, t);   // m is a NaN when its chunk ends with one: the fold goes on from the chunks behind it
    }
}

// fix_src / fix_n / fix_sr / fix_chunk (FROM_STATE only): the fold's source, the length and the stride of its reduced axis and the
// elements of it behind each partial, for fix_rows.
template <class R, int VEC, int TPR, bool FROM_STATE>
__global__ __launch_bounds__(kBlock) void reduce_rows_kernel(R r, const void* src_, typename R::Out* out, typename R::State* partial,
                                                             OuterArgs o, uint32_t rows, int64_t n, int64_t sr, int64_t chunk, uint32_t splits,
                                                             const typename R::In* fix_src, int64_t fix_n, int64_t fix_sr, int64_t fix_chunk) {
    using State = typename R::State;
    using In = typename std::conditional<FROM_STATE, State, typename R::In>::type;
    constexpr int RPB = kBlock / TPR;
    constexpr int U = 4;
    const In* src = (const In*)src_;
    const uint32_t row = blockIdx.x * RPB + threadIdx.x / TPR;
    const uint32_t lane = threadIdx.x % TPR;
    const bool active = row < rows;
    int64_t toff = 0, soff = 0;
    [[maybe_unused]] int64_t soff0 = 0;   // offset of the row in the fold's source
    if (active) {
        outer_offsets(o, row, toff, soff);
        soff0 = soff;
        if constexpr (FROM_STATE) soff = (int64_t)row * n;
    }
    const int64_t c0 = (int64_t)blockIdx.y * chunk;
    const int64_t c1 = (c0 + chunk < n) ? c0 + chunk : n;
    State st[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++) st[e] = r.init();
    if (active) {
        const In* p = src + soff;
        if constexpr (FROM_STATE) {
            for (int64_t i = c0 + lane; i < c1; i += TPR) st[0] = r.combine(st[0], p[i]);
        } else {
            int64_t i = c0 + (int64_t)lane * VEC;
            constexpr int64_t STEP = (int64_t)TPR * VEC;
            for (; i + (U - 1) * STEP + VEC <= c1; i += U * STEP) {
                Pack<In, VEC> v[U];
#pragma unroll
                for (int u = 0; u < U; u++) v[u] = load_pack<In, VEC>(p + (VEC == 1 ? (i + u * STEP) * sr : i + u * STEP));
#pragma unroll
                for (int u = 0; u < U; u++)
#pragma unroll
                    for (int e = 0; e < VEC; e++) st[e] = r.step(st[e], v[u].v[e], i + u * STEP + e);
            }
            for (; i + VEC <= c1; i += STEP) {
                Pack<In, VEC> v = load_pack<In, VEC>(p + (VEC == 1 ? i * sr : i));
#pragma unroll
                for (int e = 0; e < VEC; e++) st[e] = r.step(st[e], v.v[e], i + e);
            }
            if constexpr (VEC > 1) {
                // the (c1 - c0) % VEC trailing elements of this chunk
                const int64_t tail0 = c0 + ((c1 - c0) / VEC) * VEC;
                const int64_t j = tail0 + lane;
                if (j < c1) st[0] = r.step(st[0], p[j], j);
            }
        }
    }
    State s = st[0];
#pragma unroll
    for (int e = 1; e < VEC; e++) s = r.combine(s, st[e]);
    s = group_reduce<R, TPR>(r, s);
    if constexpr (TPR > 64) {
        __shared__ State sh[TPR / 64];
        const int wave = threadIdx.x / 64;
        if ((threadIdx.x & 63) == 0) sh[wave] = s;
        __syncthreads();
        if (threadIdx.x == 0) {
#pragma unroll
            for (int w = 1; w < TPR / 64; w++) s = r.combine(s, sh[w]);
        }
    }
    if constexpr (NeedsSeqFix<R>::value) {
        if (splits == 1) {
            __shared__ uint64_t fix_sh[kBlock / 64];
            bool fix = active && r.needs_fix(s);   // the same in every thread of a row's group of up to 64
            if constexpr (TPR > 64) {   // one row per block: thread 0 holds the block's result
                __shared__ int fix_flag;
                if (threadIdx.x == 0) fix_flag = fix;
                __syncthreads();
                fix = fix_flag != 0;
            }
            if (fix) {
                typename R::In v;
                if constexpr (FROM_STATE) v = fix_rows<R, TPR, true>(fix_src + soff0, fix_n, fix_sr, (const typename R::In*)src_ + soff, n, fix_chunk, lane, fix_sh);
                else v = fix_rows<R, TPR, false>((const typename R::In*)src_ + soff0, n, sr, nullptr, 0, 0, lane, fix_sh);
                if (lane == 0) out[toff] = v;
                return;
            }
        }
    }
    if (active && lane == 0) {
        if (splits == 1) out[toff] = r.extract(s);
        else partial[(int64_t)row * splits + blockIdx.y] = s;
    }
}

// Grid: one workgroup per (row chunk, other, column tile), linearised with the column tile fastest.  Workgroup ids are dealt
// round-robin to the 8 XCDs; `xcd_chunk` (total / 8 when divisible, else 0) re-numbers them so that every XCD takes one contiguous
// range of that order (with 8 column tiles the plain order would pin each XCD to one 4 KB-wide column strip).
// Partials of a split axis are stored [other][split][column]: the VEC states of a thread are contiguous (one vector store).
template <class R, int VEC, int WX>
__global__ __launch_bounds__(kBlock) void reduce_cols_kernel(R r, const typename R::In* src, typename R::Out* out,
                                                             typename R::State* partial, OuterArgs o, uint32_t col_tiles, uint32_t base_blocks,
                                                             uint32_t xcd_chunk, uint32_t nc, int64_t tc_stride, int64_t n, int64_t sr,
                                                             int64_t chunk, uint32_t splits) {
    using State = typename R::State;
    using In = typename R::In;
    constexpr int NY = kBlock / WX;
    constexpr int U = 2;
    const uint32_t x = threadIdx.x % WX, y = threadIdx.x / WX;
    uint32_t bid = blockIdx.x;
    if (xcd_chunk) bid = (bid % 8u) * xcd_chunk + bid / 8u;
    const uint32_t split = bid / base_blocks;
    bid -= split * base_blocks;
    const uint32_t tile = bid % col_tiles, other = bid / col_tiles;
    const uint32_t col0 = (tile * WX + x) * VEC;
    int64_t toff, soff;
    outer_offsets(o, other, toff, soff);
    const int64_t r0 = (int64_t)split * chunk;
    const int64_t r1 = (r0 + chunk < n) ? r0 + chunk : n;
    State st[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++) st[e] = r.init();
    const bool active = col0 < nc;
    if (active) {
        const In* p = src + soff + col0;
        int64_t i = r0 + y;
        for (; i + (U - 1) * NY < r1; i += U * NY) {
            Pack<In, VEC> v[U];
#pragma unroll
            for (int u = 0; u < U; u++) v[u] = load_pack<In, VEC>(p + (i + u * NY) * sr);
#pragma unroll
            for (int u = 0; u < U; u++)
#pragma unroll
                for (int e = 0; e < VEC; e++) st[e] = r.step(st[e], v[u].v[e], i + u * NY);
        }
        for (; i < r1; i += NY) {
            Pack<In, VEC> v = load_pack<In, VEC>(p + i * sr);
#pragma unroll
            for (int e = 0; e < VEC; e++) st[e] = r.step(st[e], v.v[e], i);
        }
    }
    if constexpr (NY > 1) {
        __shared__ State sh[NY - 1][WX * VEC];
        if (y > 0) {
#pragma unroll
            for (int e = 0; e < VEC; e++) sh[y - 1][x * VEC + e] = st[e];
        }
        __syncthreads();
        if (y == 0) {
#pragma unroll
            for (int e = 0; e < VEC; e++)
#pragma unroll
                for (int w = 0; w < NY - 1; w++) st[e] = r.combine(st[e], sh[w][x * VEC + e]);
        }
    }
    if (y == 0 && active) {
        if (splits == 1) {
#pragma unroll
            for (int e = 0; e < VEC; e++) out[toff + (int64_t)(col0 + e) * tc_stride] = finish_value(r, st[e], src + soff + col0 + e, n, sr);
        } else {
            State* q = partial + ((int64_t)other * splits + split) * nc + col0;
            if constexpr (VEC > 1 && sizeof(State) * VEC == 16) {
                // VEC > 1 implies nc % VEC == 0, so q is 16-byte aligned like the workspace
                typename RawWord<16>::type w;
                __builtin_memcpy(&w, st, 16);
                *reinterpret_cast<typename RawWord<16>::type*>(q) = w;
            } else {
#pragma unroll
                for (int e = 0; e < VEC; e++) q[e] = st[e];
            }
        }
    }
}

// Finishing pass of a split column reduction: partials [other][split][column] -> out.  WX lanes along the columns (coalesced reads
// of State), kBlock / WX groups share the splits and are combined through LDS in a fixed order.
template <class R, int WX>
__global__ __launch_bounds__(kBlock) void reduce_cols_finish_kernel(R r, const typename R::State* partial, typename R::Out* out, OuterArgs o,
                                                                    uint32_t col_tiles, uint32_t nc, int64_t tc_stride, uint32_t splits,
                                                                    const typename R::In* fix_src, int64_t fix_n, int64_t fix_sr, int64_t fix_chunk) {
    using State = typename R::State;
    constexpr int NY = kBlock / WX;
    const uint32_t x = threadIdx.x % WX, y = threadIdx.x / WX;
    const uint32_t tile = blockIdx.x % col_tiles, other = blockIdx.x / col_tiles;
    const uint32_t col = tile * WX + x;
    State st = r.init();
    if (col < nc) {
        const State* p = partial + (int64_t)other * splits * nc + col;
        constexpr uint32_t U = 8;   // loads in flight per thread; combined in split order
        uint32_t s = y;
        for (; s + (U - 1) * NY < splits; s += U * NY) {
            State v[U];
#pragma unroll
            for (uint32_t u = 0; u < U; u++) v[u] = p[(int64_t)(s + u * NY) * nc];
#pragma unroll
            for (uint32_t u = 0; u < U; u++) st = r.combine(st, v[u]);
        }
        for (; s < splits; s += NY) st = r.combine(st, p[(int64_t)s * nc]);
    }
    __shared__ State sh[NY][WX];
    sh[y][x] = st;
    __syncthreads();
    if (y == 0 && col < nc) {
        for (int w = 1; w < NY; w++) st = r.combine(st, sh[w][x]);
        int64_t toff, soff;
        outer_offsets(o, other, toff, soff);
        out[toff + (int64_t)col * tc_stride] = finish_value_chunked(r, st, partial + (int64_t)other * splits * nc + col, (int64_t)nc, splits,
                                                                    fix_src + soff + col, fix_n, fix_sr, fix_chunk);
    }
}

template <class R>
__global__ __launch_bounds__(kBlock) void reduce_generic_kernel(R r, const typename R::In* src, typename R::Out* out, OuterArgs o,
                                                                uint32_t nout, int64_t n, int64_t sr) {
    const uint32_t idx = blockIdx.x * kBlock + threadIdx.x;
    if (idx >= nout) return;
    int64_t toff, soff;
    outer_offsets(o, idx, toff, soff);
    typename R::State s = r.init();
    const typename R::In* p = src + soff;
    for (int64_t i = 0; i < n; i++) s = r.step(s, p[i * sr], i);
    out[toff] = finish_value(r, s, p, n, sr);
}

// ---- host-side strategy --------------------------------------------------------------------------------------------------

// Finishing pass of the two-pass tree: `nout` rows of `splits` State partials each.
template <class R>
int32_t launch_finish(const R& r, typename R::State* partial, typename R::Out* out, const OuterArgs& o, uint32_t nout, uint32_t splits,
                      const typename R::In* fix_src, int64_t fix_n, int64_t fix_sr, int64_t fix_chunk, hipStream_t stream) {
    using State = typename R::State;
#define DNH_FIN(TPR) hipLaunchKernelGGL((reduce_rows_kernel<R, 1, TPR, true>), dim3(cdiv(nout, kBlock / TPR)), dim3(kBlock), 0, stream, r, \
                                        (const void*)partial, out, (State*)nullptr, o, nout, (int64_t)splits, (int64_t)1, (int64_t)splits, 1u, fix_src, fix_n, fix_sr, fix_chunk)
    if (splits > 512) DNH_FIN(256);
    else if (splits > 32) DNH_FIN(64);
    else DNH_FIN(16);
#undef DNH_FIN
    DNH_LAUNCH_CHECK();
    return DNH_OK;
}

// Where the State partials of a two-pass fold go: the stream's grow-on-demand workspace, or a buffer of fixed size the caller
// names (the entry point that may not allocate), which refuses what does not fit.
struct PartialStore {
    void* fixed = nullptr;
    size_t fixed_bytes = 0;
};

inline int32_t partial_buffer(const PartialStore& ps, hipStream_t stream, size_t bytes, void** out, WorkspaceLease& lease, const char* what) {
    if (!ps.fixed) return workspace(stream, bytes, out, lease);
    if (bytes > ps.fixed_bytes)
        return fail(DNH_ERR_NOT_SUPPORTED, "%s: this fold needs %zu bytes of partial results, the static scratch array holds %zu", what, bytes,
                    ps.fixed_bytes);
    *out = ps.fixed;
    return DNH_OK;
}

template <class R>
int32_t launch_reduce(const R& r, const DnhTensor* t, const DnhTensor* s, hipStream_t stream, const char* what,
                      const PartialStore& ps = PartialStore()) {
    using In = typename R::In;
    using Out = typename R::Out;
    using State = typename R::State;
    constexpr int VEC = 16 / (int)sizeof(In);
    DNH_TRY(check_tensor(t, what));
    DNH_TRY(check_tensor(s, what));
    if (s->ndims != t->ndims + 1) return fail(DNH_ERR_INVALID_ARG, "%s: source rank %d must be target rank %d + 1", what, s->ndims, t->ndims);
    for (int d = 0; d < t->ndims; d++)
        if (t->shape[d] != s->shape[d]) return fail(DNH_ERR_INVALID_ARG, "%s: target shape does not match the source's leading dimensions", what);
    const int64_t n = s->shape[s->ndims - 1];
    const int64_t sr = s->stride[s->ndims - 1];
    const int64_t nout64 = nelems(t);
    if (nout64 == 0) return DNH_OK;
    if (nout64 > (int64_t)kMaxItems) return fail(DNH_ERR_NOT_SUPPORTED, "%s: more than 2^32 outputs", what);
    const uint32_t nout = (uint32_t)nout64;
    const In* src = (const In*)elem_ptr(s);
    Out* out = (Out*)elem_ptr(t);

    // collapse the kept dimensions jointly over target and source strides
    OuterArgs o;
    memset(&o, 0, sizeof(o));
    {
        int nd = 0;
        for (int d = 0; d < t->ndims; d++) {
            if (t->shape[d] == 1) continue;
            if (nd > 0 && o.tstride[nd - 1] == t->stride[d] * t->shape[d] && o.sstride[nd - 1] == s->stride[d] * t->shape[d]) {
                o.shape[nd - 1] *= (uint32_t)t->shape[d];
                o.tstride[nd - 1] = t->stride[d];
                o.sstride[nd - 1] = s->stride[d];
                continue;
            }
            o.shape[nd] = (uint32_t)t->shape[d];
            o.tstride[nd] = t->stride[d];
            o.sstride[nd] = s->stride[d];
            nd++;
        }
        o.nd = nd;
    }
    const int cus = device_cus();
    const int64_t target_blocks = (int64_t)cus * 8;

    // a kept dimension with source stride 1 (only of interest when the reduced axis itself is strided)
    int dc = -1;
    if (sr != 1)
        for (int d = 0; d < o.nd; d++)
            if (o.sstride[d] == 1 && o.shape[d] >= 32) dc = d;

    if (!(dc >= 0 && n >= 8) && n >= 16) {
        // rows
        // (vectors of 4- and 8-byte elements are fetched at element alignment, so shifted views and odd pitches keep them)
        bool vec = VEC > 1 && sr == 1 && vector_address(src, VEC, sizeof(In));
        for (int d = 0; d < o.nd && vec; d++) vec = vector_stride(o.sstride[d], VEC, sizeof(In));
        const int v = vec ? VEC : 1;
        // threads per row: at least four vectors per thread (measured on 16 Mi fp32: rows of 256-512 elements run 15-30 % faster
        // with 16 threads than with 64, rows of 1024-2048 fastest with 64, 4096 and longer with 256)
        int tpr = (n >= (int64_t)256 * v * 4) ? 256 : (n >= (int64_t)64 * v * 4 ? 64 : 16);
        // few rows (1000 x 1000: 63 blocks of 16 rows for 256 CUs): widen the rows' thread groups while that leaves every thread
        // a vector, until each CU has a block
        while (tpr < 256 && (int64_t)nout * tpr < (int64_t)cus * kBlock && n >= (int64_t)tpr * 4 * v) tpr *= 4;
        const int rpb = kBlock / tpr;
        const int64_t row_blocks = (nout + rpb - 1) / rpb;
        uint32_t splits = 1;
        int64_t chunk = n;
        if (tpr == 256 && row_blocks < target_blocks) {
            const int64_t min_chunk = (int64_t)256 * v * 8;
            int64_t want = (target_blocks + row_blocks - 1) / row_blocks;
            int64_t maxs = (n + min_chunk - 1) / min_chunk;
            int64_t sp = want < maxs ? want : maxs;
            if (sp > 1) {
                chunk = (n + sp - 1) / sp;
                chunk = ((chunk + 256 * v - 1) / (256 * v)) * (256 * v);  // keeps every chunk start vector-aligned
                splits = (uint32_t)((n + chunk - 1) / chunk);
                if (splits <= 1) { splits = 1; chunk = n; }
            }
        }
        State* partial = nullptr;
        WorkspaceLease lease;
        if (splits > 1) DNH_TRY(partial_buffer(ps, stream, sizeof(State) * (size_t)nout * splits, (void**)&partial, lease, what));
        const dim3 grid((unsigned)row_blocks, splits);
#define DNH_ROWS(V, TPR) hipLaunchKernelGGL((reduce_rows_kernel<R, V, TPR, false>), grid, dim3(kBlock), 0, stream, r, (const void*)src, out, partial, o, nout, n, sr, chunk, splits, src, n, sr, chunk)
        if (vec) {
            if (tpr == 256) DNH_ROWS(VEC, 256); else if (tpr == 64) DNH_ROWS(VEC, 64); else DNH_ROWS(VEC, 16);
        } else {
            if (tpr == 256) DNH_ROWS(1, 256); else if (tpr == 64) DNH_ROWS(1, 64); else DNH_ROWS(1, 16);
        }
#undef DNH_ROWS
        DNH_LAUNCH_CHECK();
        if (splits > 1) {
            // finishing pass: rows of `splits` State partials
            DNH_TRY(launch_finish(r, partial, out, o, nout, splits, src, n, sr, chunk, stream));
        }
        return DNH_OK;
    }

    // columns
    if (dc >= 0 && n >= 8) {
        const uint32_t nc = o.shape[dc];
        const int64_t tc_stride = o.tstride[dc];
        OuterArgs oo;  // the other kept dimensions
        memset(&oo, 0, sizeof(oo));
        uint32_t others = 1;
        for (int d = 0; d < o.nd; d++) {
            if (d == dc) continue;
            oo.shape[oo.nd] = o.shape[d];
            oo.tstride[oo.nd] = o.tstride[d];
            oo.sstride[oo.nd] = o.sstride[d];
            others *= o.shape[d];
            oo.nd++;
        }
        bool vec = VEC > 1 && vector_address(src, VEC, sizeof(In)) && (nc % VEC) == 0 && vector_stride(sr, VEC, sizeof(In));
        for (int d = 0; d < oo.nd && vec; d++) vec = vector_stride(oo.sstride[d], VEC, sizeof(In));
        const int v = vec ? VEC : 1;
        // Lanes along the kept dimension: the whole block when that still yields about four blocks per CU (4 KB contiguous per
        // row visit, no LDS step), else 64 lanes x 4 wavefronts sharing the reduced axis.  A block never takes fewer rows than
        // keeps the State partials (written and re-read once) near 1/64 of the source traffic.
        const int64_t min_rows = 64 * (int64_t)((sizeof(State) + sizeof(In) - 1) / sizeof(In));
        int wx = 256;
        uint32_t col_tiles = 1, splits = 1;
        int64_t base_blocks = 1, chunk = n;
        for (;;) {
            col_tiles = cdiv(nc, wx * v);
            base_blocks = (int64_t)col_tiles * others;
            const int64_t maxs = (n + min_rows - 1) / min_rows;
            // (two blocks per CU of the 256-lane form measured 12 % slower than four of the 64-lane form)
            if (wx == 64 || (nc >= (uint32_t)(256 * v) && base_blocks * maxs >= (int64_t)cus * 4)) {
                const int64_t want = ((int64_t)cus * 4 + base_blocks - 1) / base_blocks;
                const int64_t sp = want < maxs ? want : maxs;
                splits = 1;
                chunk = n;
                if (sp > 1) {
                    chunk = (n + sp - 1) / sp;
                    splits = (uint32_t)((n + chunk - 1) / chunk);
                    if (splits <= 1) { splits = 1; chunk = n; }
                }
                break;
            }
            wx = 64;
        }
        const int64_t total_blocks = base_blocks * splits;
        if (total_blocks <= 0x7FFFFFFF) {
            State* partial = nullptr;
            WorkspaceLease lease;
            if (splits > 1) DNH_TRY(partial_buffer(ps, stream, sizeof(State) * (size_t)nout * splits, (void**)&partial, lease, what));
            const dim3 grid((unsigned)total_blocks);
            const uint32_t xcd_chunk = (total_blocks % 8 == 0 && total_blocks >= 64) ? (uint32_t)(total_blocks / 8) : 0u;
#define DNH_COLS(V, W) hipLaunchKernelGGL((reduce_cols_kernel<R, V, W>), grid, dim3(kBlock), 0, stream, r, src, out, partial, oo, col_tiles, (uint32_t)base_blocks, xcd_chunk, nc, tc_stride, n, sr, chunk, splits)
            if (vec) { if (wx == 256) DNH_COLS(VEC, 256); else DNH_COLS(VEC, 64); }
            else { if (wx == 256) DNH_COLS(1, 256); else DNH_COLS(1, 64); }
#undef DNH_COLS
            DNH_LAUNCH_CHECK();
            if (splits > 1) {
                constexpr int FW = 32;   // (16 and 64 columns per finishing workgroup measured 1-2 % slower on 8192 x 8192)
                const uint32_t ftiles = cdiv(nc, FW);
                hipLaunchKernelGGL((reduce_cols_finish_kernel<R, FW>), dim3(ftiles * others), dim3(kBlock), 0, stream, r, (const State*)partial, out,
                                   oo, ftiles, nc, tc_stride, splits, src, n, sr, chunk);
                DNH_LAUNCH_CHECK();
            }
            return DNH_OK;
        }
    }

    hipLaunchKernelGGL((reduce_generic_kernel<R>), dim3(cdiv(nout, kBlock)), dim3(kBlock), 0, stream, r, src, out, o, nout, n, sr);
    DNH_LAUNCH_CHECK();
    return DNH_OK;
}

}  // namespace dnh
