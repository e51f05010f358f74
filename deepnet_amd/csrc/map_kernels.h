// Element-wise map kernels (target + up to three sources) for gfx950 and the launcher that picks one from a MapPlan.
//
//  map_flat  : every operand is one contiguous run (or a stride-0 scalar): 16-byte loads/stores per lane, several in
//              flight per thread, one pass over HBM.
//  map_nd    : collapsed n-d strided operands; lanes run along the target's fastest dimension (coalesced stores), 16-byte
//              vectors when the last dimension allows it, per-item index decomposition in 32-bit arithmetic.
//  map_tr    : a source whose unit-stride dimension differs from the target's is staged through LDS in 128x64 tiles (64x32 for
//              8-byte elements, 256x128 for short target rows): global reads run along the source's fast dimension, global
//              writes along the target's.
//
// An Op is a small functor: `using T/A/B/C` (target and source element types, `char` when absent), `NSRC`, and
// `__device__ T operator()(A[,B[,C]]) const`.  State (a fill value) travels by value as a kernel argument.
#pragma once

#include "common.h"

#include <type_traits>

namespace dnh {

constexpr int kBlock = 256;

// raw N-byte words for vector memory access
template <int BYTES> struct RawWord;
template <> struct RawWord<1> { using type = uint8_t; };
template <> struct RawWord<2> { using type = uint16_t; };
template <> struct RawWord<4> { using type = uint32_t; };
template <> struct RawWord<8> { typedef uint32_t type __attribute__((ext_vector_type(2))); };
template <> struct RawWord<16> { typedef uint32_t type __attribute__((ext_vector_type(4))); };

template <class T, int N>
struct Pack {
    T v[N];
};

// The word type a pack of N elements of T moves as.  Elements of 4 bytes and more: declared with the element's alignment only.
// The hardware serves 8- and 16-byte accesses at any dword address (measured on a 256 MiB copy with every combination of source
// and target offsets: 5.8-6.05 TB/s and every element right, against 3.5 TB/s with 4-byte accesses), the compiler emits the same
// single instruction, and views that start at an odd element or have odd row pitches keep the vector kernels.  Narrower
// elements keep the natural alignment of the word (their launchers check it).
template <class T, int BYTES, bool ELEM_ALIGNED = (sizeof(T) >= 4)> struct PackWord { using type = typename RawWord<BYTES>::type; };
template <class T> struct PackWord<T, 8, true> { typedef uint32_t type __attribute__((ext_vector_type(2), aligned(4))); };
template <class T> struct PackWord<T, 16, true> { typedef uint32_t type __attribute__((ext_vector_type(4), aligned(4))); };

// packs wider than 16 bytes move as consecutive 16-byte words
template <class T, int N>
__device__ __forceinline__ Pack<T, N> load_pack(const T* p) {
    Pack<T, N> r;
    if constexpr (sizeof(T) * N <= 16) {
        using W = typename PackWord<T, sizeof(T) * N>::type;
        W w = __builtin_nontemporal_load((const W*)p);
        __builtin_memcpy(&r, &w, sizeof(w));
    } else {
        using W = typename PackWord<T, 16>::type;
        constexpr int NW = (int)(sizeof(T) * N / 16);
        W w[NW];
#pragma unroll
        for (int i = 0; i < NW; i++) w[i] = __builtin_nontemporal_load((const W*)p + i);
        __builtin_memcpy(&r, w, sizeof(w));
    }
    return r;
}

template <class T, int N>
__device__ __forceinline__ void store_pack(T* p, const Pack<T, N>& r) {
    if constexpr (sizeof(T) * N <= 16) {
        using W = typename PackWord<T, sizeof(T) * N>::type;
        W w;
        __builtin_memcpy(&w, &r, sizeof(w));
        __builtin_nontemporal_store(w, (W*)p);
    } else {
        using W = typename PackWord<T, 16>::type;
        constexpr int NW = (int)(sizeof(T) * N / 16);
        W w[NW];
        __builtin_memcpy(w, &r, sizeof(w));
#pragma unroll
        for (int i = 0; i < NW; i++) __builtin_nontemporal_store(w[i], (W*)p + i);
    }
}

template <class T, int N>
__device__ __forceinline__ Pack<T, N> splat_pack(T x) {
    Pack<T, N> r;
#pragma unroll
    for (int i = 0; i < N; i++) r.v[i] = x;
    return r;
}

template <class Op>
__device__ __forceinline__ typename Op::T apply_op(const Op& op, typename Op::A a, typename Op::B b, typename Op::C c) {
    if constexpr (Op::NSRC == 0) return op();
    else if constexpr (Op::NSRC == 1) return op(a);
    else if constexpr (Op::NSRC == 2) return op(a, b);
    else return op(a, b, c);
}

// ---- flat ---------------------------------------------------------------------------------------------------------------

constexpr uint32_t kXcdRun = 64;

template <class Op, int VEC, int UNROLL>
// The target may be one of the sources (in-place ops such as FillMultiply a a b): no pointer is declared restrict, and a thread
// reads everything it needs of an element before it writes that element.
__global__ __launch_bounds__(kBlock) void map_flat_kernel(Op op, typename Op::T* t, const typename Op::A* a,
                                                          const typename Op::B* b, const typename Op::C* c, int sa, int sb, int sc,
                                                          int64_t n) {
    using T = typename Op::T;
    using A = typename Op::A;
    using B = typename Op::B;
    using C = typename Op::C;
    const int64_t nvec = n / VEC;
    // Workgroup ids are dealt round-robin to the 8 XCDs.  Inside every group of 8 * kXcdRun workgroups the ids are permuted so
    // that each XCD streams kXcdRun consecutive 4 KB pieces (256 KB) instead of every eighth piece: measured 1.5-2 % more
    // bandwidth on a three-stream add (runs of 32 to 512 pieces are equivalent, 16 and below or 1024 and above are slower).
    uint32_t bid = blockIdx.x;
    {
        constexpr uint32_t span = 8u * kXcdRun;
        if (bid < (gridDim.x / span) * span) {
            const uint32_t r = bid % span;
            bid = bid - r + (r % 8u) * kXcdRun + r / 8u;
        }
    }
    const int64_t base = (int64_t)bid * (kBlock * UNROLL) + threadIdx.x;
    Pack<A, VEC> va[UNROLL];
    Pack<B, VEC> vb[UNROLL];
    Pack<C, VEC> vc[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const int64_t i = base + (int64_t)u * kBlock;
        if (i < nvec) {
            if constexpr (Op::NSRC >= 1) va[u] = sa ? load_pack<A, VEC>(a + i * VEC) : splat_pack<A, VEC>(a[0]);
            if constexpr (Op::NSRC >= 2) vb[u] = sb ? load_pack<B, VEC>(b + i * VEC) : splat_pack<B, VEC>(b[0]);
            if constexpr (Op::NSRC >= 3) vc[u] = sc ? load_pack<C, VEC>(c + i * VEC) : splat_pack<C, VEC>(c[0]);
        }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const int64_t i = base + (int64_t)u * kBlock;
        if (i < nvec) {
            Pack<T, VEC> r;
#pragma unroll
            for (int e = 0; e < VEC; e++) r.v[e] = apply_op(op, va[u].v[e], vb[u].v[e], vc[u].v[e]);
            store_pack<T, VEC>(t + i * VEC, r);
        }
    }
    // the n % VEC trailing elements
    if (bid == 0) {
        const int64_t i = nvec * VEC + threadIdx.x;
        if (threadIdx.x < VEC && i < n) {
            A xa = A();
            B xb = B();
            C xc = C();
            if constexpr (Op::NSRC >= 1) xa = a[sa ? i : 0];
            if constexpr (Op::NSRC >= 2) xb = b[sb ? i : 0];
            if constexpr (Op::NSRC >= 3) xc = c[sc ? i : 0];
            t[i] = apply_op(op, xa, xb, xc);
        }
    }
}

// ---- n-d ----------------------------------------------------------------------------------------------------------------

// Division of a 32-bit index by an extent known on the host: q = (t + ((n - t) >> s1)) >> s2 with t = mulhi(n, m), exact for every
// n < 2^32 (m = floor(2^32 (2^l - d) / d) + 1, l = ceil(log2 d), s1 = min(l, 1), s2 = max(l - 1, 0)).  Five instructions instead of
// the twenty-odd of a hardware-free 32-bit division, once per thread and dimension.
struct FastDiv {
    uint32_t m, s1, s2, d;
};
inline FastDiv make_fast_div(uint32_t d) {
    FastDiv f;
    if (d == 0) d = 1;
    uint32_t l = 0;
    while (l < 32 && ((uint64_t)1 << l) < d) l++;
    f.m = (uint32_t)((((uint64_t)1 << 32) * (((uint64_t)1 << l) - d)) / d + 1);
    f.s1 = l < 1 ? l : 1;
    f.s2 = l > 1 ? l - 1 : 0;
    f.d = d;
    return f;
}
__device__ __forceinline__ uint32_t fast_div(uint32_t n, const FastDiv& f) {
    const uint32_t t = __umulhi(n, f.m);
    return (t + ((n - t) >> f.s1)) >> f.s2;
}

struct NdArgs {
    int nd;                                      // >= 1
    FastDiv div[DNH_MAX_DIMS];                   // division by shape[d]
    uint32_t shape[DNH_MAX_DIMS];                // shape[nd-1] counts items of VEC elements
    int64_t stride[kMaxOperands][DNH_MAX_DIMS];  // element strides; last dimension already multiplied by VEC
    int vecload[kMaxOperands];                   // source k is read as a vector (last-dim stride 1) rather than splat (stride 0)
};

// ND > 0: the collapsed rank is known at compile time (2 for a matrix with a row- or column-broadcast operand, the commonest
// case), so the index loop unrolls and its extents and strides stay in scalar registers; ND = 0: any rank, read from p.nd.
template <class Op, int VEC, int UNROLL, int ND>
__global__ __launch_bounds__(kBlock) void map_nd_kernel(Op op, typename Op::T* t, const typename Op::A* a, const typename Op::B* b,
                                                        const typename Op::C* c, NdArgs p, uint32_t nitems) {
    using T = typename Op::T;
    using A = typename Op::A;
    using B = typename Op::B;
    using C = typename Op::C;
    const uint32_t base = blockIdx.x * (uint32_t)(kBlock * UNROLL) + threadIdx.x;
    int64_t ot[UNROLL], oa[UNROLL], ob[UNROLL], oc[UNROLL];
    Pack<A, VEC> va[UNROLL];
    Pack<B, VEC> vb[UNROLL];
    Pack<C, VEC> vc[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const uint32_t item = base + (uint32_t)u * kBlock;
        ot[u] = oa[u] = ob[u] = oc[u] = 0;
        if (item < nitems) {
            uint32_t rem = item;
            const int nd = ND > 0 ? ND : p.nd;
#pragma unroll
            for (int d = nd - 1; d >= 0; d--) {
                uint32_t q = (d == 0) ? 0u : fast_div(rem, p.div[d]);
                uint32_t idx = rem - q * p.shape[d];
                rem = q;
                ot[u] += (int64_t)idx * p.stride[0][d];
                if constexpr (Op::NSRC >= 1) oa[u] += (int64_t)idx * p.stride[1][d];
                if constexpr (Op::NSRC >= 2) ob[u] += (int64_t)idx * p.stride[2][d];
                if constexpr (Op::NSRC >= 3) oc[u] += (int64_t)idx * p.stride[3][d];
            }
            if constexpr (VEC == 1) {
                if constexpr (Op::NSRC >= 1) va[u].v[0] = a[oa[u]];
                if constexpr (Op::NSRC >= 2) vb[u].v[0] = b[ob[u]];
                if constexpr (Op::NSRC >= 3) vc[u].v[0] = c[oc[u]];
            } else {
                if constexpr (Op::NSRC >= 1) va[u] = p.vecload[1] ? load_pack<A, VEC>(a + oa[u]) : splat_pack<A, VEC>(a[oa[u]]);
                if constexpr (Op::NSRC >= 2) vb[u] = p.vecload[2] ? load_pack<B, VEC>(b + ob[u]) : splat_pack<B, VEC>(b[ob[u]]);
                if constexpr (Op::NSRC >= 3) vc[u] = p.vecload[3] ? load_pack<C, VEC>(c + oc[u]) : splat_pack<C, VEC>(c[oc[u]]);
            }
        }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const uint32_t item = base + (uint32_t)u * kBlock;
        if (item < nitems) {
            Pack<T, VEC> r;
#pragma unroll
            for (int e = 0; e < VEC; e++) r.v[e] = apply_op(op, va[u].v[e], vb[u].v[e], vc[u].v[e]);
            if constexpr (VEC == 1) t[ot[u]] = r.v[0];
            else store_pack<T, VEC>(t + ot[u], r);
        }
    }
}

// The n-d kernel for calls whose target runs along the last dimension but that the vector form above cannot take: an operand that
// is misaligned (a view that starts at an odd element: x[:, 1:] - x[:, :-1]), has row pitches that are not whole vectors, or is
// strided along the last dimension, and rows whose length is not a multiple of VEC.  Every thread still handles VEC consecutive
// elements of a row; per operand, `mode` says how it gets them: 0 one element for all (stride 0), 1 one aligned vector, 2 one
// element at a time at `estride`.  The last item of a row may hold fewer than VEC elements (`lastlen` is the row length): that
// item is moved element by element, with guards.  All of a thread's loads are issued before the first use.
struct NdMixArgs {
    int mode[kMaxOperands];          // [0] is the target: 1 vector stores, 2 element stores
    int64_t estride[kMaxOperands];   // element stride along the last dimension
    uint32_t lastlen;                // elements per row
};

template <class Op, int VEC>
__global__ __launch_bounds__(kBlock) void map_nd_mix_kernel(Op op, typename Op::T* t, const typename Op::A* a, const typename Op::B* b,
                                                            const typename Op::C* c, NdArgs p, NdMixArgs m, uint32_t nitems) {
    using T = typename Op::T;
    using A = typename Op::A;
    using B = typename Op::B;
    using C = typename Op::C;
    const uint32_t item = blockIdx.x * (uint32_t)kBlock + threadIdx.x;
    if (item >= nitems) return;
    int64_t ot = 0, oa = 0, ob = 0, oc = 0;
    uint32_t rem = item, ilast = 0;
    for (int d = p.nd - 1; d >= 0; d--) {
        const uint32_t q = (d == 0) ? 0u : fast_div(rem, p.div[d]);
        const uint32_t idx = rem - q * p.shape[d];
        rem = q;
        if (d == p.nd - 1) ilast = idx;
        ot += (int64_t)idx * p.stride[0][d];
        if constexpr (Op::NSRC >= 1) oa += (int64_t)idx * p.stride[1][d];
        if constexpr (Op::NSRC >= 2) ob += (int64_t)idx * p.stride[2][d];
        if constexpr (Op::NSRC >= 3) oc += (int64_t)idx * p.stride[3][d];
    }
    const uint32_t left = m.lastlen - ilast * (uint32_t)VEC;     // elements of the row from this item on
    const bool whole = left >= (uint32_t)VEC;
    // element e of a partial item beyond the row's end reads element 0 of the item instead (and is not stored)
    auto fetch = [&](auto* src, int64_t off, int mode, int64_t es) {
        using X = std::remove_cv_t<std::remove_pointer_t<decltype(src)>>;
        Pack<X, VEC> v;
        if (mode == 1 && whole) return load_pack<X, VEC>(src + off);
        if (mode == 0) return splat_pack<X, VEC>(src[off]);
        const int64_t step = mode == 2 ? es : 1;
#pragma unroll
        for (int e = 0; e < VEC; e++) v.v[e] = src[off + ((uint32_t)e < left ? e * step : 0)];
        return v;
    };
    Pack<A, VEC> va;
    Pack<B, VEC> vb;
    Pack<C, VEC> vc;
    if constexpr (Op::NSRC >= 1) va = fetch(a, oa, m.mode[1], m.estride[1]);
    if constexpr (Op::NSRC >= 2) vb = fetch(b, ob, m.mode[2], m.estride[2]);
    if constexpr (Op::NSRC >= 3) vc = fetch(c, oc, m.mode[3], m.estride[3]);
    Pack<T, VEC> r;
#pragma unroll
    for (int e = 0; e < VEC; e++) r.v[e] = apply_op(op, va.v[e], vb.v[e], vc.v[e]);
    if (m.mode[0] == 1 && whole) {
        store_pack<T, VEC>(t + ot, r);
    } else {
#pragma unroll
        for (int e = 0; e < VEC; e++)
            if ((uint32_t)e < left) t[ot + e] = r.v[e];
    }
}

// ---- LDS-staged transpose -------------------------------------------------------------------------------------------------

struct TrArgs {
    int nouter;                                   // dimensions other than A (staged sources' fast dim) and B (target's fast dim)
    uint32_t oshape[DNH_MAX_DIMS];
    int64_t ostride[kMaxOperands][DNH_MAX_DIMS];
    uint32_t na, nb, tiles_a, tiles_b;
    int64_t sa[kMaxOperands], sb[kMaxOperands];   // element strides along A and B
    int staged[kMaxOperands];                     // source k goes through LDS
    uint32_t lds_off[kMaxOperands];               // byte offset of source k's tile in dynamic LDS (staged sources only)
    int dmode;                                    // sources that are not staged: 1 = all broadcast along B, 2 = all broadcast or in aligned vectors along B, 0 = other
};

// Direct (not LDS-staged) operand fetch of the transposing kernel for VEC consecutive positions tx.. along B at row r along A:
// one vector when the operand runs along B, one scalar when it is broadcast along B, element by element otherwise.
template <class X, int VEC>
__device__ __forceinline__ Pack<X, VEC> tr_direct(const X* g, uint32_t r, uint32_t tx, int64_t sa, int64_t sb) {
    const X* q = g + (int64_t)r * sa + (int64_t)tx * sb;
    if (sb == 0) return splat_pack<X, VEC>(*q);
    if (sb == 1 && VEC > 1 && (((uintptr_t)q) % (VEC * sizeof(X))) == 0) return load_pack<X, VEC>(q);
    Pack<X, VEC> v;
#pragma unroll
    for (int e = 0; e < VEC; e++) v.v[e] = q[(int64_t)e * sb];
    return v;
}

// Tile of TA elements along A (the staged sources' unit-stride dimension) by TB along B (the target's).  Workgroup ids walk the
// tiles with B fastest, then A, then the outer dimensions; `xcd_chunk` (total / 8, or 0) re-numbers them so that each XCD takes a
// contiguous range of that order.  MASK: bit k - 1 set = source k is staged through LDS (a compile-time choice: with run-time flags
// the store loop is full of branches, and the compiler then waits for every store before it issues the next one).
// The same fetch without a branch, for operands that are either broadcast along B (sb == 0) or run along B in aligned vectors
// (sb == 1): one vector load (from the aligned vector that holds the element when broadcast) and one element load, then a select.
// Branches around the loads of a loop make the compiler wait for each load before it issues the next.
template <class X, int VEC>
__device__ __forceinline__ Pack<X, VEC> tr_direct_fast(const X* g, uint32_t r, uint32_t tx, int64_t sa, int64_t sb) {
    const X* q = g + (int64_t)r * sa + (int64_t)tx * sb;
    if constexpr (VEC == 1) {
        Pack<X, 1> v;
        v.v[0] = *q;
        return v;
    } else {
        const bool bcast = sb == 0;
        const X* qv = bcast ? (const X*)((uintptr_t)q & ~(uintptr_t)(VEC * sizeof(X) - 1)) : q;
        Pack<X, VEC> v = load_pack<X, VEC>(qv);
        const X s = *q;
#pragma unroll
        for (int e = 0; e < VEC; e++) v.v[e] = bcast ? s : v.v[e];
        return v;
    }
}

template <class Op, int TA, int TB, int VEC, int MASK>
__global__ __launch_bounds__(kBlock) void map_tr_kernel(Op op, typename Op::T* t, const typename Op::A* a, const typename Op::B* b,
                                                        const typename Op::C* c, TrArgs p, uint32_t xcd_chunk) {
    using T = typename Op::T;
    using A = typename Op::A;
    using B = typename Op::B;
    using C = typename Op::C;
    constexpr bool S1 = (MASK & 1) != 0, S2 = (MASK & 2) != 0, S3 = (MASK & 4) != 0;
    static_assert(MASK > 0 && MASK < (1 << Op::NSRC), "staged sources");
    constexpr int TVA = TA / VEC;            // staging: threads per tile row along A
    constexpr int ROWS_S = kBlock / TVA;     // rows (along B) staged per pass
    constexpr int ITER_S = TB / ROWS_S;
    constexpr int TVB = TB / VEC;            // storing: threads per tile row along B
    constexpr int ROWS_T = kBlock / TVB;     // rows (along A) stored per pass
    constexpr int ITER_T = TA / ROWS_T;
    static_assert(TA % VEC == 0 && TB % VEC == 0 && kBlock % TVA == 0 && kBlock % TVB == 0 && TB % ROWS_S == 0 && TA % ROWS_T == 0, "tile shape");
    // only staged sources own an LDS tile ([TB][TA+1] elements each), so occupancy is not spent on unused tiles
    extern __shared__ __align__(16) unsigned char tr_lds[];
    typedef A (*TileA)[TA + 1];
    typedef B (*TileB)[TA + 1];
    typedef C (*TileC)[TA + 1];
    TileA la = (TileA)(tr_lds + p.lds_off[1]);
    TileB lb = (TileB)(tr_lds + p.lds_off[2]);
    TileC lc = (TileC)(tr_lds + p.lds_off[3]);

    uint32_t bid = blockIdx.x;
    if (xcd_chunk) bid = (bid % 8u) * xcd_chunk + bid / 8u;
    const uint32_t tb = bid % p.tiles_b;
    bid /= p.tiles_b;
    const uint32_t ta = bid % p.tiles_a;
    bid /= p.tiles_a;
    const uint32_t a0 = ta * TA, b0 = tb * TB;
    int64_t off[kMaxOperands];
#pragma unroll
    for (int k = 0; k <= Op::NSRC; k++) off[k] = (int64_t)a0 * p.sa[k] + (int64_t)b0 * p.sb[k];
    for (int d = p.nouter - 1; d >= 0; d--) {
        const uint32_t q = (d == 0) ? 0u : bid / p.oshape[d];
        const uint32_t idx = bid - q * p.oshape[d];
        bid = q;
#pragma unroll
        for (int k = 0; k <= Op::NSRC; k++) off[k] += (int64_t)idx * p.ostride[k][d];
    }
    t += off[0];
    if constexpr (Op::NSRC >= 1) a += off[1];
    if constexpr (Op::NSRC >= 2) b += off[2];
    if constexpr (Op::NSRC >= 3) c += off[3];
    const uint32_t la_n = p.na - a0 < (uint32_t)TA ? p.na - a0 : TA;   // valid extent of this tile along A and B
    const uint32_t lb_n = p.nb - b0 < (uint32_t)TB ? p.nb - b0 : TB;

    // stage: lanes run along A (the staged sources' unit-stride dimension); the LDS tile is [b][a].  All loads of a thread are
    // issued back to back, before the first LDS store, so that they are in flight together: no branch separates them (positions
    // outside an edge tile fetch element (0, 0) of the tile instead, and what they put into LDS is never read).
    {
        const uint32_t sx = (threadIdx.x % TVA) * VEC, sy = threadIdx.x / TVA;
        const uint32_t sxc = sx + VEC <= la_n ? sx : 0u;
        // (a row of the tensor that is not a whole number of vectors ends inside one thread column's vector: those threads fetch
        // column 0 with the others and then their own elements one by one)
        const bool part_a = VEC > 1 && sx < la_n && sx + VEC > la_n;
        Pack<A, VEC> ga[ITER_S];
        Pack<B, VEC> gb[ITER_S];
        Pack<C, VEC> gc[ITER_S];
        if (la_n >= (uint32_t)VEC) {   // (a tile narrower than one vector has no whole vector to fetch: elements only, below)
#pragma unroll
            for (int it = 0; it < ITER_S; it++) {
                const uint32_t r = sy + it * ROWS_S;
                const int64_t rc = r < lb_n ? (int64_t)r : 0;
                if constexpr (Op::NSRC >= 1)
                    if constexpr (S1) ga[it] = load_pack<A, VEC>(a + rc * p.sb[1] + sxc);
                if constexpr (Op::NSRC >= 2)
                    if constexpr (S2) gb[it] = load_pack<B, VEC>(b + rc * p.sb[2] + sxc);
                if constexpr (Op::NSRC >= 3)
                    if constexpr (S3) gc[it] = load_pack<C, VEC>(c + rc * p.sb[3] + sxc);
            }
        }
        if constexpr (VEC > 1) {
            if (part_a) {
#pragma unroll
                for (int it = 0; it < ITER_S; it++) {
                    const uint32_t r = sy + it * ROWS_S;
                    const int64_t rc = r < lb_n ? (int64_t)r : 0;
#pragma unroll
                    for (int e = 0; e < VEC - 1; e++) {
                        const uint32_t col = sx + e < la_n ? sx + e : 0u;
                        if constexpr (Op::NSRC >= 1)
                            if constexpr (S1) ga[it].v[e] = a[rc * p.sb[1] + col];
                        if constexpr (Op::NSRC >= 2)
                            if constexpr (S2) gb[it].v[e] = b[rc * p.sb[2] + col];
                        if constexpr (Op::NSRC >= 3)
                            if constexpr (S3) gc[it].v[e] = c[rc * p.sb[3] + col];
                    }
                }
            }
        }
#pragma unroll
        for (int it = 0; it < ITER_S; it++) {
            const uint32_t r = sy + it * ROWS_S;
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                if constexpr (Op::NSRC >= 1)
                    if constexpr (S1) la[r][sx + e] = ga[it].v[e];
                if constexpr (Op::NSRC >= 2)
                    if constexpr (S2) lb[r][sx + e] = gb[it].v[e];
                if constexpr (Op::NSRC >= 3)
                    if constexpr (S3) lc[r][sx + e] = gc[it].v[e];
            }
        }
    }
    // Sources that are not staged and are broadcast along B (a bias along A, say) have one value per stored row: they are fetched
    // here, ahead of the barrier, so that their latency is covered by the staging loads.
    constexpr int NDIRECT = Op::NSRC - (int)S1 - (int)S2 - (int)S3;
    [[maybe_unused]] A pa[ITER_T];
    [[maybe_unused]] B pb[ITER_T];
    [[maybe_unused]] C pc[ITER_T];
    if constexpr (NDIRECT > 0 && VEC > 1) {
        if (p.dmode == 1 && la_n == (uint32_t)TA && lb_n == (uint32_t)TB) {
            const uint32_t ty0 = threadIdx.x / TVB;
#pragma unroll
            for (int it = 0; it < ITER_T; it++) {
                const uint32_t r = ty0 + it * ROWS_T;
                const int64_t rc = r < la_n ? (int64_t)r : 0;
                if constexpr (Op::NSRC >= 1 && !S1) pa[it] = a[rc * p.sa[1]];
                if constexpr (Op::NSRC >= 2 && !S2) pb[it] = b[rc * p.sa[2]];
                if constexpr (Op::NSRC >= 3 && !S3) pc[it] = c[rc * p.sa[3]];
            }
        }
    }
    __syncthreads();
    // compute + store: lanes run along B (the target's unit-stride dimension), VEC consecutive elements per thread.  Operands that
    // are not staged are read in the store pattern, a group of G rows at a time: the loads of a group are issued before its first
    // store (loads and stores retire through one in-order counter on this architecture, so a load placed after a store waits for
    // that store to complete; with one workgroup per CU, as for the large tile, nothing else would cover that wait).
    constexpr int G = (NDIRECT <= 1 || ITER_T < 8) ? ITER_T : 8;   // one direct operand: all of its rows at once (at most 128 registers)
    static_assert(ITER_T % G == 0, "tile shape");
    const uint32_t tx = (threadIdx.x % TVB) * VEC, ty = threadIdx.x / TVB;
    // FULL: the tile lies inside the tensor, so no row or column test is needed.  A test around each store is a divergent branch,
    // and after such a branch the compiler waits for all outstanding memory operations, the previous store included.
    auto store_phase = [&](auto mode_tag, auto full_tag) {
        constexpr int MODE = decltype(mode_tag)::value;    // as TrArgs::dmode
        constexpr bool FULL = decltype(full_tag)::value;
        [[maybe_unused]] const bool whole_b = tx + VEC <= lb_n;   // this thread's vector lies inside the row
        // Rows beyond an edge tile's extent repeat its last row: they fetch what that row fetches and store what it stores (the same
        // values to the same addresses), so that no store of the loop sits behind a test.
        auto row_of = [&](int i) {
            const uint32_t r0 = ty + (uint32_t)i * ROWS_T;
            return FULL ? r0 : (r0 < la_n ? r0 : la_n - 1u);
        };
#pragma unroll 1
        for (int g0 = 0; g0 < ITER_T; g0 += G) {
            Pack<A, VEC> da[G];
            Pack<B, VEC> db[G];
            Pack<C, VEC> dc[G];
            if constexpr (MODE != 1) {
#pragma unroll
                for (int i = 0; i < G; i++) {
                    const uint32_t r = row_of(g0 + i);
                    if constexpr (MODE == 2) {
                        const uint32_t rc = r;
                        const uint32_t txc = (FULL || whole_b) ? tx : 0u;  // a vector that would cross the row's end fetches column 0
                        if (FULL || lb_n >= (uint32_t)VEC) {   // (as in the staging: no whole vector in a tile narrower than one)
                            if constexpr (Op::NSRC >= 1 && !S1) da[i] = tr_direct_fast<A, VEC>(a, rc, txc, p.sa[1], p.sb[1]);
                            if constexpr (Op::NSRC >= 2 && !S2) db[i] = tr_direct_fast<B, VEC>(b, rc, txc, p.sa[2], p.sb[2]);
                            if constexpr (Op::NSRC >= 3 && !S3) dc[i] = tr_direct_fast<C, VEC>(c, rc, txc, p.sa[3], p.sb[3]);
                        }
                    } else if (FULL || whole_b) {
                        if constexpr (Op::NSRC >= 1 && !S1) da[i] = tr_direct<A, VEC>(a, r, tx, p.sa[1], p.sb[1]);
                        if constexpr (Op::NSRC >= 2 && !S2) db[i] = tr_direct<B, VEC>(b, r, tx, p.sa[2], p.sb[2]);
                        if constexpr (Op::NSRC >= 3 && !S3) dc[i] = tr_direct<C, VEC>(c, r, tx, p.sa[3], p.sb[3]);
                    }
                    if constexpr (!FULL && VEC > 1) {
                        // the elements of a vector that crosses the row's end, one by one
                        if (!whole_b) {
#pragma unroll
                            for (int e = 0; e < VEC - 1; e++) {
                                const uint32_t col = tx + e < lb_n ? tx + e : tx;
                                if constexpr (Op::NSRC >= 1 && !S1) da[i].v[e] = a[(int64_t)r * p.sa[1] + (int64_t)col * p.sb[1]];
                                if constexpr (Op::NSRC >= 2 && !S2) db[i].v[e] = b[(int64_t)r * p.sa[2] + (int64_t)col * p.sb[2]];
                                if constexpr (Op::NSRC >= 3 && !S3) dc[i].v[e] = c[(int64_t)r * p.sa[3] + (int64_t)col * p.sb[3]];
                            }
                        }
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < G; i++) {
                const uint32_t r = row_of(g0 + i);
                {
                    Pack<T, VEC> res;
#pragma unroll
                    for (int e = 0; e < VEC; e++) {
                        A xa = A();
                        B xb = B();
                        C xc = C();
                        if constexpr (Op::NSRC >= 1) xa = S1 ? la[tx + e][r] : (MODE == 1 ? pa[g0 + i] : da[i].v[e]);
                        if constexpr (Op::NSRC >= 2) xb = S2 ? lb[tx + e][r] : (MODE == 1 ? pb[g0 + i] : db[i].v[e]);
                        if constexpr (Op::NSRC >= 3) xc = S3 ? lc[tx + e][r] : (MODE == 1 ? pc[g0 + i] : dc[i].v[e]);
                        res.v[e] = apply_op(op, xa, xb, xc);
                    }
                    if (FULL || whole_b) {
                        store_pack<T, VEC>(t + (int64_t)r * p.sa[0] + tx, res);
                    } else {
#pragma unroll
                        for (int e = 0; e < VEC - 1; e++)
                            if (tx + e < lb_n) t[(int64_t)r * p.sa[0] + tx + e] = res.v[e];
                    }
                }
            }
        }
    };
    using M0 = std::integral_constant<int, 0>;
    using M1 = std::integral_constant<int, 1>;
    using M2 = std::integral_constant<int, 2>;
    // (the element-wise instantiation fetches single elements through any strides without a branch: mode 2 for every layout; tiles
    // on the tensor's edge take the general path whatever the mode, which keeps the number of copies of this loop down)
    const bool full = la_n == (uint32_t)TA && lb_n == (uint32_t)TB;
    if constexpr (NDIRECT == 0 || VEC == 1) {
        if (full) store_phase(M2{}, std::true_type{});
        else if (tx < lb_n) store_phase(M2{}, std::false_type{});
    } else {
        if (full && p.dmode == 1) store_phase(M1{}, std::true_type{});
        else if (full && p.dmode == 2) store_phase(M2{}, std::true_type{});
        else if (tx < lb_n) {
            if (p.dmode == 2) store_phase(M2{}, std::false_type{});
            else store_phase(M0{}, std::false_type{});
        }
    }
}

// The transposing kernel for 4- and 8-byte staged elements and whole tiles, with both LDS phases free of bank conflicts and on
// 16-byte LDS instructions (described for 4-byte elements, VEC = 4; 8-byte elements have VEC = 2, blocks of 2 x 2 and groups of two b's).  map_tr_kernel's [b][a + 1] tile is written with one 4-byte store per element at a lane stride of four words
// (8 of the 32 banks) and read element by element (16 banks).  Here a staging thread fetches the same vector of four a's from
// four consecutive rows b, so that it holds a 4 x 4 block, and writes its four columns: LDS is [a][b] in 16-byte groups of four
// b's, group g of row a stored at g ^ ((a / 4) % 8); consecutive lanes (a four apart) then fall into different groups, and a storing
// thread fetches its four b's of row a with one 16-byte read, consecutive lanes again in different groups.
// One staged source (MASK 1 or 2); for two-operand ops the other source is read in the store pattern, MODE 1 (broadcast along B:
// one value per stored row, fetched ahead of the barrier) or MODE 2 (broadcast or in vectors along B).
// GEN = false: whole tiles.  GEN = true: tiles on the tensor's edge, target rows that are not whole vectors, a second operand with
// any strides (the staged source's rows still are whole vectors).  What it is for: short target rows of any length (250 elements,
// say) that follow one another in memory, where one workgroup writes its 256 rows as one contiguous run; cut into the 128 x 64
// tiles of map_tr_kernel the same rows are written as 256-byte pieces that start and end inside cache lines, at half the speed.
template <class Op, int TA, int TB, int MASK, bool GEN>
__global__ __launch_bounds__(kBlock) void map_tr4_kernel(Op op, typename Op::T* t, const typename Op::A* a, const typename Op::B* b,
                                                         TrArgs p, uint32_t xcd_chunk) {
    using T = typename Op::T;
    using A = typename Op::A;
    using B = typename Op::B;
    using C = typename Op::C;
    static_assert(Op::NSRC >= 1 && Op::NSRC <= 2 && (MASK == 1 || MASK == 2) && MASK <= Op::NSRC, "one staged source of one or two");
    using S0 = std::conditional_t<MASK == 1, A, B>;
    static_assert(sizeof(S0) == 4 || sizeof(S0) == 8, "staged elements of four or eight bytes");
    constexpr int VEC = 16 / (int)sizeof(S0);   // elements per 16-byte group: the blocks a staging thread holds are VEC x VEC
    constexpr bool S1 = MASK == 1;
    using S = std::conditional_t<S1, A, B>;   // the staged source
    using D = std::conditional_t<S1, B, A>;   // the other one (two-operand ops only)
    constexpr int KS = S1 ? 1 : 2, KD = S1 ? 2 : 1;
    constexpr bool HAS_D = Op::NSRC == 2;
    constexpr int TVA = TA / VEC, RS = kBlock / TVA, JT = TB / (VEC * RS);     // staging: threads along A, thread rows, passes of VEC * RS rows
    constexpr int TVB = TB / VEC, RT = kBlock / TVB, ITER_T = TA / RT;       // storing: threads along B, rows per pass, passes
    static_assert(TA % VEC == 0 && TB % 32 == 0 && kBlock % TVA == 0 && kBlock % TVB == 0 && TB % (VEC * RS) == 0 && TA % RT == 0 && TVA % 8 == 0,
                  "tile shape");
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    struct Group { S v[VEC]; };               // VEC consecutive b's of one a: 16 bytes
    extern __shared__ __align__(16) unsigned char tr_lds[];
    u32x4* l = (u32x4*)tr_lds;                // [TA][TVB] groups
    [[maybe_unused]] D* lv = (D*)(tr_lds + (size_t)TA * TB * sizeof(S));   // [TA] values of a source that has one per stored row
    constexpr int NDV = (TA + kBlock - 1) / kBlock;
    const S* sp = S1 ? (const S*)a : (const S*)b;
    const D* dp = S1 ? (const D*)b : (const D*)a;

    uint32_t bid = blockIdx.x;
    if (xcd_chunk) bid = (bid % 8u) * xcd_chunk + bid / 8u;
    const uint32_t tb = bid % p.tiles_b;
    bid /= p.tiles_b;
    const uint32_t ta = bid % p.tiles_a;
    bid /= p.tiles_a;
    const int64_t a0 = (int64_t)ta * TA, b0 = (int64_t)tb * TB;
    int64_t ot = a0 * p.sa[0] + b0 * p.sb[0], os = a0 * p.sa[KS] + b0 * p.sb[KS], od = a0 * p.sa[KD] + b0 * p.sb[KD];
    for (int d = p.nouter - 1; d >= 0; d--) {
        const uint32_t q = (d == 0) ? 0u : bid / p.oshape[d];
        const int64_t idx = bid - q * p.oshape[d];
        bid = q;
        ot += idx * p.ostride[0][d];
        os += idx * p.ostride[KS][d];
        od += idx * p.ostride[KD][d];
    }
    t += ot;
    sp += os;
    dp += od;
    // GEN: valid extent of this tile along A and B.  Positions outside it fetch what a position inside fetches, and what they put
    // into LDS is never stored.  (The staged source's rows are whole vectors, so la_n is a multiple of VEC.)
    const uint32_t la_n = GEN ? (uint32_t)min((int64_t)TA, (int64_t)p.na - a0) : (uint32_t)TA;
    const uint32_t lb_n = GEN ? (uint32_t)min((int64_t)TB, (int64_t)p.nb - b0) : (uint32_t)TB;

    const uint32_t gl = threadIdx.x % TVB, tx = gl * VEC, ty = threadIdx.x / TVB;
    const bool rows_only = p.dmode == 1;
    {
        const uint32_t lx = threadIdx.x % TVA, sy = threadIdx.x / TVA;    // a = VEC lx .. VEC lx + VEC - 1
        Pack<S, VEC> g[JT][VEC];
#pragma unroll
        for (int jt = 0; jt < JT; jt++)
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                const uint32_t rb = VEC * (RS * jt + sy) + k;
                const uint32_t rbc = (!GEN || rb < lb_n) ? rb : 0u, ac = (!GEN || VEC * lx < la_n) ? VEC * lx : 0u;
                g[jt][k] = load_pack<S, VEC>(sp + (int64_t)rbc * p.sb[KS] + ac);
            }
        // a source with one value per stored row: the tile's TA values go through LDS (one load per thread here, behind the staging
        // loads and ahead of the wait for them; fetched by every storing thread for its own rows they cost as many load
        // instructions as the tile itself)
        [[maybe_unused]] D dv[NDV];
        if constexpr (HAS_D) {
            if (rows_only) {
#pragma unroll
                for (int q = 0; q < NDV; q++) {
                    const uint32_t ia = (threadIdx.x + q * kBlock) % TA;
                    dv[q] = dp[(int64_t)((!GEN || ia < la_n) ? ia : 0u) * p.sa[KD]];
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int jt = 0; jt < JT; jt++) {
            const uint32_t grp = (RS * jt + sy) ^ (lx % 8u);
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                Group w;
#pragma unroll
                for (int k = 0; k < VEC; k++) w.v[k] = g[jt][k].v[e];
                l[(VEC * lx + e) * TVB + grp] = __builtin_bit_cast(u32x4, w);
            }
        }
        if constexpr (HAS_D) {
            if (rows_only) {
#pragma unroll
                for (int q = 0; q < NDV; q++) lv[(threadIdx.x + q * kBlock) % TA] = dv[q];
            }
        }
    }
    __syncthreads();
    // the row of this thread's i-th pass; GEN: rows beyond the tile's extent repeat its last row
    auto row_of = [&](int i) {
        const uint32_t r0 = ty + (uint32_t)i * RT;
        return !GEN ? r0 : (r0 < la_n ? r0 : la_n - 1u);
    };
    [[maybe_unused]] D pd[ITER_T];
    if constexpr (HAS_D) {
        if (rows_only) {
#pragma unroll
            for (int it = 0; it < ITER_T; it++) pd[it] = lv[row_of(it)];
        }
    }
    // MODE 1: the other source has one value per stored row (or there is none); MODE 2: it is broadcast or runs in vectors along B;
    // MODE 0 (GEN only): any strides, fetched element by element.  GEN: rows beyond the tile's extent repeat its last row (the same
    // values to the same addresses, so that no store sits behind a test); a vector that crosses the end of the target's row is
    // moved element by element, vectors beyond it are skipped.
    auto store_tile = [&](auto mode_tag) {
        constexpr int MODE = decltype(mode_tag)::value;
        const uint32_t cnt = !GEN ? (uint32_t)VEC : lb_n > tx ? min((uint32_t)VEC, lb_n - tx) : 0u;   // elements of this thread's vector inside the tile
        if (GEN && cnt == 0u) return;
        const bool whole = !GEN || cnt == (uint32_t)VEC;
        [[maybe_unused]] Pack<D, VEC> dd[ITER_T];
        if constexpr (HAS_D && MODE == 2) {
#pragma unroll
            for (int i = 0; i < ITER_T; i++) dd[i] = tr_direct_fast<D, VEC>(dp, row_of(i), whole ? tx : 0u, p.sa[KD], p.sb[KD]);
        }
        if constexpr (HAS_D && GEN && MODE != 1) {
            if (MODE == 0 || !whole) {
#pragma unroll
                for (int i = 0; i < ITER_T; i++) {
                    const int64_t ro = (int64_t)row_of(i) * p.sa[KD];
#pragma unroll
                    for (int e = 0; e < VEC; e++) dd[i].v[e] = dp[ro + (int64_t)((uint32_t)e < cnt ? tx + e : tx) * p.sb[KD]];
                }
            }
        }
#pragma unroll
        for (int i = 0; i < ITER_T; i++) {
            const uint32_t r = row_of(i);
            const Group w = __builtin_bit_cast(Group, l[r * TVB + (gl ^ ((r / (uint32_t)VEC) % 8u))]);
            Pack<T, VEC> res;
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                const S xs = w.v[e];
                D xd = D();
                if constexpr (HAS_D) xd = MODE == 1 ? pd[i] : dd[i].v[e];
                if constexpr (S1) res.v[e] = apply_op(op, xs, xd, C());
                else res.v[e] = apply_op(op, xd, xs, C());
            }
            if (whole) {
                store_pack<T, VEC>(t + (int64_t)r * p.sa[0] + tx, res);
            } else {
#pragma unroll
                for (int e = 0; e < VEC - 1; e++)
                    if ((uint32_t)e < cnt) t[(int64_t)r * p.sa[0] + tx + e] = res.v[e];
            }
        }
    };
    if constexpr (GEN && HAS_D) {
        if (p.dmode == 0) {
            store_tile(std::integral_constant<int, 0>{});
            return;
        }
    }
    if (!HAS_D || rows_only) store_tile(std::integral_constant<int, 1>{});
    else store_tile(std::integral_constant<int, 2>{});
}

// ---- launcher -------------------------------------------------------------------------------------------------------------

template <class Op>
constexpr int op_vec() {
    int m = (int)sizeof(typename Op::T);
    if (Op::NSRC >= 1 && (int)sizeof(typename Op::A) > m) m = (int)sizeof(typename Op::A);
    if (Op::NSRC >= 2 && (int)sizeof(typename Op::B) > m) m = (int)sizeof(typename Op::B);
    if (Op::NSRC >= 3 && (int)sizeof(typename Op::C) > m) m = (int)sizeof(typename Op::C);
    return 16 / m;
}

inline bool aligned_to(const void* p, size_t a) { return ((uintptr_t)p % a) == 0; }
// an operand of `esize`-byte elements can be moved in vectors of `vec` elements from `p` on: any address for elements of 4 bytes
// and more (PackWord), the vector's own alignment for narrower ones
inline bool vector_address(const void* p, int vec, size_t esize) { return esize >= 4 || aligned_to(p, vec * esize); }
// ... and a row pitch or outer stride of `stride` elements keeps every row's vectors addressable
inline bool vector_stride(int64_t stride, int vec, size_t esize) { return esize >= 4 || (stride % vec) == 0; }

constexpr uint32_t kMaxItems = 0xFFFF0000u;


template <class Op>
int32_t launch_map(const Op& op, const MapPlan& p, hipStream_t stream) {
    using T = typename Op::T;
    using A = typename Op::A;
    using B = typename Op::B;
    using C = typename Op::C;
    constexpr int VEC = op_vec<Op>();
    constexpr int NOPS = Op::NSRC + 1;
    if (p.total == 0) return DNH_OK;
    T* t = (T*)p.ptr[0];
    const A* a = (const A*)p.ptr[1];
    const B* b = (const B*)p.ptr[2];
    const C* c = (const C*)p.ptr[3];
    const size_t es[kMaxOperands] = {sizeof(T), sizeof(A), sizeof(B), sizeof(C)};
    const int nd = p.nd;
    const int last = nd - 1;

    // flat: one contiguous run per operand (or a broadcast scalar)
    bool flat = nd <= 1;
    if (flat && nd == 1) {
        flat = p.stride[0][0] == 1;
        for (int k = 1; k < NOPS; k++) flat = flat && (p.stride[k][0] == 1 || p.stride[k][0] == 0);
    }
    if (flat && nd == 1) {
        bool al = vector_address(t, VEC, es[0]);
        for (int k = 1; k < NOPS; k++)
            if (p.stride[k][0] == 1) al = al && vector_address(p.ptr[k], VEC, es[k]);
        if (al) {
            // one 16-byte vector per thread: measured fastest on MI355X (more per-thread unrolling lowers achieved bandwidth; for
            // narrowing ops such as int32 -> bool compares, four consecutive loads per thread to reach a 16-byte store measured
            // 25 % slower: each load instruction then uses only 32 bytes of every 128-byte line it touches)
            constexpr int UNROLL = 1;
            const int64_t nvec = p.total / VEC;
            const unsigned blocks = nvec ? cdiv(nvec, (int64_t)kBlock * UNROLL) : 1;
            hipLaunchKernelGGL((map_flat_kernel<Op, VEC, UNROLL>), dim3(blocks), dim3(kBlock), 0, stream, op, t, a, b, c,
                               (int)p.stride[1][0], (int)p.stride[2][0], (int)p.stride[3][0], p.total);
            DNH_LAUNCH_CHECK();
            return DNH_OK;
        }
    }

    if (nd >= 1 && p.total > (int64_t)kMaxItems) {
        // split the outermost dimension so each launch indexes fewer than 2^32 items
        MapPlan q = p;
        const int64_t inner = p.total / p.shape[0];
        if (inner > (int64_t)kMaxItems) return fail(DNH_ERR_NOT_SUPPORTED, "element-wise op: inner extent of %lld elements exceeds the 32-bit index range", (long long)inner);
        const int64_t chunk = (int64_t)kMaxItems / inner;
        for (int64_t s = 0; s < p.shape[0]; s += chunk) {
            const int64_t len = (p.shape[0] - s) < chunk ? (p.shape[0] - s) : chunk;
            q.shape[0] = len;
            q.total = len * inner;
            for (int k = 0; k < NOPS; k++) q.ptr[k] = p.ptr[k] + s * p.stride[k][0] * (int64_t)es[k];
            DNH_TRY(launch_map(op, q, stream));
        }
        return DNH_OK;
    }

    // transposing path: the target runs along `last`, some source along another dimension
    if (nd >= 2 && p.stride[0][last] == 1) {
        int dA = -1;
        for (int k = 1; k < NOPS && dA < 0; k++) {
            if (p.stride[k][last] == 0 || p.stride[k][last] == 1) continue;
            for (int d = 0; d < last; d++)
                if (p.stride[k][d] == 1 && p.shape[d] >= 16) { dA = d; break; }
        }
        if (dA >= 0 && p.shape[last] >= 16) {
            // Tile shapes (elements along A x along B), chosen from measurements of 512 MiB transposing copies on MI355X:
            //   4-byte and narrower elements: 128 x 64 (512-byte row pieces on the read side, 256-byte on the write side; 72 % of
            //   the HBM peak for both 256 x 524288 and 131072 x 1024 sources, against 71 % and 55 % with 64 x 64);
            //   when the target's rows are short (at most 256 elements) and one source is staged, 256 x 128 tiles (one workgroup per
            //   CU with 128 KB of LDS, all of a thread's 32 loads in flight): 77 % for the 256 x 524288 case;
            //   8-byte elements: 64 x 32.
            constexpr bool WIDE = sizeof(T) > 4 || (Op::NSRC >= 1 && sizeof(A) > 4) || (Op::NSRC >= 2 && sizeof(B) > 4) ||
                                  (Op::NSRC >= 3 && sizeof(C) > 4);
            constexpr int TA = WIDE ? 64 : 128, TB = WIDE ? 32 : 64;
            constexpr int ESZ = WIDE ? 8 : 4;                       // element size of the large tiles' staged source
            constexpr int BIG_TA = WIDE ? 128 : 256, BIG_TB = 128;
            TrArgs q;
            memset(&q, 0, sizeof(q));
            q.na = (uint32_t)p.shape[dA];
            q.nb = (uint32_t)p.shape[last];
            int64_t outer = 1;
            for (int d = 0; d < last; d++) {
                if (d == dA) continue;
                q.oshape[q.nouter] = (uint32_t)p.shape[d];
                for (int k = 0; k < NOPS; k++) q.ostride[k][q.nouter] = p.stride[k][d];
                outer *= p.shape[d];
                q.nouter++;
            }
            int nstaged = 0;
            size_t staged_esize = 0;
            for (int k = 0; k < NOPS; k++) {
                q.sa[k] = p.stride[k][dA];
                q.sb[k] = p.stride[k][last];
                q.staged[k] = (k >= 1 && p.stride[k][dA] == 1 && p.stride[k][last] != 0 && p.stride[k][last] != 1) ? 1 : 0;
                if (q.staged[k]) { nstaged++; staged_esize = es[k]; }
            }
            // vector path: every tile row a whole number of aligned vectors for the target and every staged source
            // (rows that are not whole vectors end inside one vector of an edge tile: the kernel moves that one element by element)
            bool vec = VEC > 1 && vector_address(t, VEC, es[0]) && vector_stride(q.sa[0], VEC, es[0]);
            for (int d = 0; d < q.nouter && vec; d++) vec = vector_stride(q.ostride[0][d], VEC, es[0]);
            for (int k = 1; k < NOPS && vec; k++) {
                if (!q.staged[k]) continue;
                vec = vector_address(p.ptr[k], VEC, es[k]) && vector_stride(q.sb[k], VEC, es[k]);
                for (int d = 0; d < q.nouter && vec; d++) vec = vector_stride(q.ostride[k][d], VEC, es[k]);
            }
            // sources that are not staged: all broadcast along B, or each broadcast or in aligned vectors along B, lets the kernel fetch
            // them without branches
            q.dmode = 1;
            for (int k = 1; k < NOPS; k++) {
                if (q.staged[k] || q.sb[k] == 0) continue;
                if (q.dmode == 1) q.dmode = 2;
                if (!vec) continue;   // the element-wise kernel fetches single elements either way
                bool ok = q.sb[k] == 1 && vector_address(p.ptr[k], VEC, es[k]) && vector_stride(q.sa[k], VEC, es[k]);
                for (int d = 0; d < q.nouter && ok; d++) ok = vector_stride(q.ostride[k][d], VEC, es[k]);
                if (!ok) q.dmode = 0;
            }
            // Large tiles (128 KB of LDS, one workgroup per CU) for 4- and 8-byte elements in whole tiles with one staged source:
            //   256 x 128 (8-byte elements: 128 x 128) when the target's rows are short (at most 256 elements);
            //   128 x 256 (8-byte: 128 x 128; map_tr4_kernel only) for longer rows whose pitch in the target stays below 256 KB: 512 MiB copies of
            //   8192 x 16384 250 -> 180 us, 16384 x 8192 207 -> 196, 1024 x 131072 207 -> 175, 64 x [2048 x 1024] 188 -> 167;
            //   with a target pitch of 512 KB (131072 x 1024, or 256 x 512 x 1024 permuted to 1024 x 256 x 512) every large
            //   tile shape and tile order measured 186 us or more, the 128 x 64 tiles' time, so those keep them.
            //   8-byte elements (512 MiB copies, 64 x 32 tiles of map_tr_kernel before): 8192 x 8192 244 -> 181 us, 4096 x 16384 245 -> 182,
            //   16384 x 4096 216 -> 195, 1024 x 65536 198 -> 174, 64 x [1024 x 1024] 197 -> 164, [256, 512, 512] permuted to [512, 512, 256]
            //   185 -> 173; 64 x 256, 256 x 64 and 32 x 512 tiles measured no better than 128 x 128 over these layouts.
            bool big = false, tall = false, tr4 = false, tr4_gen = false;
            constexpr int TALL_TA = 128, TALL_TB = WIDE ? 128 : 256;
            if constexpr (VEC == 16 / ESZ && Op::NSRC >= 1 && Op::NSRC <= 2) {
                const bool tr4_on = option(OPT_TR4) != 0;
                const bool tr4_ok = tr4_on && (Op::NSRC == 1 || q.dmode != 0);
                const bool one4 = vec && nstaged == 1 && staged_esize == ESZ;
                big = (tr4_ok || !WIDE) && one4 && q.nb <= 256 && (q.na % BIG_TA) == 0 && (q.nb % BIG_TB) == 0 &&
                      (int64_t)(q.na / BIG_TA) * (q.nb / BIG_TB) * outer >= (int64_t)device_cus() * 8;
                tall = !big && tr4_ok && one4 && q.nb > 256 && (q.na % TALL_TA) == 0 && (q.nb % TALL_TB) == 0 &&
                       q.sa[0] * (int64_t)es[0] < 256 * 1024 &&
                       (int64_t)(q.na / TALL_TA) * (q.nb / TALL_TB) * outer >= (int64_t)device_cus() * 8;
                tr4 = tr4_ok && (big || tall);
                // short rows that are ragged in any way (extents that are not multiples of the tile, rows that are not whole vectors,
                // a second operand with other strides): the kernel's general form on the 256-row tiles, whose rows follow one another
                // in a contiguous target ([250, 500, 1000] permuted to [500, 1000, 250]: 128 x 64 tiles 337 us)
                if (!tr4 && tr4_on && one4 && q.nb <= 256 && (q.na % VEC) == 0 &&
                    (int64_t)cdiv(q.na, BIG_TA) * cdiv(q.nb, BIG_TB) * outer >= (int64_t)device_cus() * 8) {
                    tr4 = tr4_gen = big = true;
                    tall = false;
                }
            }
            const int ta_n = big ? BIG_TA : tall ? TALL_TA : TA, tb_n = big ? BIG_TB : tall ? TALL_TB : TB;
            q.tiles_a = cdiv(q.na, ta_n);
            q.tiles_b = cdiv(q.nb, tb_n);
            uint32_t lds_bytes = 0;
            for (int k = 1; k < NOPS; k++) {
                if (!q.staged[k]) continue;
                q.lds_off[k] = lds_bytes;
                lds_bytes += (uint32_t)(((size_t)tb_n * (ta_n + 1) * es[k] + 15) / 16 * 16);
            }
            const int64_t blocks = (int64_t)q.tiles_a * q.tiles_b * outer;
            if (blocks <= 0x7FFFFFFF) {
                const uint32_t xcd_chunk = (!big && !tall && blocks % 8 == 0 && blocks >= 64) ? (uint32_t)(blocks / 8) : 0u;
                const int mask = (q.staged[1] ? 1 : 0) | (q.staged[2] ? 2 : 0) | (q.staged[3] ? 4 : 0);
                int32_t st = DNH_ERR_NOT_SUPPORTED;
                // launches map_tr_kernel<Op, TA_, TB_, V_, M_>; more than 64 KB of LDS (two or three staged sources, or the large tile)
                // have to be asked for once per kernel
#define DNH_TR_LAUNCH(TA_, TB_, V_, M_)                                                                                                   \
    do {                                                                                                                                  \
        auto kern = map_tr_kernel<Op, TA_, TB_, V_, M_>;                                                                                  \
        static const hipError_t attr = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,                 \
                                                          3 * (TB_ * (TA_ + 1) * (WIDE ? 8 : 4) + 16) > 160 * 1024 ? 160 * 1024           \
                                                                                                               : 3 * (TB_ * (TA_ + 1) * (WIDE ? 8 : 4) + 16)); \
        if (attr != hipSuccess) { st = fail(DNH_ERR_HIP, "hipFuncSetAttribute: %s", hipGetErrorString(attr)); break; }                    \
        hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(kBlock), lds_bytes, stream, op, t, a, b, c, q, xcd_chunk);                   \
        st = DNH_OK;                                                                                                                      \
    } while (0)
#define DNH_TR_MASKS(TA_, TB_, V_)                                                                       \
    do {                                                                                                 \
        if constexpr (Op::NSRC == 1) { DNH_TR_LAUNCH(TA_, TB_, V_, 1); }                                 \
        else if constexpr (Op::NSRC == 2) {                                                              \
            if (mask == 1) DNH_TR_LAUNCH(TA_, TB_, V_, 1);                                               \
            else if (mask == 2) DNH_TR_LAUNCH(TA_, TB_, V_, 2);                                          \
            else DNH_TR_LAUNCH(TA_, TB_, V_, 3);                                                         \
        } else if constexpr (Op::NSRC == 3) {                                                            \
            switch (mask) {                                                                              \
                case 1: DNH_TR_LAUNCH(TA_, TB_, V_, 1); break;                                           \
                case 2: DNH_TR_LAUNCH(TA_, TB_, V_, 2); break;                                           \
                case 3: DNH_TR_LAUNCH(TA_, TB_, V_, 3); break;                                           \
                case 4: DNH_TR_LAUNCH(TA_, TB_, V_, 4); break;                                           \
                case 5: DNH_TR_LAUNCH(TA_, TB_, V_, 5); break;                                           \
                case 6: DNH_TR_LAUNCH(TA_, TB_, V_, 6); break;                                           \
                default: DNH_TR_LAUNCH(TA_, TB_, V_, 7); break;                                          \
            }                                                                                            \
        }                                                                                                \
    } while (0)
#define DNH_TR4_LAUNCH(TA_, TB_, M_, G_)                                                                                                  \
    do {                                                                                                                                  \
        auto kern = map_tr4_kernel<Op, TA_, TB_, M_, G_>;                                                                                   \
        static const hipError_t attr = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, TA_ * TB_ * ESZ + TA_ * 8); \
        if (attr != hipSuccess) { st = fail(DNH_ERR_HIP, "hipFuncSetAttribute: %s", hipGetErrorString(attr)); break; }                    \
        hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(kBlock), (size_t)TA_ * TB_ * ESZ + TA_ * 8, stream, op, t, a, b, q, xcd_chunk);                    \
        st = DNH_OK;                                                                                                                      \
    } while (0)
                if (tr4) {
                    if constexpr (VEC == 16 / ESZ && Op::NSRC >= 1 && Op::NSRC <= 2) {
                        // (the staged source is the one of four bytes: `staged_esize` above)
#define DNH_TR4_PICK(TA_, TB_, G_)                                                                       \
    do {                                                                                                 \
        if (mask == 1) {                                                                                 \
            if constexpr (sizeof(A) == ESZ) DNH_TR4_LAUNCH(TA_, TB_, 1, G_);                             \
        } else if constexpr (Op::NSRC == 2) {                                                            \
            if constexpr (sizeof(B) == ESZ) DNH_TR4_LAUNCH(TA_, TB_, 2, G_);                             \
        }                                                                                                \
    } while (0)
                        if (tr4_gen) DNH_TR4_PICK(BIG_TA, BIG_TB, true);
                        else if (big) DNH_TR4_PICK(BIG_TA, BIG_TB, false);
                        else DNH_TR4_PICK(TALL_TA, TALL_TB, false);
#undef DNH_TR4_PICK
                    }
                } else if (big) {
                    if constexpr (!WIDE && VEC == 4 && Op::NSRC >= 1 && Op::NSRC <= 2) {
                        if constexpr (Op::NSRC == 1) DNH_TR_LAUNCH(BIG_TA, BIG_TB, 4, 1);
                        else if (mask == 1) DNH_TR_LAUNCH(BIG_TA, BIG_TB, 4, 1);
                        else DNH_TR_LAUNCH(BIG_TA, BIG_TB, 4, 2);
                    }
                } else if (vec) {
                    DNH_TR_MASKS(TA, TB, VEC);
                } else {
                    DNH_TR_MASKS(TA, TB, 1);
                }
#undef DNH_TR4_LAUNCH
#undef DNH_TR_MASKS
#undef DNH_TR_LAUNCH
                DNH_TRY(st);
                DNH_LAUNCH_CHECK();
                return DNH_OK;
            }
        }
    }

    // generic n-d
    NdArgs q;
    memset(&q, 0, sizeof(q));
    q.nd = nd < 1 ? 1 : nd;
    for (int d = 0; d < q.nd; d++) {
        q.shape[d] = (uint32_t)p.shape[d];
        for (int k = 0; k < NOPS; k++) q.stride[k][d] = p.stride[k][d];
    }
    bool vec = VEC > 1 && nd >= 1 && p.stride[0][last] == 1 && (p.shape[last] % VEC) == 0 && vector_address(t, VEC, es[0]);
    for (int k = 1; k < NOPS && vec; k++) {
        vec = vec && (p.stride[k][last] == 0 || p.stride[k][last] == 1);
        if (p.stride[k][last] == 1) vec = vec && vector_address(p.ptr[k], VEC, es[k]);
    }
    for (int d = 0; d < last && vec; d++)
        for (int k = 0; k < NOPS; k++)
            if (p.stride[k][last] == 1) vec = vec && vector_stride(p.stride[k][d], VEC, es[k]);
    // the target runs along the last dimension but something else keeps the vector form away: per-operand access modes
    if constexpr (VEC > 1) {
        if (!vec && nd >= 1 && p.stride[0][last] == 1 && p.shape[last] >= 4 * VEC) {
            NdMixArgs mx;
            memset(&mx, 0, sizeof(mx));
            const int64_t L = p.shape[last];
            for (int k = 0; k < NOPS; k++) {
                bool whole_vectors = p.stride[k][last] == 1 && vector_address(p.ptr[k], VEC, es[k]);
                for (int d = 0; d < last && whole_vectors; d++) whole_vectors = vector_stride(p.stride[k][d], VEC, es[k]);
                mx.mode[k] = (k > 0 && p.stride[k][last] == 0) ? 0 : whole_vectors ? 1 : 2;
                mx.estride[k] = p.stride[k][last];
                q.stride[k][last] = p.stride[k][last] * VEC;
            }
            mx.lastlen = (uint32_t)L;
            q.shape[last] = (uint32_t)((L + VEC - 1) / VEC);
            for (int d = 0; d < q.nd; d++) q.div[d] = make_fast_div(q.shape[d]);
            const int64_t nitems64 = (p.total / L) * q.shape[last];
            if (nitems64 <= (int64_t)kMaxItems) {
                const uint32_t nitems = (uint32_t)nitems64;
                hipLaunchKernelGGL((map_nd_mix_kernel<Op, VEC>), dim3(cdiv(nitems, kBlock)), dim3(kBlock), 0, stream, op, t, a, b, c, q, mx, nitems);
                DNH_LAUNCH_CHECK();
                return DNH_OK;
            }
            q.shape[last] = (uint32_t)p.shape[last];
            for (int k = 0; k < NOPS; k++) q.stride[k][last] = p.stride[k][last];
        }
    }
    constexpr int UNROLL = 1;
    if (vec) q.shape[last] = (uint32_t)(p.shape[last] / VEC);
    for (int d = 0; d < q.nd; d++) q.div[d] = make_fast_div(q.shape[d]);
    if (vec) {
        for (int k = 0; k < NOPS; k++) {
            q.vecload[k] = p.stride[k][last] == 1;
            q.stride[k][last] = p.stride[k][last] * VEC;
        }
        const uint32_t nitems = (uint32_t)(p.total / VEC);
        if (q.nd == 2) hipLaunchKernelGGL((map_nd_kernel<Op, VEC, UNROLL, 2>), dim3(cdiv(nitems, kBlock * UNROLL)), dim3(kBlock), 0, stream, op, t, a, b, c, q, nitems);
        else hipLaunchKernelGGL((map_nd_kernel<Op, VEC, UNROLL, 0>), dim3(cdiv(nitems, kBlock * UNROLL)), dim3(kBlock), 0, stream, op, t, a, b, c, q, nitems);
    } else {
        const uint32_t nitems = (uint32_t)p.total;
        hipLaunchKernelGGL((map_nd_kernel<Op, 1, UNROLL, 0>), dim3(cdiv(nitems, kBlock * UNROLL)), dim3(kBlock), 0, stream, op, t, a, b, c, q, nitems);
    }
    DNH_LAUNCH_CHECK();
    return DNH_OK;
}

// The arithmetic and comparison entry points are spread over four and two translation units (the element-wise instantiations dominate
// the library's build time, and the units compile side by side).
// map_numeric: a binary arithmetic op OpT on every numeric element type; each unit instantiates it for its own ops.
template <template <class> class OpT>
int32_t map_numeric(int dt, const MapPlan& p, hipStream_t s) {
    switch (dt) {
        case DNH_U8: return launch_map(OpT<uint8_t>{}, p, s);
        case DNH_I8: return launch_map(OpT<int8_t>{}, p, s);
        case DNH_I16: return launch_map(OpT<int16_t>{}, p, s);
        case DNH_U16: return launch_map(OpT<uint16_t>{}, p, s);
        case DNH_I32: return launch_map(OpT<int32_t>{}, p, s);
        case DNH_U32: return launch_map(OpT<uint32_t>{}, p, s);
        case DNH_I64: return launch_map(OpT<int64_t>{}, p, s);
        case DNH_U64: return launch_map(OpT<uint64_t>{}, p, s);
        case DNH_F32: return launch_map(OpT<float>{}, p, s);
        case DNH_F64: return launch_map(OpT<double>{}, p, s);
    }
    return fail(DNH_ERR_NOT_SUPPORTED, "binary arithmetic op is not defined for %s", dtype_name(dt));
}

int32_t binary_second_unit(int32_t op, int dt, const MapPlan& p, hipStream_t s);    // Divide, Modulo
int32_t binary_third_unit(int32_t op, int dt, const MapPlan& p, hipStream_t s);     // MaxElemwise, MinElemwise
int32_t binary_fourth_unit(int32_t op, int dt, const MapPlan& p, hipStream_t s);    // Multiply, Power
int32_t compare_second_unit(int32_t op, int dt, const MapPlan& p, hipStream_t s);   // LessOrEqual, Greater, GreaterOrEqual

}  // namespace dnh
