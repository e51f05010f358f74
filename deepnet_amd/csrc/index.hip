// dnh_gather, dnh_scatter, dnh_masked_get, dnh_masked_set, dnh_true_indices:
// ITensorBackend Gather / Scatter / MaskedGet / MaskedSet / TrueIndices (Tensor/Tensor/TensorBackend.fs:119-123);
// semantics Tensor/Tensor/Host/ScalarOps.fs:583-604 and :667-707.
//
// Gather/Scatter: one lane per target (gather) or source (scatter) element; an index outside the indexed tensor sets the
// library's error word and skips the element (the host reference raises, Host/FastAccess.fs:51-61).
// MaskedGet/MaskedSet/TrueIndices are order-preserving stream compactions over the row-major element order:
//   pass 1 counts selected elements per 4096-element block, pass 2 scans the block counts (one block),
//   pass 3 re-evaluates the selection, ranks within the block (wavefront shuffle scan + LDS) and moves the data.
#include "map_kernels.h"

using namespace dnh;

namespace {

struct Lay {
    int nd;
    uint32_t shape[DNH_MAX_DIMS];
    int64_t stride[DNH_MAX_DIMS];
};

Lay lay_of(const DnhTensor* t) {
    Lay l;
    l.nd = t->ndims;
    for (int d = 0; d < DNH_MAX_DIMS; d++) {
        l.shape[d] = d < t->ndims ? (uint32_t)t->shape[d] : 1;
        l.stride[d] = d < t->ndims ? t->stride[d] : 0;
    }
    return l;
}

// row-major position of linear index i; returns the element offset
__device__ __forceinline__ int64_t unravel(const Lay& l, uint32_t i, uint32_t* pos) {
    int64_t off = 0;
    for (int d = l.nd - 1; d >= 0; d--) {
        const uint32_t q = (d == 0) ? 0u : i / l.shape[d];
        const uint32_t p = i - q * l.shape[d];
        i = q;
        pos[d] = p;
        off += (int64_t)p * l.stride[d];
    }
    return off;
}
__device__ __forceinline__ int64_t offset_of(const Lay& l, uint32_t i) {
    int64_t off = 0;
    for (int d = l.nd - 1; d >= 0; d--) {
        const uint32_t q = (d == 0) ? 0u : i / l.shape[d];
        off += (int64_t)(i - q * l.shape[d]) * l.stride[d];
        i = q;
    }
    return off;
}

// ---- gather / scatter -------------------------------------------------------------------------------------------------------

struct IndexArgs {
    Lay iter;                              // the iteration space: target (gather) or source (scatter)
    Lay other;                             // the indexed tensor: source (gather) or target (scatter)
    int64_t other_shape[DNH_MAX_DIMS];     // its extents in full width: the indexed tensor may hold more than 2^32 elements
    const int64_t* idx[DNH_MAX_DIMS];      // per dimension of `other`; nullptr = identity
    int64_t idx_stride[DNH_MAX_DIMS][DNH_MAX_DIMS];
};

__device__ __forceinline__ bool indexed_offset(const IndexArgs& a, const uint32_t* pos, int64_t* off) {
    int64_t o = 0;
    bool ok = true;
    for (int d = 0; d < a.other.nd; d++) {
        int64_t j;
        if (a.idx[d]) {
            int64_t io = 0;
            for (int e = 0; e < a.iter.nd; e++) io += (int64_t)pos[e] * a.idx_stride[d][e];
            j = a.idx[d][io];
        } else {
            j = pos[d];
        }
        ok = ok && j >= 0 && j < a.other_shape[d];
        o += j * a.other.stride[d];
    }
    *off = o;
    return ok;
}

template <class W>
__global__ __launch_bounds__(kBlock) void gather_kernel(W* t, const W* s, IndexArgs a, uint32_t n, int32_t* err) {
    const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    uint32_t pos[DNH_MAX_DIMS];
    const int64_t toff = unravel(a.iter, i, pos);
    int64_t soff;
    if (indexed_offset(a, pos, &soff)) t[toff] = s[soff];
    else *err = 1;
}

template <class X> __device__ __forceinline__ void atomic_add_any(X* p, X v) { atomicAdd(p, v); }
template <> __device__ __forceinline__ void atomic_add_any<int64_t>(int64_t* p, int64_t v) { atomicAdd((unsigned long long*)p, (unsigned long long)v); }
template <> __device__ __forceinline__ void atomic_add_any<uint64_t>(uint64_t* p, uint64_t v) { atomicAdd((unsigned long long*)p, (unsigned long long)v); }
// one-byte integers: compare-and-swap on the containing 32-bit word
template <> __device__ __forceinline__ void atomic_add_any<uint8_t>(uint8_t* p, uint8_t v) {
    uint32_t* w = (uint32_t*)((uintptr_t)p & ~(uintptr_t)3);
    const unsigned sh = ((uintptr_t)p & 3) * 8;
    uint32_t old = *w, assumed;
    do {
        assumed = old;
        const uint32_t b = ((assumed >> sh) + v) & 0xFFu;
        old = atomicCAS(w, assumed, (assumed & ~(0xFFu << sh)) | (b << sh));
    } while (old != assumed);
}

// two-byte integers: the same on the containing 32-bit word
template <> __device__ __forceinline__ void atomic_add_any<uint16_t>(uint16_t* p, uint16_t v) {
    uint32_t* w = (uint32_t*)((uintptr_t)p & ~(uintptr_t)3);
    const unsigned sh = ((uintptr_t)p & 2) * 8;
    uint32_t old = *w, assumed;
    do {
        assumed = old;
        const uint32_t b = ((assumed >> sh) + v) & 0xFFFFu;
        old = atomicCAS(w, assumed, (assumed & ~(0xFFFFu << sh)) | (b << sh));
    } while (old != assumed);
}

template <class X>
__global__ __launch_bounds__(kBlock) void scatter_kernel(X* t, const X* s, IndexArgs a, uint32_t n, int32_t* err) {
    const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    uint32_t pos[DNH_MAX_DIMS];
    const int64_t soff = unravel(a.iter, i, pos);
    int64_t toff;
    if (indexed_offset(a, pos, &toff)) atomic_add_any<X>(t + toff, s[soff]);
    else *err = 1;
}

int32_t make_index_args(IndexArgs* a, const DnhTensor* iter, const DnhTensor* other, const DnhTensor* const* idx, int32_t n_idx, const char* what) {
    DNH_TRY(check_tensor(iter, what));
    DNH_TRY(check_tensor(other, what));
    if (iter->dtype != other->dtype) return fail(DNH_ERR_INVALID_ARG, "%s: source and target dtypes differ", what);
    if (n_idx != other->ndims) return fail(DNH_ERR_INVALID_ARG, "%s: %d index tensors given for a tensor of rank %d", what, n_idx, other->ndims);
    if (n_idx > 0 && !idx) return fail(DNH_ERR_INVALID_ARG, "%s: null index list", what);
    memset(a, 0, sizeof(*a));
    a->iter = lay_of(iter);
    a->other = lay_of(other);
    for (int d = 0; d < DNH_MAX_DIMS; d++) a->other_shape[d] = d < other->ndims ? other->shape[d] : 1;
    for (int d = 0; d < n_idx; d++) {
        if (idx[d]) {
            DNH_TRY(check_tensor(idx[d], what));
            if (idx[d]->dtype != DNH_I64) return fail(DNH_ERR_INVALID_ARG, "%s: index tensors must be int64", what);
            if (!same_shape(idx[d], iter)) return fail(DNH_ERR_INVALID_ARG, "%s: index tensor %d is not broadcast to the iteration shape", what, d);
            a->idx[d] = (const int64_t*)elem_ptr(idx[d]);
            for (int e = 0; e < iter->ndims; e++) a->idx_stride[d][e] = idx[d]->stride[e];
        } else if (d >= iter->ndims) {
            return fail(DNH_ERR_INVALID_ARG, "%s: dimension %d has no index tensor and no matching dimension to map identically", what, d);
        }
    }
    return DNH_OK;
}

// ---- compaction -------------------------------------------------------------------------------------------------------------

constexpr int kItems = 16;                     // consecutive elements per thread
constexpr int kChunk = kBlock * kItems;        // elements per block

struct MaskArgs {
    Lay full;                                  // the masked tensor (source of MaskedGet, target of MaskedSet, source of TrueIndices)
    const uint8_t* mask[DNH_MAX_DIMS];         // per-dimension rank-1 masks (nullptr = all true) — or mask[0] = the bool tensor itself
    int64_t mask_stride[DNH_MAX_DIMS];
    int whole;                                 // 1: mask[0] is a bool tensor with layout `full` (TrueIndices)
};

__device__ __forceinline__ bool selected(const MaskArgs& m, const uint32_t* pos, int64_t off) {
    if (m.whole) return m.mask[0][off] != 0;
    bool s = true;
    for (int d = 0; d < m.full.nd; d++)
        if (m.mask[d]) s = s && m.mask[d][(int64_t)pos[d] * m.mask_stride[d]] != 0;
    return s;
}

// exclusive prefix of `c` over the block; `total` receives the block sum
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t c, uint32_t* total) {
    __shared__ uint32_t wave_sum[kBlock / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t inc = c;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t y = (uint32_t)__shfl_up((int)inc, d, 64);
        if (lane >= d) inc += y;
    }
    if (lane == 63) wave_sum[wave] = inc;
    __syncthreads();
    uint32_t base = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < kBlock / 64; w++) {
        if (w < wave) base += wave_sum[w];
        tot += wave_sum[w];
    }
    *total = tot;
    return base + inc - c;
}

// ---- binned scatter ------------------------------------------------------------------------------------------------------------
// t[idx[i]] += s[i] for 32-bit integers, every tensor rank 1 with unit stride, many updates into a large table.  A random update
// costs the memory system a 32-byte read-modify-write at the memory side (device-scope atomics do not run in the per-XCD L2):
// 4 Mi of them into a 64 MB table take 166 us.  Here the (index, value) pairs are first sorted by bucket of kBinElems consecutive
// target elements, then one workgroup per bucket sums its pairs in LDS and adds the bucket to the table in one coalesced pass, so
// the table is read and written once, in whole lines:
//   1. bin_count:   each workgroup counts its kBinChunk pairs per bucket (LDS histogram)            -> counts[workgroup][bucket]
//   2. bin_colscan: exclusive prefix of every bucket's column of counts, and the bucket totals       -> counts (in place), totals[bucket]
//   3. bin_move:    each workgroup ranks its pairs by bucket in LDS and writes them out in runs      -> pairs (bucket order)
//   4. bin_apply:   one workgroup per bucket: LDS accumulate (integer adds commute: bit-exact and deterministic), then table += sums
// An index outside the table sets the error word and is skipped, as in the direct kernel.
constexpr int kBinShift = 14;
constexpr uint32_t kBinElems = 1u << kBinShift;          // target elements per bucket: 64 KB of LDS
constexpr uint32_t kBinChunk = 8192;                      // pairs per workgroup of passes 1 and 3
constexpr uint32_t kBinMaxBuckets = 4096;                 // LDS histogram of passes 1 and 3
constexpr int kBinThreads = 1024;                         // passes 1, 3 and 4: many wavefronts per workgroup cover the latency of their few, dependent steps
constexpr int kBinPerThread = kBinChunk / kBinThreads;

// exclusive prefix of `c` over a workgroup of kBinThreads threads; `total` receives the sum.  `wave_sum`: kBinThreads / 64 words of LDS,
// free for reuse after the call's second barrier.
__device__ __forceinline__ uint32_t bin_block_scan(uint32_t c, uint32_t* total, uint32_t* wave_sum) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t inc = c;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t y = (uint32_t)__shfl_up((int)inc, d, 64);
        if (lane >= d) inc += y;
    }
    if (lane == 63) wave_sum[wave] = inc;
    __syncthreads();
    uint32_t base = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < kBinThreads / 64; w++) {
        const uint32_t x = wave_sum[w];
        if (w < wave) base += x;
        tot += x;
    }
    __syncthreads();
    *total = tot;
    return base + inc - c;
}

__global__ __launch_bounds__(kBinThreads) void bin_count_kernel(const int64_t* __restrict__ idx, uint32_t m, int64_t n, uint32_t nb, uint32_t nchunks,
                                                                uint32_t* __restrict__ counts, int32_t* err) {
    extern __shared__ uint32_t bin_lds[];   // nb counters
    uint32_t* hist = bin_lds;
    for (uint32_t b = threadIdx.x; b < nb; b += kBinThreads) hist[b] = 0;
    const uint32_t i0 = blockIdx.x * kBinChunk;
    bool bad = false;
    int64_t jj[kBinPerThread];   // every load is issued before the first LDS atomic: a load inside the loop would wait for the one before it
#pragma unroll
    for (int e = 0; e < kBinPerThread; e++) {
        const uint32_t i = i0 + e * kBinThreads + threadIdx.x;
        jj[e] = i < m ? __builtin_nontemporal_load(idx + i) : 0;
    }
    __syncthreads();
#pragma unroll
    for (int e = 0; e < kBinPerThread; e++) {
        const uint32_t i = i0 + e * kBinThreads + threadIdx.x;
        if (i < m) {
            if (jj[e] >= 0 && jj[e] < n) atomicAdd(&hist[(uint32_t)(jj[e] >> kBinShift)], 1u);
            else bad = true;
        }
    }
    if (bad) *err = 1;
    __syncthreads();
    for (uint32_t b = threadIdx.x; b < nb; b += kBinThreads) counts[(size_t)blockIdx.x * nb + b] = hist[b];
}

// counts is [workgroup of pass 1][bucket] (rows written and read whole); this pass replaces every column by its exclusive prefix
// and leaves the column sums in totals.  A workgroup owns 64 adjacent buckets: lanes run along the buckets (256-byte row pieces),
// the 16 wavefronts split a tile of 512 rows, 32 rows each (all loads of a tile in flight together), and the tiles follow one another with a running carry per bucket.
__global__ __launch_bounds__(kBinThreads) void bin_colscan_kernel(uint32_t* __restrict__ counts, uint32_t* __restrict__ totals, uint32_t nb, uint32_t nchunks) {
    constexpr int GROUPS = kBinThreads / 64, ROWS = 32;
    __shared__ uint32_t gsum[GROUPS][64];
    const uint32_t lane = threadIdx.x & 63, g = threadIdx.x >> 6;
    const uint32_t b = blockIdx.x * 64 + lane;
    const bool live = b < nb;
    uint32_t carry = 0;
    for (uint32_t k0 = 0; k0 < nchunks; k0 += GROUPS * ROWS) {
        uint32_t c[ROWS], sum = 0;
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            const uint32_t k = k0 + g * ROWS + r;
            c[r] = (live && k < nchunks) ? counts[(size_t)k * nb + b] : 0u;
        }
#pragma unroll
        for (int r = 0; r < ROWS; r++) sum += c[r];
        gsum[g][lane] = sum;
        __syncthreads();
        uint32_t run = carry, all = 0;
#pragma unroll
        for (int w = 0; w < GROUPS; w++) {
            const uint32_t x = gsum[w][lane];
            if (w < (int)g) run += x;
            all += x;
        }
        carry += all;
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            const uint32_t k = k0 + g * ROWS + r;
            if (live && k < nchunks) counts[(size_t)k * nb + b] = run;
            run += c[r];
        }
        __syncthreads();
    }
    if (live && g == 0) totals[b] = carry;
}

__global__ __launch_bounds__(kBinThreads) void bin_move_kernel(const int64_t* __restrict__ idx, const uint32_t* __restrict__ src, uint32_t m, int64_t n,
                                                               uint32_t nb, uint32_t nchunks, const uint32_t* __restrict__ counts,
                                                               const uint32_t* __restrict__ totals, uint2* __restrict__ pairs) {
    constexpr int PER = kBinMaxBuckets / kBinThreads;   // buckets per thread in the two prefix sums
    __shared__ uint2 sorted[kBinChunk];           // (index into the table, value), grouped by bucket; the index holds bucket and offset
    __shared__ uint32_t wave_sum[kBinThreads / 64];
    extern __shared__ uint32_t bin_lds[];         // 2 * nb words, sized by the launch so that two workgroups fit a CU for tables up to 64 MB
    uint32_t* cursor = bin_lds;                   // next free slot of each bucket's group in `sorted`
    uint32_t* gbase = bin_lds + nb;               // where this workgroup's run of each bucket starts in `pairs`, minus the group's start in `sorted`
    for (uint32_t b = threadIdx.x; b < nb; b += kBinThreads) cursor[b] = 0;
    // everything this workgroup reads from memory is requested here, before the first dependent step
    const uint32_t i0 = blockIdx.x * kBinChunk;
    int64_t jj[kBinPerThread];
    uint32_t sv[kBinPerThread], tot[PER], off[PER];
#pragma unroll
    for (int e = 0; e < kBinPerThread; e++) {
        const uint32_t i = i0 + e * kBinThreads + threadIdx.x;
        jj[e] = i < m ? __builtin_nontemporal_load(idx + i) : -1;
        sv[e] = i < m ? __builtin_nontemporal_load(src + i) : 0u;
    }
#pragma unroll
    for (int e = 0; e < PER; e++) {
        const uint32_t b = threadIdx.x * PER + e;
        tot[e] = b < nb ? totals[b] : 0u;
        off[e] = b < nb ? counts[(size_t)blockIdx.x * nb + b] : 0u;
    }
    __syncthreads();
    // group sizes (recounting is cheaper than keeping the histograms of pass 1)
#pragma unroll
    for (int e = 0; e < kBinPerThread; e++) {
        if (jj[e] >= n) jj[e] = -1;
        if (jj[e] >= 0) atomicAdd(&cursor[(uint32_t)(jj[e] >> kBinShift)], 1u);
    }
    __syncthreads();
    // group starts inside `sorted`, and each bucket's start in `pairs`
    {
        uint32_t v[PER], sum = 0, tsum = 0, total;
#pragma unroll
        for (int e = 0; e < PER; e++) {
            const uint32_t b = threadIdx.x * PER + e;
            v[e] = b < nb ? cursor[b] : 0u;
            sum += v[e];
            tsum += tot[e];
        }
        uint32_t run = bin_block_scan(sum, &total, wave_sum);
        uint32_t trun = bin_block_scan(tsum, &total, wave_sum);
#pragma unroll
        for (int e = 0; e < PER; e++) {
            const uint32_t b = threadIdx.x * PER + e;
            if (b < nb) {
                cursor[b] = run;
                gbase[b] = trun + off[e] - run;
            }
            run += v[e];
            trun += tot[e];
        }
    }
    __syncthreads();
#pragma unroll
    for (int e = 0; e < kBinPerThread; e++) {
        if (jj[e] >= 0) {
            const uint32_t slot = atomicAdd(&cursor[(uint32_t)(jj[e] >> kBinShift)], 1u);
            sorted[slot] = make_uint2((uint32_t)jj[e], sv[e]);   // table index < 2^32 here
        }
    }
    __syncthreads();
    const uint32_t valid = cursor[nb - 1];   // every group has moved up by its size: the last cursor is the number of valid pairs
    for (uint32_t sI = threadIdx.x; sI < valid; sI += kBinThreads) {
        const uint2 pr = sorted[sI];
        pairs[gbase[pr.x >> kBinShift] + sI] = pr;
    }
}

__global__ __launch_bounds__(kBinThreads) void bin_apply_kernel(uint32_t* __restrict__ t, int64_t n, uint32_t nb, const uint32_t* __restrict__ totals,
                                                                const uint2* __restrict__ pairs) {
    __shared__ uint32_t acc[kBinElems];
    __shared__ uint32_t wave_sum[kBinThreads / 64];
    const uint32_t b = blockIdx.x;
    const uint32_t cnt = totals[b];
    if (cnt == 0) return;               // uniform: nothing lands in this bucket
    // the bucket's slice of the table is fetched first (whole buckets: 4 vectors per thread), so that its latency is covered by
    // everything else the workgroup does
    const int64_t e0 = (int64_t)b << kBinShift;
    const uint32_t len = (uint32_t)((n - e0) < (int64_t)kBinElems ? (n - e0) : (int64_t)kBinElems);
    uint32_t* tp = t + e0;
    const bool whole = len == kBinElems && (((uintptr_t)tp) & 15) == 0;
    constexpr int NV = kBinElems / 4 / kBinThreads;
    Pack<uint32_t, 4> v[NV];
    if (whole) {
#pragma unroll
        for (int k = 0; k < NV; k++) v[k] = load_pack<uint32_t, 4>(tp + (k * kBinThreads + threadIdx.x) * 4u);
    }
    // where the bucket's pairs start: the sum of the totals before it
    uint32_t before = 0;
    for (uint32_t i = threadIdx.x; i < b; i += kBinThreads) before += totals[i];
    for (uint32_t i = threadIdx.x * 4u; i < kBinElems; i += kBinThreads * 4u) *reinterpret_cast<uint4*>(&acc[i]) = make_uint4(0, 0, 0, 0);
    uint32_t p0;
    (void)bin_block_scan(before, &p0, wave_sum);   // its barriers also publish the cleared accumulators
    constexpr int U = 4;   // loads in flight per thread
    for (uint32_t i0 = 0; i0 < cnt; i0 += kBinThreads * U) {
        uint2 pr[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint32_t i = i0 + u * kBinThreads + threadIdx.x;
            const Pack<uint32_t, 2> w = load_pack<uint32_t, 2>(reinterpret_cast<const uint32_t*>(pairs + p0 + (i < cnt ? i : 0u)));
            pr[u] = make_uint2(w.v[0], w.v[1]);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint32_t i = i0 + u * kBinThreads + threadIdx.x;
            if (i < cnt) atomicAdd(&acc[pr[u].x & (kBinElems - 1u)], pr[u].y);
        }
    }
    __syncthreads();
    if (whole) {
#pragma unroll
        for (int k = 0; k < NV; k++) {
            const uint32_t i = (k * kBinThreads + threadIdx.x) * 4u;
#pragma unroll
            for (int e = 0; e < 4; e++) v[k].v[e] += acc[i + e];
            store_pack<uint32_t, 4>(tp + i, v[k]);
        }
    } else {
        for (uint32_t i = threadIdx.x; i < len; i += kBinThreads) tp[i] += acc[i];
    }
}

// Workspace of the binned form for m updates into a table of n elements: the per-workgroup bucket counts, the bucket totals and
// the sorted pairs.
constexpr size_t kBinMaxWorkspace = (size_t)1 << 30;   // beyond this the direct kernel is taken (the stream keeps its workspace)
inline size_t binned_workspace_bytes(int64_t m, int64_t n, size_t* counts_bytes, size_t* totals_bytes) {
    const size_t nb = (size_t)((n + kBinElems - 1) >> kBinShift), nchunks = (size_t)((m + kBinChunk - 1) / kBinChunk);
    *counts_bytes = (nb * nchunks * 4 + 255) / 256 * 256;
    *totals_bytes = (nb * 4 + 255) / 256 * 256;
    return *counts_bytes + *totals_bytes + (size_t)m * 8;
}

// Whether m updates of 32-bit integers into a rank-1 table of n elements take the binned form: its workspace in bytes, or 0 for the
// direct kernel.  Cost model (measured on MI355X): a direct update costs about 40 ps (memory-side read-modify-write); the binned form
// moves the table twice, the pairs four and a half times and the per-workgroup bucket counts four times (written, scanned in place,
// read by the moving pass) at about 5.5 TB/s, plus three more launches.
inline size_t binned_choice(int64_t m, int64_t n, size_t* counts_bytes, size_t* totals_bytes) {
    if (m < (1 << 20) || m > 0x7FFFFFFFLL || n < 1 || n > ((int64_t)kBinMaxBuckets << kBinShift)) return 0;
    const size_t ws_bytes = binned_workspace_bytes(m, n, counts_bytes, totals_bytes);
    const double direct_us = (double)m * 40e-6, binned_us = ((double)n * 8.0 + (double)m * 36.0 + (double)*counts_bytes * 4.0) / 5.5e6 + 10.0;
    if (binned_us >= direct_us || ws_bytes > kBinMaxWorkspace) return 0;
    return ws_bytes;
}

// Takes the call when it has the binned form's shape and the binned form is the cheaper one; *status then holds its result.
bool try_scatter_binned(const DnhTensor* t, const DnhTensor* const* idx, int32_t n_idx, const DnhTensor* src, hipStream_t stream, int32_t* err,
                        int32_t* status) {
    if (t->dtype != DNH_I32 && t->dtype != DNH_U32) return false;
    if (t->ndims != 1 || src->ndims != 1 || n_idx != 1 || !idx[0] || idx[0]->ndims != 1) return false;
    if (t->stride[0] != 1 || src->stride[0] != 1 || idx[0]->stride[0] != 1) return false;
    const int64_t n = t->shape[0], m = src->shape[0];
    size_t counts_bytes, totals_bytes;
    const size_t ws_bytes = binned_choice(m, n, &counts_bytes, &totals_bytes);
    if (ws_bytes == 0) return false;
    const uint32_t nb = (uint32_t)((n + kBinElems - 1) >> kBinShift), nchunks = cdiv(m, kBinChunk);
    char* ws = nullptr;
    WorkspaceLease lease;
    if (workspace(stream, ws_bytes, (void**)&ws, lease) != DNH_OK) {
        last_error().clear();   // the direct kernel needs no memory: take that one
        return false;
    }
    uint32_t* counts = (uint32_t*)ws;
    uint32_t* totals = (uint32_t*)(ws + counts_bytes);
    uint2* pairs = (uint2*)(ws + counts_bytes + totals_bytes);
    const int64_t* ip = (const int64_t*)elem_ptr(idx[0]);
    hipLaunchKernelGGL(bin_count_kernel, dim3(nchunks), dim3(kBinThreads), nb * 4, stream, ip, (uint32_t)m, n, nb, nchunks, counts, err);
    hipLaunchKernelGGL(bin_colscan_kernel, dim3(cdiv(nb, 64)), dim3(kBinThreads), 0, stream, counts, totals, nb, nchunks);
    hipLaunchKernelGGL(bin_move_kernel, dim3(nchunks), dim3(kBinThreads), nb * 8, stream, ip, (const uint32_t*)elem_ptr(src), (uint32_t)m, n, nb, nchunks,
                       (const uint32_t*)counts, (const uint32_t*)totals, pairs);
    hipLaunchKernelGGL(bin_apply_kernel, dim3(nb), dim3(kBinThreads), 0, stream, (uint32_t*)elem_ptr(t), n, nb, (const uint32_t*)totals, (const uint2*)pairs);
    *status = hipGetLastError() == hipSuccess ? DNH_OK : fail(DNH_ERR_HIP, "binned scatter: launch failed");
    return true;
}

// ---- ordered scatter (floating point) ------------------------------------------------------------------------------------------
// t[idx[s]] += src[s] for single and double, any ranks and strides.  The reference adds the sources in row-major order
// (Host/ScalarOps.fs:593-604), so a target element that several sources name receives ((t + s_a) + s_b) + ... in source order, and
// floating-point addition does not commute with itself: atomics give another order on every run.  Here every target element receives
// its sources in the reference's order, hence the reference's bits, whatever the duplication:
//   1. ordered_cells:  cell[s] = row-major position in t that source s names (-1 and the error word when out of range)
//   2. ordered_count:  per workgroup of kOrdChunk sources, how many fall into each bucket of 2^shift consecutive cells   -> counts
//   3. bin_colscan, ordered_starts: where each workgroup's share of each bucket starts in the bucket's list             -> counts, starts
//   4. ordered_move:   each workgroup sorts its sources by cell in LDS (a stable radix sort: sources of one cell keep their order)
//                      and appends every bucket's run to that bucket's list: a list is ordered by workgroup, then by cell, then by
//                      source position
//   5. ordered_apply:  one workgroup per bucket keeps the bucket's cells in LDS and walks the list in batches of 1024 entries.
//                      Entries of one cell that are neighbours in a batch form a run, which the thread at its head adds in order;
//                      runs of one cell that are not neighbours (they come from different workgroups of pass 4) are applied in
//                      list order: each round the first pending run of a cell claims it (LDS atomic minimum of the position).
// A table of more than 4096 buckets is processed in slabs of 4096 x 2^shift cells (passes 2-5 per slab).
constexpr int kOrdThreads = 1024;
constexpr int kOrdLiBits = 13;
constexpr uint32_t kOrdChunk = 1u << kOrdLiBits;     // sources per workgroup of passes 2 and 4
constexpr int kOrdPer = kOrdChunk / kOrdThreads;
constexpr int kOrdMaxShift = 13;                     // at most 8192 cells of a bucket in LDS
constexpr uint32_t kOrdMaxBuckets = 4096;
constexpr uint32_t kOrdNone = 0xFFFFFFFFu;

__global__ __launch_bounds__(kBlock) void ordered_cells_kernel(IndexArgs a, uint32_t m, int64_t* __restrict__ cell, int32_t* err) {
    const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= m) return;
    uint32_t pos[DNH_MAX_DIMS];
    (void)unravel(a.iter, i, pos);
    int64_t c = 0;
    bool ok = true;
    for (int d = 0; d < a.other.nd; d++) {
        int64_t j;
        if (a.idx[d]) {
            int64_t io = 0;
            for (int e = 0; e < a.iter.nd; e++) io += (int64_t)pos[e] * a.idx_stride[d][e];
            j = a.idx[d][io];
        } else {
            j = pos[d];
        }
        ok = ok && j >= 0 && j < a.other_shape[d];
        c = c * a.other_shape[d] + j;
    }
    if (!ok) *err = 1;
    cell[i] = ok ? c : -1;
}

__global__ __launch_bounds__(kOrdThreads) void ordered_count_kernel(const int64_t* __restrict__ cell, uint32_t m, int64_t lo, int64_t hi, int shift,
                                                                    uint32_t nb, uint32_t* __restrict__ counts) {
    extern __shared__ uint32_t ord_hist[];   // nb counters
    for (uint32_t b = threadIdx.x; b < nb; b += kOrdThreads) ord_hist[b] = 0;
    const uint32_t i0 = blockIdx.x * kOrdChunk;
    int64_t c[kOrdPer];
#pragma unroll
    for (int e = 0; e < kOrdPer; e++) {
        const uint32_t i = i0 + e * kOrdThreads + threadIdx.x;
        c[e] = i < m ? cell[i] : -1;
    }
    __syncthreads();
#pragma unroll
    for (int e = 0; e < kOrdPer; e++)
        if (c[e] >= lo && c[e] < hi) atomicAdd(&ord_hist[(uint32_t)((c[e] - lo) >> shift)], 1u);
    __syncthreads();
    for (uint32_t b = threadIdx.x; b < nb; b += kOrdThreads) counts[(size_t)blockIdx.x * nb + b] = ord_hist[b];
}

// starts[b] = totals[0] + .. + totals[b - 1], one workgroup
__global__ __launch_bounds__(kOrdThreads) void ordered_starts_kernel(const uint32_t* __restrict__ totals, uint32_t* __restrict__ starts, uint32_t nb) {
    constexpr int PER = kOrdMaxBuckets / kOrdThreads;
    __shared__ uint32_t wave_sum[kOrdThreads / 64];
    uint32_t v[PER], sum = 0, total;
#pragma unroll
    for (int e = 0; e < PER; e++) {
        const uint32_t b = threadIdx.x * PER + e;
        v[e] = b < nb ? totals[b] : 0u;
        sum += v[e];
    }
    uint32_t run = bin_block_scan(sum, &total, wave_sum);
#pragma unroll
    for (int e = 0; e < PER; e++) {
        const uint32_t b = threadIdx.x * PER + e;
        if (b < nb) starts[b] = run;
        run += v[e];
    }
}

// Pass 4.  The chunk's sources are sorted by cell with a least-significant-digit radix sort in LDS (digits of kOrdDigitBits bits,
// every pass stable, so sources of one cell stay in source order).  A thread keeps its kOrdPer keys in registers; key e of thread t
// stands at position e * 1024 + t, so a wavefront holds 64 consecutive positions ("a row") per e.  Per pass: the lanes of a row that
// share a digit find each other with one ballot per digit bit, which gives each its rank among them and, to the first of them, their
// number for the counter of (digit, row); an exclusive scan over the counters in (digit, row) order is every group's start; the keys
// go to LDS at start + rank and come back by position.  Sources outside the slab carry one cell number beyond its last cell, so
// they end up behind everything that is moved.
constexpr int kOrdDigitBits = 5, kOrdDigits = 1 << kOrdDigitBits, kOrdRows = kOrdChunk / 64;
template <class X>
__global__ __launch_bounds__(kOrdThreads) void ordered_move_kernel(const int64_t* __restrict__ cell, const X* __restrict__ src, Lay slay, uint32_t m,
                                                                   int64_t lo, int64_t hi, int shift, uint32_t nb, int npass,
                                                                   const uint32_t* __restrict__ counts, const uint32_t* __restrict__ starts,
                                                                   uint32_t* __restrict__ pc, X* __restrict__ pv) {
    extern __shared__ __align__(16) unsigned char ord_lds[];
    uint64_t* keys = reinterpret_cast<uint64_t*>(ord_lds);            // by position: (cell - lo) << 13 | position the source had in the chunk
    X* vals = reinterpret_cast<X*>(keys + kOrdChunk);                  // by position the source had in the chunk
    uint32_t* cnt = reinterpret_cast<uint32_t*>(vals + kOrdChunk);     // kOrdDigits x kOrdRows counters; afterwards: where each bucket's run starts
    uint32_t* gstart = cnt;
    __shared__ uint32_t wave_sum[kOrdThreads / 64];
    const uint32_t i0 = blockIdx.x * kOrdChunk, lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint64_t outside = (uint64_t)(hi - lo);
    uint64_t key[kOrdPer];
#pragma unroll
    for (int e = 0; e < kOrdPer; e++) {
        const uint32_t li = e * kOrdThreads + threadIdx.x, i = i0 + li;
        const int64_t c = i < m ? cell[i] : -1;
        key[e] = (((c >= lo && c < hi) ? (uint64_t)(c - lo) : outside) << kOrdLiBits) | li;
        vals[li] = i < m ? src[offset_of(slay, i)] : X(0);
    }
    constexpr int CPT = kOrdDigits * kOrdRows / kOrdThreads;   // counters per thread in the scan
    for (int pass = 0; pass < npass; pass++) {
        const int sh = kOrdLiBits + pass * kOrdDigitBits;
#pragma unroll
        for (int q = 0; q < CPT; q++) cnt[threadIdx.x * CPT + q] = 0;
        __syncthreads();   // counters cleared (and the previous pass's keys read back)
        uint32_t rank[kOrdPer], slot[kOrdPer];
#pragma unroll
        for (int e = 0; e < kOrdPer; e++) {
            const uint32_t d = (uint32_t)(key[e] >> sh) & (kOrdDigits - 1);
            unsigned long long peers = ~0ull;
#pragma unroll
            for (int bit = 0; bit < kOrdDigitBits; bit++) {
                const bool set = (d >> bit) & 1u;
                const unsigned long long with = __ballot(set);
                peers &= set ? with : ~with;
            }
            rank[e] = (uint32_t)__popcll(peers & ((1ull << lane) - 1ull));
            slot[e] = d * kOrdRows + (uint32_t)e * (kOrdThreads / 64) + wave;
            if (rank[e] == 0) cnt[slot[e]] = (uint32_t)__popcll(peers);
        }
        __syncthreads();
        {
            uint32_t v[CPT], sum = 0, total;
#pragma unroll
            for (int q = 0; q < CPT; q++) {
                v[q] = cnt[threadIdx.x * CPT + q];
                sum += v[q];
            }
            uint32_t run = bin_block_scan(sum, &total, wave_sum);   // (two barriers inside)
#pragma unroll
            for (int q = 0; q < CPT; q++) {
                cnt[threadIdx.x * CPT + q] = run;
                run += v[q];
            }
        }
        __syncthreads();
#pragma unroll
        for (int e = 0; e < kOrdPer; e++) keys[cnt[slot[e]] + rank[e]] = key[e];
        __syncthreads();
#pragma unroll
        for (int e = 0; e < kOrdPer; e++) key[e] = keys[e * kOrdThreads + threadIdx.x];
    }
    if (npass == 0) {
#pragma unroll
        for (int e = 0; e < kOrdPer; e++) keys[e * kOrdThreads + threadIdx.x] = key[e];
    }
    __syncthreads();   // keys[] holds the sorted keys; cnt is free for the buckets' starts
#pragma unroll
    for (int e = 0; e < kOrdPer; e++) {
        const uint32_t k = e * kOrdThreads + threadIdx.x;
        const uint64_t cl = key[e] >> kOrdLiBits;
        if (cl < outside) {
            const uint32_t b = (uint32_t)(cl >> shift);
            if (k == 0 || (uint32_t)((keys[k - 1] >> kOrdLiBits) >> shift) != b) gstart[b] = k;
        }
    }
    __syncthreads();
#pragma unroll
    for (int e = 0; e < kOrdPer; e++) {
        const uint32_t k = e * kOrdThreads + threadIdx.x;
        const uint64_t cl = key[e] >> kOrdLiBits;
        if (cl < outside) {
            const uint32_t b = (uint32_t)(cl >> shift);
            const uint32_t dst = starts[b] + counts[(size_t)blockIdx.x * nb + b] + (k - gstart[b]);
            pc[dst] = (uint32_t)(cl & ((1u << shift) - 1u));
            pv[dst] = vals[(uint32_t)key[e] & (kOrdChunk - 1u)];
        }
    }
}

// element offset of row-major position i of a layout (positions beyond 2^32 included)
__device__ __forceinline__ int64_t offset_of64(const Lay& l, int64_t i) {
    int64_t off = 0;
    for (int d = l.nd - 1; d >= 0; d--) {
        const int64_t q = (d == 0) ? 0 : i / (int64_t)l.shape[d];
        off += (i - q * (int64_t)l.shape[d]) * l.stride[d];
        i = q;
    }
    return off;
}

template <class X>
__global__ __launch_bounds__(kOrdThreads) void ordered_apply_kernel(X* __restrict__ t, Lay tlay, int dense, int64_t lo, int64_t ncells, int shift,
                                                                    const uint32_t* __restrict__ totals, const uint32_t* __restrict__ starts,
                                                                    const uint32_t* __restrict__ pc, const X* __restrict__ pv) {
    extern __shared__ __align__(16) unsigned char ord_lds[];
    const uint32_t cells = 1u << shift;
    X* acc = reinterpret_cast<X*>(ord_lds);                                      // the bucket's cells
    X* bv = acc + cells;                                                         // the batch: values
    uint32_t* claim = reinterpret_cast<uint32_t*>(bv + kOrdThreads);             // per cell: position in the batch of the first pending run, or kOrdNone
    uint32_t* bc = claim + cells;                                                // the batch: cells (inside the bucket)
    const uint32_t b = blockIdx.x;
    const uint32_t cnt = totals[b];
    if (cnt == 0) return;   // uniform: nothing lands in this bucket
    const int64_t c0 = lo + ((int64_t)b << shift);
    const uint32_t len = (uint32_t)((ncells - c0) < (int64_t)cells ? (ncells - c0) : (int64_t)cells);
    for (uint32_t x = threadIdx.x; x < len; x += kOrdThreads) {
        acc[x] = t[dense ? c0 + x : offset_of64(tlay, c0 + x)];
        claim[x] = kOrdNone;
    }
    const uint32_t p0 = starts[b];
    for (uint32_t base = 0; base < cnt; base += kOrdThreads) {
        const uint32_t nbat = cnt - base < (uint32_t)kOrdThreads ? cnt - base : (uint32_t)kOrdThreads;
        uint32_t c = 0;
        if (threadIdx.x < nbat) {
            c = pc[p0 + base + threadIdx.x];
            bc[threadIdx.x] = c;
            bv[threadIdx.x] = pv[p0 + base + threadIdx.x];
        }
        __syncthreads();   // the batch (and, the first time, the cells) are in LDS
        bool pending = threadIdx.x < nbat && (threadIdx.x == 0 || bc[threadIdx.x - 1] != c);   // head of a run
        for (;;) {
            if (pending) atomicMin(&claim[c], threadIdx.x);
            __syncthreads();
            if (pending && claim[c] == threadIdx.x) {
                // the run is added in order, entry by entry (a cell that receives L sources is a chain of L dependent additions; fetching
                // the entries of long runs ahead of the additions measured 3x faster for a single cell that takes everything, and
                // 15-50 % slower for everything else: the fetched entries' registers cost the common, short runs more than they save)
                X a = acc[c];
                for (uint32_t k = threadIdx.x; k < nbat && bc[k] == c; k++) a = a + bv[k];
                acc[c] = a;
                claim[c] = kOrdNone;
                pending = false;
            }
            if (!__syncthreads_or((int)pending)) break;
        }
    }
    __syncthreads();
    for (uint32_t x = threadIdx.x; x < len; x += kOrdThreads) t[dense ? c0 + x : offset_of64(tlay, c0 + x)] = acc[x];
}

// Workspace of the ordered scatter of m sources into ncells cells with buckets of 2^shift cells.
struct OrderedPlan {
    int shift;
    uint32_t nb_max, nchunks;
    size_t cell_bytes, counts_bytes, totals_bytes, pc_bytes, pv_bytes, total;
};
inline OrderedPlan ordered_plan(int64_t m, int64_t ncells, int esize) {
    OrderedPlan p;
    int lg = 0;
    while (((int64_t)1 << lg) < ncells) lg++;
    p.shift = lg - 10 < 4 ? 4 : (lg - 10 > kOrdMaxShift ? kOrdMaxShift : lg - 10);   // about a thousand buckets where the table allows
    const int64_t buckets = (ncells + ((int64_t)1 << p.shift) - 1) >> p.shift;
    p.nb_max = (uint32_t)(buckets < (int64_t)kOrdMaxBuckets ? buckets : (int64_t)kOrdMaxBuckets);
    p.nchunks = (uint32_t)((m + kOrdChunk - 1) / kOrdChunk);
    auto up = [](size_t b) { return (b + 255) / 256 * 256; };
    p.cell_bytes = up((size_t)m * 8);
    p.counts_bytes = up((size_t)p.nb_max * p.nchunks * 4);
    p.totals_bytes = up((size_t)p.nb_max * 4);
    p.pc_bytes = up((size_t)m * 4);
    p.pv_bytes = up((size_t)m * (size_t)esize);
    p.total = p.cell_bytes + p.counts_bytes + 2 * p.totals_bytes + p.pc_bytes + p.pv_bytes;
    return p;
}

template <class X>
int32_t scatter_ordered(const DnhTensor* t, const DnhTensor* src, const IndexArgs& a, hipStream_t stream, int32_t* err) {
    const int64_t m = nelems(src), ncells = nelems(t);
    const OrderedPlan p = ordered_plan(m, ncells, (int)sizeof(X));
    char* ws = nullptr;
    WorkspaceLease lease;
    const int32_t st = workspace(stream, p.total, (void**)&ws, lease);
    if (st != DNH_OK)
        return fail(st, "dnh_scatter: no memory for the %zu-byte workspace of the ordered floating-point scatter (dnh_set_option(\"scatter_fp_atomic\", 1) "
                        "selects the atomic form, which needs none)", p.total);
    int64_t* cell = (int64_t*)ws;
    uint32_t* counts = (uint32_t*)(ws + p.cell_bytes);
    uint32_t* totals = (uint32_t*)(ws + p.cell_bytes + p.counts_bytes);
    uint32_t* starts = (uint32_t*)(ws + p.cell_bytes + p.counts_bytes + p.totals_bytes);
    uint32_t* pc = (uint32_t*)(ws + p.cell_bytes + p.counts_bytes + 2 * p.totals_bytes);
    X* pv = (X*)(ws + p.cell_bytes + p.counts_bytes + 2 * p.totals_bytes + p.pc_bytes);
    static_assert(kOrdDigits * kOrdRows <= (int)kOrdMaxBuckets, "the radix counters share the bucket starts' array");
    const size_t move_lds = (size_t)kOrdChunk * (8 + sizeof(X)) + (size_t)kOrdMaxBuckets * 4;   // keys, values, then the counters / bucket starts
    const size_t apply_lds = ((size_t)1 << p.shift) * (sizeof(X) + 4) + (size_t)kOrdThreads * (sizeof(X) + 4);
    static const hipError_t attr_move = hipFuncSetAttribute(reinterpret_cast<const void*>(&ordered_move_kernel<X>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                                            (int)move_lds);
    static const hipError_t attr_apply = hipFuncSetAttribute(reinterpret_cast<const void*>(&ordered_apply_kernel<X>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                                             (int)(((size_t)1 << kOrdMaxShift) * (sizeof(X) + 4) + (size_t)kOrdThreads * (sizeof(X) + 4)));
    if (attr_move != hipSuccess || attr_apply != hipSuccess) return fail(DNH_ERR_HIP, "dnh_scatter: cannot size the LDS of the ordered scatter");
    // the target's cells in row-major order lie one after the other in memory?
    int dense = 1;
    {
        int64_t expect = 1;
        for (int d = t->ndims - 1; d >= 0; d--) {
            if (t->shape[d] != 1 && t->stride[d] != expect) dense = 0;
            expect *= t->shape[d];
        }
    }
    const Lay slay = lay_of(src), tlay = lay_of(t);
    X* tp = (X*)elem_ptr(t);
    hipLaunchKernelGGL(ordered_cells_kernel, dim3(cdiv(m, kBlock)), dim3(kBlock), 0, stream, a, (uint32_t)m, cell, err);
    DNH_LAUNCH_CHECK();
    const int64_t slab = (int64_t)kOrdMaxBuckets << p.shift;
    for (int64_t lo = 0; lo < ncells; lo += slab) {
        const int64_t hi = lo + slab < ncells ? lo + slab : ncells;
        const uint32_t nb = (uint32_t)((hi - lo + ((int64_t)1 << p.shift) - 1) >> p.shift);
        hipLaunchKernelGGL(ordered_count_kernel, dim3(p.nchunks), dim3(kOrdThreads), nb * 4, stream, (const int64_t*)cell, (uint32_t)m, lo, hi, p.shift, nb, counts);
        hipLaunchKernelGGL(bin_colscan_kernel, dim3(cdiv(nb, 64)), dim3(kBinThreads), 0, stream, counts, totals, nb, p.nchunks);
        hipLaunchKernelGGL(ordered_starts_kernel, dim3(1), dim3(kOrdThreads), 0, stream, (const uint32_t*)totals, starts, nb);
        int bits = 0;   // of the largest cell number inside the slab, hi - lo, which stands for "outside"
        while (((int64_t)1 << bits) <= hi - lo) bits++;
        const int npass = (bits + kOrdDigitBits - 1) / kOrdDigitBits;
        hipLaunchKernelGGL((ordered_move_kernel<X>), dim3(p.nchunks), dim3(kOrdThreads), move_lds, stream, (const int64_t*)cell, (const X*)elem_ptr(src), slay,
                           (uint32_t)m, lo, hi, p.shift, nb, npass, (const uint32_t*)counts, (const uint32_t*)starts, pc, pv);
        hipLaunchKernelGGL((ordered_apply_kernel<X>), dim3(nb), dim3(kOrdThreads), apply_lds, stream, tp, tlay, dense, lo, ncells, p.shift,
                           (const uint32_t*)totals, (const uint32_t*)starts, (const uint32_t*)pc, (const X*)pv);
        DNH_LAUNCH_CHECK();
    }
    return DNH_OK;
}

__global__ __launch_bounds__(kBlock) void compact_count_kernel(MaskArgs m, uint32_t n, uint32_t* counts) {
    const uint32_t i0 = blockIdx.x * (uint32_t)kChunk + threadIdx.x * kItems;
    uint32_t c = 0;
    if (i0 < n) {
        if (m.full.nd == 1 && !m.whole && m.mask[0] && m.mask_stride[0] == 1 && i0 + kItems <= n && (((uintptr_t)(m.mask[0] + i0)) & 15) == 0) {
            const Pack<uint8_t, kItems> v = load_pack<uint8_t, kItems>(m.mask[0] + i0);
#pragma unroll
            for (int e = 0; e < kItems; e++) c += v.v[e] != 0;
        } else {
            for (int e = 0; e < kItems && i0 + e < n; e++) {
                uint32_t pos[DNH_MAX_DIMS];
                const int64_t off = unravel(m.full, i0 + e, pos);
                c += selected(m, pos, off);
            }
        }
    }
    uint32_t total;
    block_exclusive_scan(c, &total);
    if (threadIdx.x == 0) counts[blockIdx.x] = total;
}

// in-place exclusive scan of counts[0..nb) by one block
__global__ __launch_bounds__(kBlock) void compact_scan_kernel(uint32_t* counts, uint32_t nb) {
    const uint32_t seg = (nb + kBlock - 1) / kBlock;
    const uint32_t b0 = threadIdx.x * seg;
    uint32_t sum = 0;
    for (uint32_t i = b0; i < b0 + seg && i < nb; i++) sum += counts[i];
    uint32_t total;
    uint32_t run = block_exclusive_scan(sum, &total);
    for (uint32_t i = b0; i < b0 + seg && i < nb; i++) {
        const uint32_t c = counts[i];
        counts[i] = run;
        run += c;
    }
}

enum CompactMode { kMaskedGet = 0, kMaskedSet = 1, kTrueIndices = 2 };

// MODE kMaskedGet : out[k]        = full[i]      for the k-th selected element i
//      kMaskedSet : full[i]       = out[k]       (`out` is the value tensor)
//      kTrueIndices: out[k, 0..nd) = position of i
template <class W, int MODE>
__global__ __launch_bounds__(kBlock) void compact_move_kernel(MaskArgs m, W* full, W* out, Lay olay, uint32_t n, uint32_t nout,
                                                              const uint32_t* block_base) {
    const uint32_t i0 = blockIdx.x * (uint32_t)kChunk + threadIdx.x * kItems;
    uint32_t flags = 0, c = 0;
    if (i0 < n) {
        if (m.full.nd == 1 && !m.whole && m.mask[0] && m.mask_stride[0] == 1 && i0 + kItems <= n && (((uintptr_t)(m.mask[0] + i0)) & 15) == 0) {
            const Pack<uint8_t, kItems> v = load_pack<uint8_t, kItems>(m.mask[0] + i0);
#pragma unroll
            for (int e = 0; e < kItems; e++) flags |= (uint32_t)(v.v[e] != 0) << e;
        } else {
            for (int e = 0; e < kItems && i0 + e < n; e++) {
                uint32_t pos[DNH_MAX_DIMS];
                const int64_t off = unravel(m.full, i0 + e, pos);
                flags |= (uint32_t)selected(m, pos, off) << e;
            }
        }
        c = __popc(flags);
    }
    uint32_t total;
    uint32_t k = block_base[blockIdx.x] + block_exclusive_scan(c, &total);
    while (flags) {
        const int e = __ffs(flags) - 1;
        flags &= flags - 1;
        if (k < nout) {
            uint32_t pos[DNH_MAX_DIMS];
            const int64_t foff = unravel(m.full, i0 + e, pos);
            if constexpr (MODE == kMaskedGet) out[offset_of(olay, k)] = full[foff];
            else if constexpr (MODE == kMaskedSet) full[foff] = out[offset_of(olay, k)];
            else {
                for (int d = 0; d < m.full.nd; d++) out[(int64_t)k * olay.stride[0] + (int64_t)d * olay.stride[1]] = (W)pos[d];
            }
        }
        k++;
    }
}

// ---- tiles of one launch that meet through memory ------------------------------------------------------------------------------
// One-pass compaction: every workgroup ("tile") needs the number of selected elements before its region.  Instead of a counting
// launch in front, a tile publishes the count of its own region in a word of device memory and adds up the words of the tiles
// before it, walking back 64 at a time until it meets a tile that already knows the count of everything up to itself, which it then
// publishes for its own position in turn.  A tile is a workgroup and its number the workgroup's: the hardware starts workgroups in
// ascending order, so the tiles a workgroup waits for are normally running or done, but nothing depends on that: the wait is bounded.
// After `spins` polls the tile counts the mask in front of its region itself, so every workgroup finishes whatever the others do.
// (Tile numbers drawn as tickets from one counter, which would make the starting order certain, cost 11 ns each, one after the
// other: 46 us for the 4096 tiles of a 16 Mi-element maskedGet.)
// Measured on MI355X, 16 Mi int32 with half the elements selected: maskedGet 41.8 us in one pass against 26.6 us with a counting
// launch in front, maskedSet 53.1 against 39.4, trueIndices 25.8 against 24.7.  A published word crosses XCDs through memory, about
// 2 us per hop; the tiles resident together (2048) publish at the same moment and then need about eight hops before the last of
// them knows its count, and nothing is written meanwhile.  The counting launch costs 5 us.  The one-pass form is therefore not the
// default (option compact_one_pass).
// A word: [63:34] the launch's epoch (words of earlier launches read as "not published"), [33:32] 1 = count of the tile's own region,
// 2 = count of everything up to and including the tile, [31:0] the count.  Words are read and written with device-scope atomics (one
// word carries flag and value, so no ordering between separate locations is relied on).
struct TileSync {
    unsigned long long* desc;
    uint32_t epoch;
    uint32_t spins;
};
constexpr unsigned long long kTileOwn = 1ull << 32, kTileUpTo = 2ull << 32;

__device__ __forceinline__ unsigned long long tile_word(uint32_t epoch, unsigned long long status, uint32_t value) {
    return ((unsigned long long)epoch << 34) | status | value;
}
__device__ __forceinline__ void tile_publish(const TileSync& ts, uint32_t tile, unsigned long long status, uint32_t value) {
    __hip_atomic_store(ts.desc + tile, tile_word(ts.epoch, status, value), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Count of everything before `tile`, by the workgroup's first wavefront (threads 0..63 call; every one of them gets the result).
// *gave_up: a tile in front had not published after ts.spins polls; the tile's own count is published, the caller counts the rest.
__device__ __forceinline__ uint32_t look_back(const TileSync& ts, uint32_t tile, uint32_t own, bool* gave_up) {
    const uint32_t lane = threadIdx.x;
    *gave_up = false;
    if (tile == 0) {
        if (lane == 0) tile_publish(ts, 0, kTileUpTo, own);
        return 0;
    }
    if (lane == 0) tile_publish(ts, tile, kTileOwn, own);
    uint32_t excl = 0;
    int64_t pos = (int64_t)tile - 1;
    for (;;) {
        const int64_t j = pos - (int64_t)lane;   // lane 0 looks at the nearest tile
        unsigned long long w;
        int first_upto;
        for (uint32_t polls = 0;; polls++) {
            w = j >= 0 ? __hip_atomic_load(ts.desc + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : tile_word(ts.epoch, kTileUpTo, 0u);
            const bool ready = (uint32_t)(w >> 34) == ts.epoch && (w & (kTileOwn | kTileUpTo)) != 0;
            const unsigned long long ready_mask = __ballot(ready), upto_mask = __ballot(ready && (w & kTileUpTo) != 0);
            first_upto = upto_mask ? __ffsll((long long)upto_mask) - 1 : 64;
            const unsigned long long need = first_upto >= 63 ? ~0ull : ((2ull << first_upto) - 1ull);   // lanes 0 .. first_upto
            if ((ready_mask & need) == need) break;
            if (polls >= ts.spins) {
                *gave_up = true;
                return 0;
            }
            __builtin_amdgcn_s_sleep(2);
        }
        uint32_t c = (int)lane <= first_upto ? (uint32_t)w : 0u;
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) c += (uint32_t)__shfl_xor((int)c, m, 64);
        excl += c;
        if (first_upto < 64) break;
        pos -= 64;
    }
    if (lane == 0) tile_publish(ts, tile, kTileUpTo, excl + own);
    return excl;
}

// number of nonzero bytes in mask[0, nbytes), counted by the whole workgroup (nbytes a multiple of 16, mask 4-byte aligned)
__device__ __forceinline__ uint32_t block_count_mask(const uint8_t* mask, uint64_t nbytes) {
    __shared__ uint32_t part[kBlock / 64];
    uint32_t c = 0;
    for (uint64_t i = (uint64_t)threadIdx.x * 16; i < nbytes; i += (uint64_t)kBlock * 16) {
        const Pack<uint32_t, 4> v = load_pack<uint32_t, 4>((const uint32_t*)(mask + i));
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const uint32_t x = v.v[w];
            c += ((x & 0xFFu) != 0) + ((x & 0xFF00u) != 0) + ((x & 0xFF0000u) != 0) + ((x & 0xFF000000u) != 0);
        }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) c += (uint32_t)__shfl_xor((int)c, m, 64);
    __syncthreads();   // an earlier use of `part` is over
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = c;
    __syncthreads();
    uint32_t tot = 0;
#pragma unroll
    for (int w = 0; w < kBlock / 64; w++) tot += part[w];
    return tot;
}

// Count of everything before this workgroup's tile, for all of its threads.  region_bytes: mask bytes per tile.
__device__ __forceinline__ uint32_t tile_exclusive(const TileSync& ts, uint32_t tile, uint32_t own, const uint8_t* mask, uint32_t region_bytes) {
    __shared__ uint32_t excl_sh;
    __shared__ int gave_sh;
    if (threadIdx.x < 64) {
        bool g;
        const uint32_t e = look_back(ts, tile, own, &g);
        if (threadIdx.x == 0) {
            excl_sh = e;
            gave_sh = g;
        }
    }
    __syncthreads();
    if (gave_sh) {   // the same in every thread
        const uint32_t e = block_count_mask(mask, (uint64_t)tile * region_bytes);
        if (threadIdx.x == 0) tile_publish(ts, tile, kTileUpTo, e + own);
        return e;
    }
    return excl_sh;
}

// ---- contiguous 1-d fast path ------------------------------------------------------------------------------------------------
// Rank-1 unit-stride data and mask (the `a.M(mask)` form after the frontend's reshape/flatten, Tensor.fs:3044-3052): a block
// covers kFastJ * 256 vectors of VEC elements; thread t owns vector t of each of the kFastJ segments, so mask bytes and data
// are read with fully coalesced vector loads and no index arithmetic.  Ranks follow the element order (segment, thread,
// element): the per-segment counts of a thread are packed into one 64-bit word (16 bits each) and scanned together.
constexpr int kFastJ = 4;

template <int VEC>
__device__ __forceinline__ uint32_t flags_of(const Pack<uint8_t, VEC>& v) {
    uint32_t f = 0;
#pragma unroll
    for (int e = 0; e < VEC; e++) f |= (uint32_t)(v.v[e] != 0) << e;
    return f;
}
template <int VEC>
__device__ __forceinline__ uint32_t mask_flags(const uint8_t* m) {
    return flags_of<VEC>(load_pack<uint8_t, VEC>(m));
}

__device__ __forceinline__ uint64_t block_exclusive_scan64(uint64_t c, uint64_t* total) {
    __shared__ uint64_t wave_sum[kBlock / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint64_t inc = c;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t lo = (uint32_t)__shfl_up((int)(uint32_t)inc, d, 64);
        const uint32_t hi = (uint32_t)__shfl_up((int)(uint32_t)(inc >> 32), d, 64);
        if (lane >= d) inc += ((uint64_t)hi << 32) | lo;
    }
    if (lane == 63) wave_sum[wave] = inc;
    __syncthreads();
    uint64_t base = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < kBlock / 64; w++) {
        if (w < wave) base += wave_sum[w];
        tot += wave_sum[w];
    }
    *total = tot;
    return base + inc - c;
}

// Counts the selected elements of each block's region (kFastJ * 256 * VEC consecutive mask bytes).  Counting is order-free,
// so the region is read with 16-byte loads regardless of how the move pass assigns elements to threads.
template <int VEC>
__global__ __launch_bounds__(kBlock) void compact_count_fast_kernel(const uint8_t* mask, uint32_t nvec, uint32_t* counts) {
    constexpr uint32_t REGION = kFastJ * kBlock * VEC;                 // mask bytes per block
    const uint64_t n = (uint64_t)nvec * VEC;
    const uint64_t r0 = (uint64_t)blockIdx.x * REGION;
    const uint64_t r1 = r0 + REGION < n ? r0 + REGION : n;
    uint32_t c = 0;
    for (uint64_t i = r0 + (uint64_t)threadIdx.x * 16; i < r1; i += (uint64_t)kBlock * 16) {
        if (i + 16 <= r1) {
            const Pack<uint32_t, 4> v = load_pack<uint32_t, 4>((const uint32_t*)(mask + i));
#pragma unroll
            for (int w = 0; w < 4; w++) {
                // bytes are 0/1 booleans in the common case, but any nonzero byte counts as true
                const uint32_t x = v.v[w];
                c += ((x & 0xFFu) != 0) + ((x & 0xFF00u) != 0) + ((x & 0xFF0000u) != 0) + ((x & 0xFF000000u) != 0);
            }
        } else {
            for (uint64_t j = i; j < r1; j++) c += mask[j] != 0;
        }
    }
    uint32_t total;
    block_exclusive_scan(c, &total);
    if (threadIdx.x == 0) counts[blockIdx.x] = total;
}

// SET = false: out[k] = full[i] (MaskedGet);  SET = true: full[i] = out[k] (MaskedSet)
// Sum of counts[0..n): the exclusive prefix a block needs, computed by the block itself from the (L2-resident) per-block
// counts so that no separate scan launch sits between the count and move passes.
__device__ __forceinline__ uint32_t block_sum_before(const uint32_t* counts, uint32_t n) {
    __shared__ uint32_t part[kBlock / 64];
    uint32_t s = 0;
    // eight loads in flight per thread (one after the other they cost a trip to L2 each: up to 32 in a row for 8192 blocks)
    constexpr uint32_t U = 8;
    uint32_t i = threadIdx.x;
    for (; i + (U - 1) * kBlock < n; i += U * kBlock) {
        uint32_t v[U];
#pragma unroll
        for (uint32_t u = 0; u < U; u++) v[u] = counts[i + u * kBlock];
#pragma unroll
        for (uint32_t u = 0; u < U; u++) s += v[u];
    }
    {
        uint32_t v[U];   // the rest: clamped loads, masked sums (no branch between the loads)
#pragma unroll
        for (uint32_t u = 0; u < U; u++) v[u] = counts[i + u * kBlock < n ? i + u * kBlock : 0];
#pragma unroll
        for (uint32_t u = 0; u < U; u++) s += i + u * kBlock < n ? v[u] : 0u;
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) s += (uint32_t)__shfl_xor((int)s, m, 64);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
    __syncthreads();
    uint32_t tot = 0;
#pragma unroll
    for (int w = 0; w < kBlock / 64; w++) tot += part[w];
    return tot;
}

// Where a workgroup of the moving kernels learns how many selected elements lie before its region.
enum BaseMode {
    kBaseSumCounts = 0,   // it sums the counts of the workgroups before it (block_base = the counting pass's per-workgroup counts)
    kBasePrefixed = 1,    // block_base holds the scanned counts
    kBaseLookBack = 2     // one pass: the workgroups meet through `ts`
};

template <class W, bool SET, int BASE>
__global__ __launch_bounds__(kBlock) void compact_move_fast_kernel(const uint8_t* mask, W* full, W* out, uint32_t nvec, uint32_t nout,
                                                                   const uint32_t* block_base, TileSync ts) {
    constexpr int VEC = 16 / (int)sizeof(W);
    uint32_t flags[kFastJ];
    Pack<W, VEC> data[kFastJ];
    uint64_t packed = 0;
    uint32_t seg_base = 0;
    const uint32_t blk = blockIdx.x;
    {
        // every load of the thread is issued before the first one is used, without a branch in between (a vector beyond the end reads
        // vector 0 and counts nothing): with `if (v < nvec) { load; use }` per segment each segment waited for its own mask bytes
        // before the next segment's loads went out
        Pack<uint8_t, VEC> mk[kFastJ];
#pragma unroll
        for (int j = 0; j < kFastJ; j++) {
            const uint32_t v = (blk * kFastJ + j) * kBlock + threadIdx.x;
            const size_t vc = v < nvec ? (size_t)v : 0;
            mk[j] = load_pack<uint8_t, VEC>(mask + vc * VEC);
            if constexpr (!SET || sizeof(W) >= 4) data[j] = load_pack<W, VEC>(full + vc * VEC);
        }
        // (the counts of the blocks before this one are fetched while the loads above are on their way)
        if constexpr (BASE == kBasePrefixed) seg_base = block_base[blk];
        else if constexpr (BASE == kBaseSumCounts) seg_base = block_sum_before(block_base, blk);
#pragma unroll
        for (int j = 0; j < kFastJ; j++) {
            const uint32_t v = (blk * kFastJ + j) * kBlock + threadIdx.x;
            flags[j] = v < nvec ? flags_of<VEC>(mk[j]) : 0u;
            packed |= (uint64_t)__popc(flags[j]) << (16 * j);
        }
    }
    uint64_t total;
    const uint64_t pre = block_exclusive_scan64(packed, &total);
    if constexpr (BASE == kBaseLookBack) {
        uint32_t own = 0;
#pragma unroll
        for (int j = 0; j < kFastJ; j++) own += (uint32_t)((total >> (16 * j)) & 0xFFFF);
        seg_base = tile_exclusive(ts, blk, own, mask, (uint32_t)(kFastJ * kBlock * VEC));
    }
    if constexpr (!SET && sizeof(W) >= 4) {
        // masked get: the block's selected elements are gathered in LDS at their rank inside the block and leave as one
        // contiguous run, so every store instruction of a wavefront writes 64 consecutive elements
        __shared__ W stage[kFastJ * kBlock * VEC];
        uint32_t lbase = 0;
#pragma unroll
        for (int j = 0; j < kFastJ; j++) {
            uint32_t k = lbase + (uint32_t)((pre >> (16 * j)) & 0xFFFF);
            lbase += (uint32_t)((total >> (16 * j)) & 0xFFFF);
#pragma unroll
            for (int e = 0; e < VEC; e++)
                if (flags[j] & (1u << e)) stage[k++] = data[j].v[e];
        }
        __syncthreads();
        for (uint32_t i = threadIdx.x; i < lbase; i += kBlock)
            if (seg_base + i < nout) out[seg_base + i] = stage[i];
    } else if constexpr (SET && sizeof(W) >= 4) {
        // masked set: the block's run of values is fetched into LDS with whole-wavefront loads, every thread picks the values of
        // its selected elements by their rank inside the block, merges them into the vectors it read and writes whole vectors
        // back: a wavefront then stores 1 KB of whole cache lines instead of scattered 4-byte pieces, which the memory side turns
        // into read-modify-write cycles (54 -> 47 us for 16 Mi int32 with half the elements selected, although the target is now
        // also read)
        __shared__ W stage[kFastJ * kBlock * VEC];
        uint32_t btotal = 0;
#pragma unroll
        for (int j = 0; j < kFastJ; j++) btotal += (uint32_t)((total >> (16 * j)) & 0xFFFF);
        {
            // the block's run of values: at most kFastJ * VEC fetches per thread, all issued before the first is written to LDS
            // (positions beyond the run fetch its first value again and write nothing)
            constexpr int NI = kFastJ * VEC;
            const uint32_t limit = btotal < nout - (seg_base < nout ? seg_base : nout) ? btotal : nout - (seg_base < nout ? seg_base : nout);
            W val[NI];
#pragma unroll
            for (int q = 0; q < NI; q++) {
                const uint32_t i = threadIdx.x + q * kBlock;
                val[q] = out[(seg_base < nout ? seg_base : 0) + (i < limit ? i : 0)];
            }
#pragma unroll
            for (int q = 0; q < NI; q++) {
                const uint32_t i = threadIdx.x + q * kBlock;
                if (i < limit) stage[i] = val[q];
            }
        }
        __syncthreads();
        uint32_t lbase = 0;
#pragma unroll
        for (int j = 0; j < kFastJ; j++) {
            uint32_t k = lbase + (uint32_t)((pre >> (16 * j)) & 0xFFFF);
            lbase += (uint32_t)((total >> (16 * j)) & 0xFFFF);
            const uint32_t v = (blk * kFastJ + j) * kBlock + threadIdx.x;
            if (flags[j] == 0) continue;
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                if (flags[j] & (1u << e)) {
                    if (seg_base + k < nout) data[j].v[e] = stage[k];
                    k++;
                }
            }
            store_pack<W, VEC>(full + (size_t)v * VEC, data[j]);
        }
    } else {
#pragma unroll
        for (int j = 0; j < kFastJ; j++) {
            uint32_t k = seg_base + (uint32_t)((pre >> (16 * j)) & 0xFFFF);
            seg_base += (uint32_t)((total >> (16 * j)) & 0xFFFF);
            const uint32_t v = (blk * kFastJ + j) * kBlock + threadIdx.x;
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                if (flags[j] & (1u << e)) {
                    if (k < nout) {
                        if constexpr (SET) full[(size_t)v * VEC + e] = out[k];
                        else out[k] = data[j].v[e];
                    }
                    k++;
                }
            }
        }
    }
}

// TrueIndices of a mask whose elements lie in row-major order in memory: the block counts of compact_count_fast_kernel<16>, then
// every thread ranks the selected elements of its four 16-byte mask vectors and notes their positions inside the block's region
// (16 Ki elements, so 16 bits each) in LDS at their rank; the block then writes the coordinates rank by rank, so a wavefront's
// store instruction covers 64 consecutive rows of the target (per-thread runs straight from registers measured 1.6x slower than
// the general kernel: every store instruction touched 64 different cache lines).
template <int BASE, bool PAIR>
__global__ __launch_bounds__(kBlock) void true_indices_fast_kernel(const uint8_t* mask, int64_t* out, Lay shp, uint32_t nvec, uint32_t nout,
                                                                   const uint32_t* block_base, TileSync ts) {
    constexpr int VEC = 16;
    __shared__ uint16_t stage[kFastJ * kBlock * VEC];
    uint32_t flags[kFastJ];
    uint64_t packed = 0;
    uint32_t seg_base = 0;
    const uint32_t blk = blockIdx.x;
    {
        Pack<uint8_t, VEC> mk[kFastJ];   // all loads first, as in compact_move_fast_kernel
#pragma unroll
        for (int j = 0; j < kFastJ; j++) {
            const uint32_t v = (blk * kFastJ + j) * kBlock + threadIdx.x;
            mk[j] = load_pack<uint8_t, VEC>(mask + (v < nvec ? (size_t)v : 0) * VEC);
        }
        if constexpr (BASE == kBasePrefixed) seg_base = block_base[blk];
        else if constexpr (BASE == kBaseSumCounts) seg_base = block_sum_before(block_base, blk);
#pragma unroll
        for (int j = 0; j < kFastJ; j++) {
            const uint32_t v = (blk * kFastJ + j) * kBlock + threadIdx.x;
            flags[j] = v < nvec ? flags_of<VEC>(mk[j]) : 0u;
            packed |= (uint64_t)__popc(flags[j]) << (16 * j);
        }
    }
    uint64_t total;
    const uint64_t pre = block_exclusive_scan64(packed, &total);
    if constexpr (BASE == kBaseLookBack) {
        uint32_t own = 0;
#pragma unroll
        for (int j = 0; j < kFastJ; j++) own += (uint32_t)((total >> (16 * j)) & 0xFFFF);
        seg_base = tile_exclusive(ts, blk, own, mask, (uint32_t)(kFastJ * kBlock * VEC));
    }
    uint32_t lbase = 0;
#pragma unroll
    for (int j = 0; j < kFastJ; j++) {
        uint32_t k = lbase + (uint32_t)((pre >> (16 * j)) & 0xFFFF);
        lbase += (uint32_t)((total >> (16 * j)) & 0xFFFF);
        uint32_t f = flags[j];
        while (f) {
            const int e = __ffs((int)f) - 1;
            f &= f - 1;
            stage[k++] = (uint16_t)((j * kBlock + threadIdx.x) * VEC + e);
        }
    }
    __syncthreads();
    const uint32_t region = blk * (uint32_t)(kFastJ * kBlock * VEC);
    for (uint32_t r = threadIdx.x; r < lbase; r += kBlock) {
        const uint32_t k = seg_base + r;
        if (k >= nout) break;
        uint32_t i = region + stage[r];
        if constexpr (PAIR) {   // two coordinates: one 16-byte store
            const uint32_t q = i / shp.shape[1];
            Pack<int64_t, 2> pr;
            pr.v[0] = (int64_t)q;
            pr.v[1] = (int64_t)(i - q * shp.shape[1]);
            store_pack<int64_t, 2>(out + (size_t)k * 2, pr);
        } else {
            for (int d = shp.nd - 1; d >= 0; d--) {
                const uint32_t q = (d == 0) ? 0u : i / shp.shape[d];
                out[(size_t)k * shp.nd + d] = (int64_t)(i - q * shp.shape[d]);
                i = q;
            }
        }
    }
}

// The words `ntiles` tiles of one launch meet through.
int32_t tile_sync(hipStream_t stream, uint32_t ntiles, TileSync* ts, WorkspaceLease& lease) {
    char* p = nullptr;
    DNH_TRY(sync_words(stream, kSyncTileWords + (size_t)ntiles * 8, (void**)&p, &ts->epoch, lease));
    ts->desc = (unsigned long long*)(p + kSyncTileWords);
    ts->spins = (uint32_t)option(OPT_LOOKBACK_SPINS);
    return DNH_OK;
}

template <class W, bool SET>
int32_t run_compaction_fast(const uint8_t* mask, void* full, void* out, int64_t n, int64_t nout64, hipStream_t stream) {
    constexpr int VEC = 16 / (int)sizeof(W);
    const uint32_t nvec = (uint32_t)(n / VEC);
    const uint32_t nout = (uint32_t)(nout64 > (int64_t)kMaxItems ? kMaxItems : nout64);
    const uint32_t nb = cdiv(nvec, kFastJ * kBlock);
    WorkspaceLease lease;
    if (option(OPT_COMPACT_ONE_PASS) != 0) {
        TileSync ts;
        DNH_TRY(tile_sync(stream, nb, &ts, lease));
        hipLaunchKernelGGL((compact_move_fast_kernel<W, SET, kBaseLookBack>), dim3(nb), dim3(kBlock), 0, stream, mask, (W*)full, (W*)out, nvec, nout,
                           (const uint32_t*)nullptr, ts);
        DNH_LAUNCH_CHECK();
        return DNH_OK;
    }
    uint32_t* counts;
    DNH_TRY(workspace(stream, sizeof(uint32_t) * (size_t)nb, (void**)&counts, lease));
    hipLaunchKernelGGL(compact_count_fast_kernel<VEC>, dim3(nb), dim3(kBlock), 0, stream, mask, nvec, counts);
    DNH_LAUNCH_CHECK();
    const TileSync none{};
    if (nb <= 8192) {
        // few blocks: each block sums the counts before it (at most 32 KB of L2 reads) instead of waiting for a scan launch
        hipLaunchKernelGGL((compact_move_fast_kernel<W, SET, kBaseSumCounts>), dim3(nb), dim3(kBlock), 0, stream, mask, (W*)full, (W*)out, nvec, nout, counts, none);
    } else {
        hipLaunchKernelGGL(compact_scan_kernel, dim3(1), dim3(kBlock), 0, stream, counts, nb);
        DNH_LAUNCH_CHECK();
        hipLaunchKernelGGL((compact_move_fast_kernel<W, SET, kBasePrefixed>), dim3(nb), dim3(kBlock), 0, stream, mask, (W*)full, (W*)out, nvec, nout, counts, none);
    }
    DNH_LAUNCH_CHECK();
    return DNH_OK;
}

// The fast path applies to one unit-stride dimension whose length is a whole number of 16-byte vectors, 16-byte aligned data.
template <bool SET>
bool try_compaction_fast(const MaskArgs& m, void* full, void* out, const Lay& olay, int esize, int64_t n, int64_t nout, hipStream_t stream, int32_t* status) {
    if (m.whole || m.full.nd != 1 || !m.mask[0] || m.mask_stride[0] != 1 || m.full.stride[0] != 1) return false;
    if (olay.nd != 1 || olay.stride[0] != 1) return false;
    if (n > (int64_t)kMaxItems || n == 0 || nout == 0) return false;
    const int vec = 16 / esize;
    // (the tensor's vectors of 4- and 8-byte elements are accessed at element alignment; the mask is read in 4-byte words by the
    // counting pass and in words of `vec` bytes by the moving pass)
    if ((n % vec) != 0 || !vector_address(full, vec, (size_t)esize) || !aligned_to(m.mask[0], (size_t)(vec < 4 ? 4 : vec))) return false;
    switch (esize) {
        case 1: *status = run_compaction_fast<uint8_t, SET>(m.mask[0], full, out, n, nout, stream); return true;
        case 2: *status = run_compaction_fast<uint16_t, SET>(m.mask[0], full, out, n, nout, stream); return true;
        case 4: *status = run_compaction_fast<uint32_t, SET>(m.mask[0], full, out, n, nout, stream); return true;
        case 8: *status = run_compaction_fast<uint64_t, SET>(m.mask[0], full, out, n, nout, stream); return true;
    }
    return false;
}

template <int MODE>
int32_t run_compaction(const MaskArgs& m, void* full, void* out, const Lay& olay, int esize, int64_t n64, int64_t nout64, hipStream_t stream) {
    if (n64 == 0 || nout64 == 0) return DNH_OK;
    if (n64 > (int64_t)kMaxItems) return fail(DNH_ERR_NOT_SUPPORTED, "masked op over more than 2^32 elements");
    const uint32_t n = (uint32_t)n64;
    const uint32_t nout = (uint32_t)(nout64 > (int64_t)kMaxItems ? kMaxItems : nout64);
    const uint32_t nb = cdiv(n, kChunk);
    uint32_t* counts;
    WorkspaceLease lease;
    DNH_TRY(workspace(stream, sizeof(uint32_t) * (size_t)nb, (void**)&counts, lease));
    hipLaunchKernelGGL(compact_count_kernel, dim3(nb), dim3(kBlock), 0, stream, m, n, counts);
    DNH_LAUNCH_CHECK();
    hipLaunchKernelGGL(compact_scan_kernel, dim3(1), dim3(kBlock), 0, stream, counts, nb);
    DNH_LAUNCH_CHECK();
    switch (esize) {
        case 1: hipLaunchKernelGGL((compact_move_kernel<uint8_t, MODE>), dim3(nb), dim3(kBlock), 0, stream, m, (uint8_t*)full, (uint8_t*)out, olay, n, nout, counts); break;
        case 2: hipLaunchKernelGGL((compact_move_kernel<uint16_t, MODE>), dim3(nb), dim3(kBlock), 0, stream, m, (uint16_t*)full, (uint16_t*)out, olay, n, nout, counts); break;
        case 4: hipLaunchKernelGGL((compact_move_kernel<uint32_t, MODE>), dim3(nb), dim3(kBlock), 0, stream, m, (uint32_t*)full, (uint32_t*)out, olay, n, nout, counts); break;
        case 8: hipLaunchKernelGGL((compact_move_kernel<uint64_t, MODE>), dim3(nb), dim3(kBlock), 0, stream, m, (uint64_t*)full, (uint64_t*)out, olay, n, nout, counts); break;
        default: return fail(DNH_ERR_NOT_SUPPORTED, "masked op: unsupported element width");
    }
    DNH_LAUNCH_CHECK();
    return DNH_OK;
}

int32_t make_mask_args(MaskArgs* m, const DnhTensor* full, const DnhTensor* const* masks, int32_t n_masks, const char* what) {
    memset(m, 0, sizeof(*m));
    m->full = lay_of(full);
    if (n_masks != full->ndims) return fail(DNH_ERR_INVALID_ARG, "%s: %d masks given for a tensor of rank %d", what, n_masks, full->ndims);
    if (n_masks > 0 && !masks) return fail(DNH_ERR_INVALID_ARG, "%s: null mask list", what);
    for (int d = 0; d < n_masks; d++) {
        if (!masks[d]) continue;
        DNH_TRY(check_tensor(masks[d], what));
        if (masks[d]->dtype != DNH_BOOL || masks[d]->ndims != 1 || masks[d]->shape[0] != full->shape[d])
            return fail(DNH_ERR_INVALID_ARG, "%s: mask %d must be a rank-1 bool tensor of length %lld", what, d, (long long)full->shape[d]);
        m->mask[d] = (const uint8_t*)elem_ptr(masks[d]);
        m->mask_stride[d] = masks[d]->stride[0];
    }
    return DNH_OK;
}

}  // namespace

extern "C" int32_t dnh_gather(const DnhTensor* t, const DnhTensor* const* idx, int32_t n_idx, const DnhTensor* src, void* stream) {
    DNH_TRY(ensure_init());
    IndexArgs a;
    DNH_TRY(make_index_args(&a, t, src, idx, n_idx, "dnh_gather"));
    const int64_t n = nelems(t);
    if (n == 0) return DNH_OK;
    if (n > (int64_t)kMaxItems) return fail(DNH_ERR_NOT_SUPPORTED, "dnh_gather: more than 2^32 elements");
    hipStream_t s = (hipStream_t)stream;
    int32_t* eflag = nullptr;
    DNH_TRY(error_flag_ptr(s, &eflag));
    const dim3 grid(cdiv(n, kBlock));
    switch (dtype_size(t->dtype)) {
        case 1: hipLaunchKernelGGL(gather_kernel<uint8_t>, grid, dim3(kBlock), 0, s, (uint8_t*)elem_ptr(t), (const uint8_t*)elem_ptr(src), a, (uint32_t)n, eflag); break;
        case 2: hipLaunchKernelGGL(gather_kernel<uint16_t>, grid, dim3(kBlock), 0, s, (uint16_t*)elem_ptr(t), (const uint16_t*)elem_ptr(src), a, (uint32_t)n, eflag); break;
        case 4: hipLaunchKernelGGL(gather_kernel<uint32_t>, grid, dim3(kBlock), 0, s, (uint32_t*)elem_ptr(t), (const uint32_t*)elem_ptr(src), a, (uint32_t)n, eflag); break;
        case 8: hipLaunchKernelGGL(gather_kernel<uint64_t>, grid, dim3(kBlock), 0, s, (uint64_t*)elem_ptr(t), (const uint64_t*)elem_ptr(src), a, (uint32_t)n, eflag); break;
        default: return fail(DNH_ERR_NOT_SUPPORTED, "dnh_gather: unsupported element width");
    }
    DNH_LAUNCH_CHECK();
    return DNH_OK;
}

extern "C" int32_t dnh_scatter(const DnhTensor* t, const DnhTensor* const* idx, int32_t n_idx, const DnhTensor* src, void* stream) {
    DNH_TRY(ensure_init());
    IndexArgs a;
    DNH_TRY(make_index_args(&a, src, t, idx, n_idx, "dnh_scatter"));
    const int64_t n = nelems(src);
    if (n == 0) return DNH_OK;
    if (n > (int64_t)kMaxItems) return fail(DNH_ERR_NOT_SUPPORTED, "dnh_scatter: more than 2^32 elements");
    hipStream_t s = (hipStream_t)stream;
    int32_t* eflag = nullptr;
    DNH_TRY(error_flag_ptr(s, &eflag));
    int32_t bst = DNH_OK;
    if (try_scatter_binned(t, idx, n_idx, src, s, eflag, &bst)) return bst;
    if (dtype_is_fp(t->dtype) && option(OPT_SCATTER_FP_ATOMIC) == 0 && nelems(t) > 0)   // (an empty target: every index is out of range)
        return t->dtype == DNH_F32 ? scatter_ordered<float>(t, src, a, s, eflag) : scatter_ordered<double>(t, src, a, s, eflag);
    const dim3 grid(cdiv(n, kBlock));
#define CASE(DT, X) case DT: hipLaunchKernelGGL(scatter_kernel<X>, grid, dim3(kBlock), 0, s, (X*)elem_ptr(t), (const X*)elem_ptr(src), a, (uint32_t)n, eflag); break;
    switch (t->dtype) {
        CASE(DNH_U8, uint8_t)
        case DNH_I8: hipLaunchKernelGGL(scatter_kernel<uint8_t>, grid, dim3(kBlock), 0, s, (uint8_t*)elem_ptr(t), (const uint8_t*)elem_ptr(src), a, (uint32_t)n, eflag); break;
        case DNH_I16: case DNH_U16: hipLaunchKernelGGL(scatter_kernel<uint16_t>, grid, dim3(kBlock), 0, s, (uint16_t*)elem_ptr(t), (const uint16_t*)elem_ptr(src), a, (uint32_t)n, eflag); break;
        CASE(DNH_I32, int32_t) CASE(DNH_U32, uint32_t) CASE(DNH_I64, int64_t) CASE(DNH_U64, uint64_t) CASE(DNH_F32, float) CASE(DNH_F64, double)
        default: return fail(DNH_ERR_NOT_SUPPORTED, "dnh_scatter on %s", dtype_name(t->dtype));
    }
#undef CASE
    DNH_LAUNCH_CHECK();
    return DNH_OK;
}

extern "C" int32_t dnh_scatter_workspace_bytes(int32_t dtype, int64_t sources, int64_t cells, size_t* bytes) {
    if (!bytes || sources < 0 || cells < 0 || dtype < 0 || dtype >= DNH_DTYPE_COUNT)
        return fail(DNH_ERR_INVALID_ARG, "dnh_scatter_workspace_bytes: bad argument");
    *bytes = 0;
    if (sources == 0 || cells == 0) return DNH_OK;
    if (dtype == DNH_I32 || dtype == DNH_U32) {
        size_t c, t;
        *bytes = binned_choice(sources, cells, &c, &t);
    } else if (dtype_is_fp(dtype) && option(OPT_SCATTER_FP_ATOMIC) == 0) {
        *bytes = ordered_plan(sources, cells, dtype_size(dtype)).total;
    }
    return DNH_OK;
}

extern "C" int32_t dnh_masked_get(const DnhTensor* t, const DnhTensor* src, const DnhTensor* const* masks, int32_t n_masks, void* stream) {
    DNH_TRY(ensure_init());
    DNH_TRY(check_tensor(t, "dnh_masked_get"));
    DNH_TRY(check_tensor(src, "dnh_masked_get"));
    if (t->dtype != src->dtype) return fail(DNH_ERR_INVALID_ARG, "dnh_masked_get: dtypes differ");
    MaskArgs m;
    DNH_TRY(make_mask_args(&m, src, masks, n_masks, "dnh_masked_get"));
    int32_t st = DNH_OK;
    if (try_compaction_fast<false>(m, elem_ptr(src), elem_ptr(t), lay_of(t), dtype_size(t->dtype), nelems(src), nelems(t), (hipStream_t)stream, &st)) return st;
    return run_compaction<kMaskedGet>(m, elem_ptr(src), elem_ptr(t), lay_of(t), dtype_size(t->dtype), nelems(src), nelems(t), (hipStream_t)stream);
}

extern "C" int32_t dnh_masked_set(const DnhTensor* t, const DnhTensor* const* masks, int32_t n_masks, const DnhTensor* src, void* stream) {
    DNH_TRY(ensure_init());
    DNH_TRY(check_tensor(t, "dnh_masked_set"));
    DNH_TRY(check_tensor(src, "dnh_masked_set"));
    if (t->dtype != src->dtype) return fail(DNH_ERR_INVALID_ARG, "dnh_masked_set: dtypes differ");
    MaskArgs m;
    DNH_TRY(make_mask_args(&m, t, masks, n_masks, "dnh_masked_set"));
    int32_t st = DNH_OK;
    if (try_compaction_fast<true>(m, elem_ptr(t), elem_ptr(src), lay_of(src), dtype_size(t->dtype), nelems(t), nelems(src), (hipStream_t)stream, &st)) return st;
    return run_compaction<kMaskedSet>(m, elem_ptr(t), elem_ptr(src), lay_of(src), dtype_size(t->dtype), nelems(t), nelems(src), (hipStream_t)stream);
}

extern "C" int32_t dnh_true_indices(const DnhTensor* t, const DnhTensor* src, void* stream) {
    DNH_TRY(ensure_init());
    DNH_TRY(check_tensor(t, "dnh_true_indices"));
    DNH_TRY(check_tensor(src, "dnh_true_indices"));
    if (t->dtype != DNH_I64 || src->dtype != DNH_BOOL) return fail(DNH_ERR_INVALID_ARG, "dnh_true_indices: needs an int64 target and a bool source");
    if (t->ndims != 2 || t->shape[1] != src->ndims) return fail(DNH_ERR_INVALID_ARG, "dnh_true_indices: target must have shape [nTrue; %d]", src->ndims);
    MaskArgs m;
    memset(&m, 0, sizeof(m));
    m.full = lay_of(src);
    m.whole = 1;
    m.mask[0] = (const uint8_t*)elem_ptr(src);
    if (src->ndims == 0) {
        // a 0-d source has one element and no coordinates: nothing to write
        return DNH_OK;
    }
    const int64_t n = nelems(src), nout = t->shape[0];
    // fast path: the mask's elements lie in row-major order (extent-1 dimensions aside), whole 16-byte vectors, a dense target
    bool dense = n > 0 && nout > 0 && n <= (int64_t)kMaxItems && (n % 16) == 0 && aligned_to(elem_ptr(src), 16) &&
                 t->stride[1] == 1 && t->stride[0] == t->shape[1];
    int64_t expect = 1;
    for (int d = src->ndims - 1; d >= 0 && dense; d--) {
        if (src->shape[d] != 1 && src->stride[d] != expect) dense = false;
        expect *= src->shape[d];
    }
    if (dense) {
        hipStream_t s = (hipStream_t)stream;
        const uint8_t* mask = (const uint8_t*)elem_ptr(src);
        int64_t* out = (int64_t*)elem_ptr(t);
        const uint32_t nvec = (uint32_t)(n / 16);
        const uint32_t no = (uint32_t)(nout > (int64_t)kMaxItems ? kMaxItems : nout);
        const uint32_t nb = cdiv(nvec, kFastJ * kBlock);
        const bool pair = src->ndims == 2 && aligned_to(out, 16);
        WorkspaceLease lease;
        const Lay shp = lay_of(src);
        if (option(OPT_COMPACT_ONE_PASS) != 0) {
            TileSync ts;
            DNH_TRY(tile_sync(s, nb, &ts, lease));
            if (pair) hipLaunchKernelGGL((true_indices_fast_kernel<kBaseLookBack, true>), dim3(nb), dim3(kBlock), 0, s, mask, out, shp, nvec, no, (const uint32_t*)nullptr, ts);
            else hipLaunchKernelGGL((true_indices_fast_kernel<kBaseLookBack, false>), dim3(nb), dim3(kBlock), 0, s, mask, out, shp, nvec, no, (const uint32_t*)nullptr, ts);
            DNH_LAUNCH_CHECK();
            return DNH_OK;
        }
        uint32_t* counts;
        DNH_TRY(workspace(s, sizeof(uint32_t) * (size_t)nb, (void**)&counts, lease));
        hipLaunchKernelGGL(compact_count_fast_kernel<16>, dim3(nb), dim3(kBlock), 0, s, mask, nvec, counts);
        DNH_LAUNCH_CHECK();
        const TileSync none{};
        if (nb <= 8192) {
            if (pair) hipLaunchKernelGGL((true_indices_fast_kernel<kBaseSumCounts, true>), dim3(nb), dim3(kBlock), 0, s, mask, out, shp, nvec, no, counts, none);
            else hipLaunchKernelGGL((true_indices_fast_kernel<kBaseSumCounts, false>), dim3(nb), dim3(kBlock), 0, s, mask, out, shp, nvec, no, counts, none);
        } else {
            hipLaunchKernelGGL(compact_scan_kernel, dim3(1), dim3(kBlock), 0, s, counts, nb);
            DNH_LAUNCH_CHECK();
            if (pair) hipLaunchKernelGGL((true_indices_fast_kernel<kBasePrefixed, true>), dim3(nb), dim3(kBlock), 0, s, mask, out, shp, nvec, no, counts, none);
            else hipLaunchKernelGGL((true_indices_fast_kernel<kBasePrefixed, false>), dim3(nb), dim3(kBlock), 0, s, mask, out, shp, nvec, no, counts, none);
        }
        DNH_LAUNCH_CHECK();
        return DNH_OK;
    }
    return run_compaction<kTrueIndices>(m, nullptr, elem_ptr(t), lay_of(t), 8, n, nout, (hipStream_t)stream);
}
