// ITensorBackend.BatchedInvert (Tensor/Tensor/TensorBackend.fs:144; host: LAPACK getrf + getri per matrix,
// Host/HostBackend.fs:548-576; CUDA: cuBLAS getrfBatched + getriBatched, Cuda/CudaBackend.fs:451-484).
//
// Blocked in-place Gauss-Jordan inversion with partial (row) pivoting, all matrices of the batch side by side:
//   for each block of NB columns
//     1. panel kernel (one workgroup per matrix): NB Gauss-Jordan steps restricted to the block's columns, over all rows;
//        the pivot of step k is the entry of largest magnitude in column k among rows >= k (lowest row on ties, as LAPACK's
//        i?amax); rows are exchanged inside the panel and the exchange recorded.  In-place Gauss-Jordan leaves the column of
//        the elimination matrix where the eliminated column was, so afterwards the panel holds G = columns of the product of
//        the NB elimination steps.
//     2. swap kernel: the recorded row exchanges are applied to the other columns, and the block's rows are copied to T.
//     3. one GEMM on the matrix cores: W += (G - I_block) . T, i.e. the NB elimination steps applied to every other column.
//   finally the row exchanges are undone as column exchanges in reverse order (composed into one permutation, one pass).
// A pivot that is exactly zero marks the matrix singular (LAPACK's info > 0), reported as DNH_ERR_SINGULAR_MATRIX.
// Floating point only; the work is 2 n^3 flops per matrix, nearly all of it in step 3.
// Matrices of more than NB rows replace step 1 by a tournament for the block's pivot rows followed by G = [-C P^-1; P^-1] from the
// exchanged panel (further down: "pivots by tournament"): no step of it waits for a search over all rows, and the update of the
// columns the next block's tournament does not need runs beside that tournament on a second stream.  The option invert_tournament
// forces either form.
#include "common.h"
#include <mutex>
#include <utility>
#include "wave_argmax.h"

namespace dnh {
int32_t gemm_accumulate(int32_t dtype, void* c, const void* a, const void* b, int64_t M, int64_t N, int64_t K, int64_t lda,
                        int64_t ldb, int64_t ldc, int64_t batch, int64_t bsa, int64_t bsb, int64_t bsc, hipStream_t stream);
}

using namespace dnh;

namespace {

constexpr int NB = 32;             // panel width = K of the update GEMM
constexpr int kMaxPanelThreads = 1024;

template <class T>
__device__ inline T abs_of(T x) { return x < T(0) ? -x : x; }

// (value, row) candidates are combined so that the largest magnitude wins and, on equal magnitudes, the lowest row.
template <class T>
__device__ inline void block_arg_max(T& best, int& bi, T* red_v, int* red_i) {
    const int tid = threadIdx.x, nwaves = blockDim.x >> 6;
    wave_arg_max_to_lane63(best, bi);
    if ((tid & 63) == 63) { red_v[tid >> 6] = best; red_i[tid >> 6] = bi; }
    __syncthreads();
    // the wavefronts' candidates (at most 16) are combined by every wavefront for itself: one LDS read per lane and four lane
    // shifts (a loop over the entries cost 0.9 us of a 5 us elimination step, rolled or unrolled)
    arg_max_of_entries(red_v, red_i, nwaves, tid & 63, best, bi);
}

// Thread layout of the panel kernel: lane l of a wavefront works on panel column l % 32 of row l / 32 + 2 * (wavefront, pass),
// so one wavefront instruction touches two whole 32-element row segments (coalesced), and the multiplier of a row — its entry in
// the pivot column — comes from the lane that holds it by a shuffle.
template <class T>
__global__ __launch_bounds__(kMaxPanelThreads) void invert_panel_kernel(T* __restrict__ w, T* __restrict__ gbuf, int32_t* __restrict__ ipiv,
                                                                        int32_t* singular, int n, int ld, int kb, int wc, int64_t bs_w,
                                                                        int64_t bs_g) {
    T* P = w + (int64_t)blockIdx.x * bs_w;
    T* G = gbuf + (int64_t)blockIdx.x * bs_g;
    int32_t* piv = ipiv + (int64_t)blockIdx.x * n;
    const int tid = threadIdx.x, nt = blockDim.x;
    const int jj = tid & 31, rsub = tid >> 5, rpp = nt >> 5, half = tid & 32;
    const bool in_panel = jj < wc;
    __shared__ T srow[NB];
    __shared__ T red_v[2][kMaxPanelThreads / 64];
    __shared__ int red_i[2][kMaxPanelThreads / 64];

    // pivot candidates of the panel's first column; for the later columns they are collected while the column is updated
    T best = T(-1);
    int bi = n;
    for (int r = kb + tid; r < n; r += nt) {
        const T v = abs_of(P[(int64_t)r * ld + kb]);
        if (v > best) { best = v; bi = r; }
    }
    for (int j = 0; j < wc; j++) {
        const int col = kb + j;
        block_arg_max(best, bi, red_v[j & 1], red_i[j & 1]);   // NaN never wins; lowest row on ties
        int p = bi;
        if (!(best > T(0))) {   // zero column (or nothing comparable): singular; carry on so every thread reaches the end
            p = col;
            if (tid == 0) *singular = 1;
        }
        if (tid == 0) piv[col] = p;
        if (p != col && tid < wc) {
            T* x = P + (int64_t)col * ld + kb + tid;
            T* y = P + (int64_t)p * ld + kb + tid;
            const T t = *x; *x = *y; *y = t;
        }
        __syncthreads();
        // the pivot row, scaled: the in-place form puts 1/pivot where the pivot was
        if (tid < wc) {
            const T pv = P[(int64_t)col * ld + col];
            const T x = P[(int64_t)col * ld + kb + tid];
            srow[tid] = (tid == j ? T(1) : x) / pv;
        }
        __syncthreads();
        const T sj = in_panel ? srow[jj] : T(0);
        best = T(-1);
        bi = n;
        constexpr int U = 16;   // loads in flight per thread: the update is bound by the latency of its cache round trips
        for (int r0 = rsub; r0 < n; r0 += rpp * U) {
            T v[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int r = r0 + u * rpp;
                v[u] = (in_panel && r < n) ? P[(int64_t)r * ld + kb + jj] : T(0);
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int r = r0 + u * rpp;
                const T f = __shfl(v[u], half | j, 64);   // this row's entry in the pivot column
                if (in_panel && r < n) {
                    const T nv = (r == col) ? sj : ((jj == j) ? T(0) : v[u]) - f * sj;
                    P[(int64_t)r * ld + kb + jj] = nv;
                    if (jj == j + 1 && r > col) {           // next column's pivot candidates, rows in ascending order per thread
                        const T a = abs_of(nv);
                        if (a > best) { best = a; bi = r; }
                    }
                }
            }
        }
        __syncthreads();
    }
    // G - I_block for the update of the other columns; columns beyond the panel's width are never read (the GEMM's K is wc)
    if (in_panel)
        for (int r = rsub; r < n; r += rpp)
            G[(int64_t)r * NB + jj] = P[(int64_t)r * ld + kb + jj] - ((r == kb + jj) ? T(1) : T(0));
}

// Replays the row exchanges of the block of rows [kb, kb + wc), wc <= NB, on row numbers: entry i of the result says that row pos[i]
// ends up with the content of row src[i] (the block's own rows first, then their partners outside the block; at most 2 * wc = 64
// rows take part).  A column then needs one round of independent loads and one round of stores instead of wc dependent round
// trips.  Run by one whole wavefront: lane j < wc passes the pivot of step j and every lane keeps entry `lane` in registers, so a
// step is a ballot and two lane reads instead of a search through LDS (which took 40 us of a 49 us exchange kernel).
// Writes the entries to pos[] / src[] and returns their number.
__device__ inline int replay_exchanges_wave(int my_pivot, int kb, int wc, int lane, int* pos, int* src) {
    int ps = lane < wc ? kb + lane : -1, sr = ps;
    int m = wc;
    for (int j = 0; j < wc; j++) {
        const int p = __builtin_amdgcn_readlane(my_pivot, j);
        if (p == kb + j) continue;
        int ip;
        if (p < kb + wc) {
            ip = p - kb;
        } else {
            const unsigned long long hit = __ballot(lane >= wc && lane < m && ps == p);
            if (hit) {
                ip = __builtin_ctzll(hit);
            } else {
                ip = m;
                if (lane == m) { ps = p; sr = p; }
                m++;
            }
        }
        const int sj = __builtin_amdgcn_readlane(sr, j), sip = __builtin_amdgcn_readlane(sr, ip);
        if (lane == j) sr = sip;
        if (lane == ip) sr = sj;
    }
    pos[lane] = ps;
    src[lane] = sr;
    return m;
}

// The same Gauss-Jordan steps on a sub-panel of sw <= CW columns held in LDS, so that the dependent chain pivot search ->
// exchange -> pivot row -> update runs at LDS latency instead of cache round trips.  Element (r, c) of the sub-panel lives at
// L[r * CW + c] and is owned by thread (r % rows_per_pass) * CW + c: every access of the update is linear in the thread index,
// the CW lanes of a row sit in one wavefront, and the row's multiplier (its entry in the pivot column) is read by all of them
// before the owner of that column overwrites it — same wavefront, program order — so the update needs no second buffer.
// gsub receives the sub-panel minus the identity (n x sw, row stride gld) for the update of the other columns.
template <class T, int CW>
__global__ __launch_bounds__(kMaxPanelThreads) void invert_subpanel_lds_kernel(T* __restrict__ w, T* __restrict__ gsub, int32_t* __restrict__ ipiv,
                                                                               int32_t* singular, int n, int ld, int cs, int sw, int gld,
                                                                               int64_t bs_w, int64_t bs_gs, T* __restrict__ tbuf, int kb, int wc,
                                                                               int64_t bs_t) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    T* P = w + (int64_t)blockIdx.x * bs_w;
    T* Gs = gsub + (int64_t)blockIdx.x * bs_gs;
    int32_t* piv = ipiv + (int64_t)blockIdx.x * n;
    const int tid = threadIdx.x, nt = blockDim.x;
    const int c = tid % CW, rsub = tid / CW, rpp = nt / CW;
    const bool in_panel = c < sw;
    T* L = (T*)lds_raw;
    __shared__ T red_v[2][kMaxPanelThreads / 64];
    __shared__ int red_i[2][kMaxPanelThreads / 64];
    __shared__ int piv_s[NB];   // pivots go to memory once, at the end: a barrier waits for the stores issued before it
    __shared__ T prow[2][NB];
    {
        // sixteen loads in flight per thread: a single workgroup fetches the whole sub-panel, so the fetch is latency-bound
        constexpr int UL = 16;
        for (int r0 = rsub; r0 < n; r0 += UL * rpp) {
            T v[UL];
#pragma unroll
            for (int u = 0; u < UL; u++) {
                const int r = r0 + u * rpp;
                v[u] = (in_panel && r < n) ? P[(int64_t)r * ld + cs + c] : T(0);
            }
#pragma unroll
            for (int u = 0; u < UL; u++) {
                const int r = r0 + u * rpp;
                if (r < n) L[r * CW + c] = v[u];
            }
        }
    }
    __syncthreads();
    T best = T(-1);
    int bi = n;
    for (int r = cs + tid; r < n; r += nt) {
        const T v = abs_of(L[r * CW]);
        if (v > best) { best = v; bi = r; }
    }
    for (int j = 0; j < sw; j++) {
        const int col = cs + j;
        block_arg_max(best, bi, red_v[j & 1], red_i[j & 1]);
        int p = bi;
        if (!(best > T(0))) {
            p = col;
            if (tid == 0) *singular = 1;
        }
        if (tid == 0) piv_s[j] = p;
        if (tid < CW) {
            // exchange rows col and p; the pivot row also goes to a side buffer (one per step parity), so that nobody reads it
            // from L while its owners rewrite it below and the step needs no barrier between the two
            const T a = L[p * CW + tid];
            if (p != col) {
                L[p * CW + tid] = L[col * CW + tid];
                L[col * CW + tid] = a;
            }
            prow[j & 1][tid] = a;
        }
        __syncthreads();
        const T sj = (c == j ? T(1) : prow[j & 1][c]) / prow[j & 1][j];   // my column's entry of the scaled pivot row
        const bool is_pivot_col = c == j;
        // The update is bound by the instruction issue rate of the one CU that runs it, so the loop body is kept minimal: every
        // row is treated alike (the pivot row is rewritten by its owners afterwards, the next column's pivot search is a separate
        // short walk instead of a compare in every lane).  Four rows per round: all reads of a round are issued before its writes
        // (the rows of a round are distinct, and the lanes of a row read its multiplier before the owner of the pivot column
        // overwrites it).
        constexpr int U = 4;
        int r0 = rsub;
        for (; r0 + (U - 1) * rpp < n; r0 += U * rpp) {
            T v[U], f[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                v[u] = L[(r0 + u * rpp) * CW + c];
                f[u] = L[(r0 + u * rpp) * CW + j];
            }
#pragma unroll
            for (int u = 0; u < U; u++) L[(r0 + u * rpp) * CW + c] = (is_pivot_col ? T(0) : v[u]) - f[u] * sj;
        }
        for (; r0 < n; r0 += rpp) {
            const T v = L[r0 * CW + c], f = L[r0 * CW + j];
            L[r0 * CW + c] = (is_pivot_col ? T(0) : v) - f * sj;
        }
        if (rsub == col % rpp) L[col * CW + c] = sj;   // the owners of the pivot row (they wrote it last, in the loop above)
        __syncthreads();
        // pivot candidates of the next column
        best = T(-1);
        bi = n;
        if (j + 1 < sw)
            for (int r = col + 1 + tid; r < n; r += nt) {
                const T a = abs_of(L[r * CW + j + 1]);
                if (a > best) { best = a; bi = r; }
            }
    }
    if (tid < sw) piv[cs + tid] = piv_s[tid];
    if (in_panel)
        for (int r = rsub; r < n; r += rpp) {
            const T v = L[r * CW + c];
            P[(int64_t)r * ld + cs + c] = v;
            Gs[(int64_t)r * gld + c] = v - ((r == cs + c) ? T(1) : T(0));
        }
    // The sub-panel's row exchanges applied to the other columns of its panel [kb, kb + wc), and the exchanged rows cs .. cs + sw
    // of those columns copied to T (zeros in the sub-panel's own columns) for invert_panel_update_kernel.  One thread per column:
    // all its loads, then all its stores, so no thread reads what another one writes.
    if (wc > sw) {
        __shared__ int pos[2 * NB], src[2 * NB], cnt;
        if (tid < 64) {
            const int m = replay_exchanges_wave(tid < sw ? piv_s[tid] : 0, cs, sw, tid, pos, src);
            if (tid == 0) cnt = m;
        }
        __syncthreads();
        if (tid < wc) {
            const int col = kb + tid;
            T* Tb = tbuf + (int64_t)blockIdx.x * bs_t;
            if (col >= cs && col < cs + sw) {
                for (int j = 0; j < sw; j++) Tb[(int64_t)j * ld + col] = T(0);
            } else {
                const int m = cnt;
                T val[2 * CW];
#pragma unroll
                for (int i = 0; i < 2 * CW; i++)
                    if (i < m) val[i] = P[(int64_t)src[i] * ld + col];
#pragma unroll
                for (int i = 0; i < 2 * CW; i++)
                    if (i < m) {
                        if (src[i] != pos[i]) P[(int64_t)pos[i] * ld + col] = val[i];
                        if (i < sw) Tb[(int64_t)i * ld + col] = val[i];
                    }
            }
        }
    }
}

// W[r, c] += sum_j Gs[r, j] * T[j, c] for the columns c of a panel [kb, kb + wc) outside the sub-panel [cs, cs + sw) that was just
// eliminated (T is zero in the sub-panel's own columns, which therefore stay as they are).  One thread per row and column.
template <class T>
__global__ __launch_bounds__(256) void invert_panel_update_kernel(T* __restrict__ w, const T* __restrict__ gsub, const T* __restrict__ tbuf, int n,
                                                                  int ld, int gld, int kb, int wc, int cs, int sw, int64_t bs_w, int64_t bs_gs,
                                                                  int64_t bs_t) {
    __shared__ T ts[NB][NB + 1];
    const T* Tb = tbuf + (int64_t)blockIdx.y * bs_t;
    for (int i = threadIdx.x; i < sw * wc; i += 256) ts[i / wc][i % wc] = Tb[(int64_t)(i / wc) * ld + kb + i % wc];
    __syncthreads();
    const int cc = threadIdx.x % NB, r = blockIdx.x * (256 / NB) + threadIdx.x / NB;
    const int col = kb + cc;
    if (r >= n || cc >= wc || (col >= cs && col < cs + sw)) return;
    const T* g = gsub + (int64_t)blockIdx.y * bs_gs + (int64_t)r * gld;
    T acc = T(0);
    for (int j = 0; j < sw; j++) acc += g[j] * ts[j][cc];
    T* dst = w + (int64_t)blockIdx.y * bs_w + (int64_t)r * ld + col;
    *dst += acc;
}

// G - I_block of a panel that was processed in sub-panels.
template <class T>
__global__ __launch_bounds__(256) void invert_extract_g_kernel(const T* __restrict__ w, T* __restrict__ gbuf, int n, int ld, int kb, int wc,
                                                               int64_t bs_w, int64_t bs_g) {
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= n * wc) return;
    const int r = idx / wc, c = idx - r * wc;
    gbuf[(int64_t)blockIdx.y * bs_g + (int64_t)r * NB + c] = w[(int64_t)blockIdx.y * bs_w + (int64_t)r * ld + kb + c] - ((r == kb + c) ? T(1) : T(0));
}

// One thread per column in [c_begin, c_end) outside the block's own columns [kb, kb + wc): applies the block's row exchanges in
// order, then copies the block's rows to T.  The block's own columns of T are zero so the update leaves them as they are.
// The exchanges are first replayed on row numbers (thread 0, at most 2 * NB rows take part: the block's rows and their
// partners), which gives for every affected row the row its final content comes from; the columns then see one round of
// independent loads and one round of stores instead of wc dependent round trips.
// OWN: the block's own columns are exchanged as well (their T stays zero); the panel kernels that eliminate column by column have
// exchanged them already.
// Four threads share a column (64 columns per workgroup), each taking every fourth of the affected rows: a quarter of the round
// trips per thread and four times the loads in flight, which is what a kernel this small lives on when another runs beside it.
constexpr int kSwapCols = 64, kSwapThreads = 256;
template <class T, bool OWN>
__global__ __launch_bounds__(kSwapThreads) void invert_swap_kernel(T* __restrict__ w, T* __restrict__ tbuf, const int32_t* __restrict__ ipiv,
                                                                   int n, int ld, int kb, int wc, int c_begin, int c_end, int64_t bs_w,
                                                                   int64_t bs_t) {
    __shared__ int pos[2 * NB];   // affected row positions: the block's rows first, then partners outside the block
    __shared__ int src[2 * NB];   // the row whose content ends up at pos[i]
    __shared__ int cnt;
    const int32_t* piv = ipiv + (int64_t)blockIdx.y * n;
    if (threadIdx.x < 64) {
        const int m = replay_exchanges_wave(threadIdx.x < wc ? piv[kb + threadIdx.x] : 0, kb, wc, threadIdx.x, pos, src);
        if (threadIdx.x == 0) cnt = m;
    }
    __syncthreads();
    const int c = c_begin + blockIdx.x * kSwapCols + (threadIdx.x & 63), part = threadIdx.x >> 6;
    const bool in = c < c_end;
    T* P = w + (int64_t)blockIdx.y * bs_w;
    T* Tb = tbuf + (int64_t)blockIdx.y * bs_t;
    const bool own = c >= kb && c < kb + wc;
    const bool move = in && (OWN || !own);
    if (in && !move)
        for (int j = part; j < wc; j += 4) Tb[(int64_t)j * ld + c] = T(0);
    const int m = cnt;
    T val[2 * NB / 4];
#pragma unroll
    for (int u = 0; u < 2 * NB / 4; u++) {
        const int i = part + 4 * u;
        if (move && i < m) val[u] = P[(int64_t)src[i] * ld + c];
    }
    __syncthreads();   // a column's four threads have read their rows before any of them is overwritten
#pragma unroll
    for (int u = 0; u < 2 * NB / 4; u++) {
        const int i = part + 4 * u;
        if (move && i < m) {
            if (src[i] != pos[i]) P[(int64_t)pos[i] * ld + c] = val[u];
            if (i < wc) Tb[(int64_t)i * ld + c] = own ? T(0) : val[u];
        }
    }
}

// ---- pivots by tournament ---------------------------------------------------------------------------------------------------------
// Eliminating a panel column by column makes every step wait for a pivot search over all remaining rows, which one workgroup can do
// at LDS speed but many cannot do at all without a trip through memory per step.  A block Gauss-Jordan step needs less: once the
// block's NB pivot rows are known and exchanged into place, with P their NB x NB block and C the rest of the panel,
//     G = [ -C P^-1 ; P^-1 ]    (the rows of P^-1 at the block's rows)
// is the panel of the product of the NB elimination steps, and every row of it is independent of the others.  The pivot rows are
// chosen by tournament (communication-avoiding LU).  A game is one wavefront's: it holds 64 R rows of the panel, R per lane in
// registers, runs Gaussian elimination with partial pivoting on them without leaving its registers (the largest entry by lane moves,
// the pivot row read lane by lane into scalars) and names the NB rows it pivoted on.  Rounds of games on kTournRows rows each reduce
// the panel's rows to at most kTournLast, on which one workgroup plays four games and a last one among their winners, always on the
// rows' original values: the last game's pivots, in their order, are the block's.  Every game picks as partial pivoting picks
// (largest magnitude; the lowest lane on ties); over several games the growth bound is weaker in theory and as good in practice.
// The elimination inside a game only ranks rows, so it multiplies by a reciprocal and fuses multiply and add; P^-1 and G are computed
// from the original values with true divisions.
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) { (f(std::integral_constant<int, I>()), ...); }
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) { static_for_impl(f, std::make_integer_sequence<int, N>()); }

template <class T>
__device__ __forceinline__ T read_lane(T v, int lane) {
    if constexpr (sizeof(T) == 4) {
        return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
    } else {
        const long long b = __double_as_longlong(v);
        const int lo = __builtin_amdgcn_readlane((int)(unsigned)(b & 0xFFFFFFFFLL), lane);
        const int hi = __builtin_amdgcn_readlane((int)(b >> 32), lane);
        return __longlong_as_double(((long long)hi << 32) | (unsigned)lo);
    }
}

// The largest value of a wavefront, in every lane.  Values are >= 0 and no NaN, so single precision compares its bit patterns as
// integers (one instruction per step with the lane move folded in).
__device__ __forceinline__ float wave_max(float x) {
    unsigned u = __float_as_uint(x);
    u = max(u, (unsigned)dpp_move<0x111, 0xF>((int)u));   // row_shr:1
    u = max(u, (unsigned)dpp_move<0x112, 0xF>((int)u));   // row_shr:2
    u = max(u, (unsigned)dpp_move<0x114, 0xF>((int)u));   // row_shr:4
    u = max(u, (unsigned)dpp_move<0x118, 0xF>((int)u));   // row_shr:8
    u = max(u, (unsigned)dpp_move<0x142, 0xA>((int)u));   // row_bcast:15 into rows 1 and 3
    u = max(u, (unsigned)dpp_move<0x143, 0xC>((int)u));   // row_bcast:31 into rows 2 and 3
    return __uint_as_float((unsigned)__builtin_amdgcn_readlane((int)u, 63));
}
__device__ __forceinline__ double wave_max(double x) {
    x = __builtin_fmax(x, dpp_move<0x111, 0xF>(x));
    x = __builtin_fmax(x, dpp_move<0x112, 0xF>(x));
    x = __builtin_fmax(x, dpp_move<0x114, 0xF>(x));
    x = __builtin_fmax(x, dpp_move<0x118, 0xF>(x));
    x = __builtin_fmax(x, dpp_move<0x142, 0xA>(x));
    x = __builtin_fmax(x, dpp_move<0x143, 0xC>(x));
    return read_lane(x, 63);
}
__device__ __forceinline__ float fma_of(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double fma_of(double a, double b, double c) { return __builtin_fma(a, b, c); }
// 1 / x to within a few units of the last place: the games only rank rows with it.
__device__ __forceinline__ float quick_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ double quick_rcp(double x) {
    const double r = __builtin_amdgcn_rcp(x);
    return r * (2.0 - x * r);
}

// A thread's row of the panel (live threads), zeros beyond the panel's width.
template <class T>
__device__ __forceinline__ void tourn_load_row(T (&v)[NB], const T* P, bool live, int id, int ld, int kb, int wc) {
    typedef T vec4 __attribute__((ext_vector_type(4)));   // rows start 16-byte aligned (ld and kb are multiples of 4)
    if (wc == NB) {
        const vec4* src = reinterpret_cast<const vec4*>(P + (int64_t)(live ? id : 0) * ld + kb);
#pragma unroll
        for (int q = 0; q < NB / 4; q++) {
            const vec4 x = src[q];
#pragma unroll
            for (int e = 0; e < 4; e++) v[q * 4 + e] = live ? x[e] : T(0);
        }
    } else {
#pragma unroll
        for (int j = 0; j < NB; j++) v[j] = (live && j < wc) ? P[(int64_t)id * ld + kb + j] : T(0);
    }
}

// One game: Gaussian elimination with partial pivoting over the 64 R rows a wavefront holds, R per lane in registers (v: the rows,
// destroyed; id: their numbers, negative for none).  mine[r] receives the step at which the lane's row r was pivoted on, or -1.  A
// column without a non-zero entry among the rows left has no pivot: its step is nobody's.
template <class T, int R>
__device__ __forceinline__ void tourn_game(T (&v)[R][NB], const int (&id)[R], int wc, int (&mine)[R]) {
    const int lane = threadIdx.x & 63;
    T lv[R];   // 1 while the row is in the game, 0 once it was pivoted on (or was never there): a factor, not a branch
#pragma unroll
    for (int r = 0; r < R; r++) {
        lv[r] = id[r] >= 0 ? T(1) : T(0);
        mine[r] = -1;
    }
    static_for<NB>([&](auto kk) {
        constexpr int k = decltype(kk)::value;
        if (k >= wc) return;
        T a[R], amax = T(0);
#pragma unroll
        for (int r = 0; r < R; r++) {
            a[r] = abs_of(v[r][k]) * lv[r];
            amax = max(amax, a[r]);                            // a NaN is passed over
        }
        const T top = wave_max(amax);
        if (!(top > T(0))) return;                             // same in every lane
        const int owner = __builtin_ctzll(__ballot(amax == top));
        int rs = 0;
#pragma unroll
        for (int r = R - 1; r >= 0; r--) rs = (a[r] == top) ? r : rs;
        const int rsel = R == 1 ? 0 : __builtin_amdgcn_readlane(rs, owner);
        T pr[NB];
        static_for<R>([&](auto rr) {
            constexpr int r = decltype(rr)::value;
            if (rsel != r) return;                             // same in every lane
#pragma unroll
            for (int j = k; j < NB; j++) pr[j] = read_lane(v[r][j], owner);
            lv[r] = lane == owner ? T(0) : lv[r];
            mine[r] = lane == owner ? k : mine[r];
        });
        const T rinv = -quick_rcp(pr[k]);
#pragma unroll
        for (int r = 0; r < R; r++) {
            const T m = v[r][k] * rinv * lv[r];
#pragma unroll
            for (int j = k + 1; j < NB; j++) v[r][j] = fma_of(m, pr[j], v[r][j]);
        }
    });
}

// A wavefront's game on entries [first, first + 64 R) of a list of `count` rows (list: row numbers, negative for none; null: the rows
// from kb on), lane l taking entries first + l, first + 64 + l, ...; the winners' row numbers go to out[0 .. NB) (-1 where a step
// found none).  out is written by this wavefront only.
template <class T, int R>
__device__ __forceinline__ void tourn_play(const T* P, const int32_t* list, int first, int count, int ld, int kb, int wc, int* out) {
    const int lane = threadIdx.x & 63;
    int id[R];
    T v[R][NB];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int e = first + r * 64 + lane;
        id[r] = e < count ? (list ? list[e] : kb + e) : -1;
        tourn_load_row(v[r], P, id[r] >= 0, id[r], ld, kb, wc);
    }
    int mine[R];
    if (lane < NB) out[lane] = -1;
    tourn_game<T, R>(v, id, wc, mine);
#pragma unroll
    for (int r = 0; r < R; r++)
        if (mine[r] >= 0) out[mine[r]] = id[r];
}

// One round: workgroup x (two wavefronts) elects among entries [x * kTournRows, (x + 1) * kTournRows) of the round's list (rows_in,
// or the rows from kb on when it is null) and writes NB row numbers (-1: none) to rows_out.  Each wavefront plays 128 rows, two per
// lane, and the first then plays their 64 winners: two short games instead of one on four rows per lane, because that one needs 170
// registers, and a wavefront that wants more than the 128 a retiring wavefront of the update running beside it sets free waits long
// for its place.
constexpr int kTournRows = 256, kTournLast = 512;
template <class T>
__global__ __launch_bounds__(128) void invert_tourn_round_kernel(const T* __restrict__ w, const int32_t* __restrict__ rows_in, int count,
                                                                int32_t* __restrict__ rows_out, int ld, int kb, int wc, int64_t bs_w,
                                                                int64_t bs_rows) {
    __shared__ int won[2][NB];
    __shared__ int out[NB];
    const T* P = w + (int64_t)blockIdx.y * bs_w;
    const int wave = threadIdx.x >> 6;
    tourn_play<T, 2>(P, rows_in ? rows_in + (int64_t)blockIdx.y * bs_rows : nullptr, blockIdx.x * kTournRows + wave * 128,
                     min(count, (int)(blockIdx.x + 1) * kTournRows), ld, kb, wc, won[wave]);
    __syncthreads();
    if (wave != 0) return;
    tourn_play<T, 1>(P, &won[0][0], 0, 2 * NB, ld, kb, wc, out);
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    if (threadIdx.x < NB) rows_out[(int64_t)blockIdx.y * bs_rows + blockIdx.x * NB + threadIdx.x] = out[threadIdx.x];
}

// The last round: elects the block's pivot rows among at most kTournLast rows (four wavefronts play 128 each, the first then plays
// their winners), records them as the exchanges of steps kb .. kb + wc - 1 (ipiv[kb + k] = the position row k's content has reached
// when its turn comes) and inverts their wc x wc block (Gauss-Jordan in the order of election, whose pivots are the elimination's
// own) into pinv (NB x NB per matrix, row-major).
constexpr int kTournLastThreads = 256;
template <class T>
__global__ __launch_bounds__(kTournLastThreads) void invert_tourn_last_kernel(const T* __restrict__ w, const int32_t* __restrict__ rows_in,
                                                                              int count, int32_t* __restrict__ ipiv, T* __restrict__ pinv,
                                                                              int32_t* singular, int n, int ld, int kb, int wc, int64_t bs_w,
                                                                              int64_t bs_rows) {
    static_assert(NB == 32 && kTournLastThreads == 256, "the inversion deals 32 x 32 entries to 256 threads");
    constexpr int W0 = kTournLastThreads / 64, R = kTournLast / kTournLastThreads;
    __shared__ int won[W0][NB];
    __shared__ int ids[NB];
    __shared__ T pm[2][NB][NB + 1];
    const T* P = w + (int64_t)blockIdx.x * bs_w;
    const int32_t* list = rows_in ? rows_in + (int64_t)blockIdx.x * bs_rows : nullptr;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    // one copy of the game's code (the two rounds in a loop): three would not fit the instruction cache
    const bool single = count <= 64 * R;
#pragma unroll 1
    for (int level = single ? 1 : 0; level < 2; level++) {
        const bool second = level == 1 && !single;
        if (level == 0 || wave == 0)
            tourn_play<T, R>(P, second ? &won[0][0] : list, level == 0 ? wave * 64 * R : 0, second ? W0 * NB : count, ld, kb, wc,
                             level == 0 ? won[wave] : ids);
        __syncthreads();
    }
    if (wave == 0 && __ballot(lane < wc && ids[lane] < 0)) {
        // a column without a pivot: the matrix is singular; rows nobody elected keep the bookkeeping consistent
        if (lane == 0) {
            *singular = 1;
            for (int k = 0; k < wc; k++) {
                if (ids[k] >= 0) continue;
                for (int g = kb; g < n; g++) {
                    bool taken = false;
                    for (int j = 0; j < wc; j++) taken |= ids[j] == g;
                    if (!taken) { ids[k] = g; break; }
                }
            }
        }
    }
    __syncthreads();
    // The inversion: thread t keeps entries (t / 32 + 8 e, t % 32), e = 0 .. 3, in registers and posts them after every step to the
    // LDS copy the next step reads its pivot row and column from (two copies in turn: one barrier per step).  The first wavefront
    // also does the bookkeeping of the exchanges, one row per step: lane j keeps exchange j.
    const int j = tid & 31, i0 = tid >> 5;
    T a[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const int i = i0 + 8 * e;
        a[e] = (i < wc && j < wc) ? P[(int64_t)ids[i] * ld + kb + j] : (i == j ? T(1) : T(0));
        pm[0][i][j] = a[e];
    }
    const int sel = lane < wc ? ids[lane] : -1;
    int partner = 0;   // lane k of the first wavefront: where the content of elected row k sits after the exchanges of steps 0 .. k - 1
    __syncthreads();
    for (int k = 0; k < wc; k++) {
        const T(*src)[NB + 1] = pm[k & 1];
        T(*dst)[NB + 1] = pm[(k + 1) & 1];
        const T pv = src[k][k];
        if (tid == 0 && !(abs_of(pv) > T(0))) *singular = 1;
        const T sj = (j == k ? T(1) : src[k][j]) / pv;         // the pivot row, scaled: 1 / pivot where the pivot was
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int i = i0 + 8 * e;
            const T f = src[i][k];                             // the row's entry in the pivot column
            a[e] = (i == k) ? sj : ((j == k) ? T(0) : a[e]) - f * sj;
            dst[i][j] = a[e];
        }
        if (wave == 0) {
            int pos = __builtin_amdgcn_readlane(sel, k);
            // exchange x moves the row when it sits at kb + x or at partner[x]; the exchanges are looked at in order, few ever match
            unsigned long long later = ~0ull;
            while (true) {
                const unsigned long long hit = __ballot(lane < k && (partner == pos || kb + lane == pos)) & later;
                if (!hit) break;
                const int x = __builtin_ctzll(hit);
                const int px = __builtin_amdgcn_readlane(partner, x);
                pos = (pos == kb + x) ? px : kb + x;
                later = ~0ull << (x + 1);   // x <= 30
            }
            if (lane == k) partner = pos;
        }
        __syncthreads();
    }
    if (wave == 0 && lane < wc) ipiv[(int64_t)blockIdx.x * n + kb + lane] = partner;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const int i = i0 + 8 * e;
        pinv[(int64_t)blockIdx.x * NB * NB + i * NB + j] = (i < wc && j < wc) ? a[e] : T(0);
    }
}

// After the exchanges: the panel becomes G (row r of the block's rows: row r - kb of P^-1; any other row: minus its panel entries
// times P^-1), and gbuf receives G - I_block for the update of the other columns.  Four threads per row, eight columns each.
// The same threads apply the update to the w1 columns from next0 on (the next block's panel, which its tournament is waiting for):
// W[r, next0 + c] += sum_j (G - I)[r, j] T[j, next0 + c], the row's 32 factors passed round its four threads through LDS.
constexpr int kTournGThreads = 256;
template <class T>
__global__ __launch_bounds__(kTournGThreads) void invert_tourn_g_kernel(T* __restrict__ w, T* __restrict__ gbuf, const T* __restrict__ pinv,
                                                                        const T* __restrict__ tbuf, int n, int ld, int kb, int wc, int next0,
                                                                        int w1, int64_t bs_w, int64_t bs_g, int64_t bs_t) {
    typedef T vec4 __attribute__((ext_vector_type(4)));
    __shared__ __align__(16) T pi[NB][NB];
    __shared__ __align__(16) T tn[NB][NB];
    __shared__ __align__(16) T gsh[kTournGThreads / 4][NB + 4];
    for (int e = threadIdx.x; e < NB * NB; e += kTournGThreads) {
        const int i = e / NB, c = e % NB;
        pi[i][c] = pinv[(int64_t)blockIdx.y * NB * NB + e];
        tn[i][c] = (i < wc && c < w1) ? tbuf[(int64_t)blockIdx.y * bs_t + (int64_t)i * ld + next0 + c] : T(0);
    }
    __syncthreads();
    // rows beyond n keep their lanes and store nothing
    const int r = blockIdx.x * (kTournGThreads / 4) + threadIdx.x / 4, c0 = (threadIdx.x & 3) * 8;
    const bool in = r < n;
    T* row = w + (int64_t)blockIdx.y * bs_w + (int64_t)(in ? r : 0) * ld;
    T out[8];
    if (in && r >= kb && r < kb + wc) {
#pragma unroll
        for (int j = 0; j < 8; j++) out[j] = pi[r - kb][c0 + j];
    } else {
        T c[NB];
        tourn_load_row(c, w + (int64_t)blockIdx.y * bs_w, in, r, ld, kb, wc);
#pragma unroll
        for (int j = 0; j < 8; j++) out[j] = T(0);
#pragma unroll
        for (int i = 0; i < NB; i++) {
            const vec4 p0 = *reinterpret_cast<const vec4*>(&pi[i][c0]), p1 = *reinterpret_cast<const vec4*>(&pi[i][c0 + 4]);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                out[e] += c[i] * p0[e];
                out[4 + e] += c[i] * p1[e];
            }
        }
#pragma unroll
        for (int j = 0; j < 8; j++) out[j] = -out[j];
    }
    // every thread of a row has read the row's panel entries before any of them is replaced: the four sit in one wavefront
    __builtin_amdgcn_wave_barrier();
    T gi[8];   // G - I
#pragma unroll
    for (int j = 0; j < 8; j++) gi[j] = out[j] - ((r == kb + c0 + j) ? T(1) : T(0));
    if (in) {
        T* g = gbuf + (int64_t)blockIdx.y * bs_g + (int64_t)r * NB;
#pragma unroll
        for (int j = 0; j < 8; j++)
            if (c0 + j < wc) {
                row[kb + c0 + j] = out[j];
                g[c0 + j] = gi[j];
            }
    }
    if (w1 <= 0) return;
    // the row's 32 factors, from its four threads (one wavefront: no barrier, only program order)
    const int rl = threadIdx.x / 4;
    *reinterpret_cast<vec4*>(&gsh[rl][c0]) = vec4{gi[0], gi[1], gi[2], gi[3]};
    *reinterpret_cast<vec4*>(&gsh[rl][c0 + 4]) = vec4{gi[4], gi[5], gi[6], gi[7]};
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    T acc[8];
#pragma unroll
    for (int e = 0; e < 8; e++) acc[e] = T(0);
#pragma unroll 4   // rolled: unrolled whole, the compiler fetches every factor and every vector of tn before the first product
    for (int j = 0; j < NB; j++) {
        const T f = gsh[rl][j];
        const vec4 t0 = *reinterpret_cast<const vec4*>(&tn[j][c0]), t1 = *reinterpret_cast<const vec4*>(&tn[j][c0 + 4]);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            acc[e] += f * t0[e];
            acc[4 + e] += f * t1[e];
        }
    }
    if (!in) return;
#pragma unroll
    for (int e = 0; e < 8; e++)
        if (c0 + e < w1) row[next0 + c0 + e] += acc[e];
}

// Composes the column permutation that undoes the row exchanges: exchanges are applied to columns in reverse order.
// perm[j] = the column of the work matrix that becomes column j of the inverse.  The exchanges of a block of NB steps touch at most
// 2 NB entries; what they do together is found by one wavefront in registers (replay_exchanges_wave: entry pos[i] ends up with the
// content of entry src[i] when the block's exchanges are applied in order; in reverse order, entry src[i] with that of pos[i]).  Four
// wavefronts replay four blocks at a time, the first then applies them to the permutation, last block first: two LDS round trips a
// block instead of four a step.
__global__ __launch_bounds__(256) void invert_perm_kernel(int32_t* __restrict__ perm, const int32_t* __restrict__ ipiv, int n, int use_lds) {
    extern __shared__ int32_t sp[];
    __shared__ int pos[4][2 * NB], src[4][2 * NB], cnt[4];
    int32_t* out = perm + (int64_t)blockIdx.x * n;
    const int32_t* piv = ipiv + (int64_t)blockIdx.x * n;
    int32_t* cur = use_lds ? sp : out;
    for (int i = threadIdx.x; i < n; i += 256) cur[i] = i;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int blocks = (n + NB - 1) / NB;
    for (int top = blocks - 1; top >= 0; top -= 4) {
        const int blk = top - wave;
        if (blk >= 0) {
            const int kb = blk * NB, wc = min(NB, n - kb);
            const int m = replay_exchanges_wave(lane < wc ? piv[kb + lane] : 0, kb, wc, lane, pos[wave], src[wave]);
            if (lane == 0) cnt[wave] = m;
        }
        __syncthreads();   // also: the identity is in place before the first block is applied
        if (wave == 0) {
            for (int x = 0; x < 4 && top - x >= 0; x++) {
                const bool in = lane < cnt[x];
                const int32_t v = in ? cur[pos[x][lane]] : 0;
                __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");   // every lane has read before any writes
                if (in) cur[src[x][lane]] = v;
                __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");   // and the next block reads what this one wrote
            }
        }
        __syncthreads();
    }
    if (use_lds)
        for (int i = threadIdx.x; i < n; i += 256) out[i] = sp[i];
}

template <class T>
__global__ __launch_bounds__(256) void invert_unpermute_kernel(T* __restrict__ out, const T* __restrict__ w, const int32_t* __restrict__ perm,
                                                               int n, int ld, int64_t bs_w) {
    const int j = blockIdx.x * 256 + threadIdx.x;
    if (j >= n) return;
    const int i = blockIdx.y;
    const int64_t b = blockIdx.z;
    out[(b * n + i) * (int64_t)n + j] = w[b * bs_w + (int64_t)i * ld + perm[b * n + j]];
}

__global__ void invert_clear_flag_kernel(int32_t* flag) { *flag = 0; }

size_t align_up(size_t x) { return (x + 255) / 256 * 256; }

// One more stream, created on first use and kept: the update of the columns a tournament does not need runs on it beside the tournament.
int32_t side_stream(hipStream_t* out) {
    static std::mutex mu;
    static hipStream_t s = nullptr;
    std::lock_guard<std::mutex> lock(mu);
    if (!s) DNH_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *out = s;
    return DNH_OK;
}

template <class T>
int32_t invert_impl(const DnhTensor* t, const DnhTensor* src, hipStream_t stream) {
    const int nd = t->ndims;
    const int64_t n64 = t->shape[nd - 1];
    int64_t batch = 1;
    for (int d = 0; d < nd - 2; d++) batch *= t->shape[d];
    if (n64 == 0 || batch == 0) return DNH_OK;
    if (n64 > 46340 || batch > 65535) return fail(DNH_ERR_NOT_SUPPORTED, "dnh_batched_invert: matrix size or batch too large");
    const int n = (int)n64;
    const int ld = (n + 3) / 4 * 4;  // rows start 16-byte aligned, which the update GEMM's vector loads need
    const int64_t bs_w = (int64_t)n * ld, bs_g = (int64_t)n * NB, bs_t = (int64_t)NB * ld;

    bool t_is_c = true;
    {
        int64_t expect = 1;
        for (int d = nd - 1; d >= 0; d--) {
            if (t->shape[d] > 1 && t->stride[d] != expect) t_is_c = false;
            expect *= t->shape[d];
        }
    }
    const size_t sz_w = align_up((size_t)batch * bs_w * sizeof(T)), sz_g = align_up((size_t)batch * bs_g * sizeof(T));
    const size_t sz_t = align_up((size_t)batch * bs_t * sizeof(T)), sz_i = align_up((size_t)batch * n * sizeof(int32_t));
    const size_t sz_r = t_is_c ? 0 : align_up((size_t)batch * n * n * sizeof(T));
    // pivots by tournament: two lists of candidate rows (NB per workgroup of the first round) and the inverted pivot block
    const int tourn_opt = option(OPT_INVERT_TOURNAMENT);
    const bool tourn = tourn_opt == 1 || (tourn_opt < 0 && n > NB);   // measured faster from two blocks on, single and batched
    const int64_t bs_rows = (int64_t)cdiv(n, kTournRows) * NB;
    const size_t sz_rows = tourn ? align_up((size_t)batch * bs_rows * sizeof(int32_t)) : 0;
    const size_t sz_pinv = tourn ? align_up((size_t)batch * NB * NB * sizeof(T)) : 0;
    void* block = nullptr;
    DNH_TRY(dnh_alloc_async(sz_w + 2 * sz_g + sz_t + 2 * sz_i + sz_r + 256 + 2 * sz_rows + sz_pinv, stream, &block));
    char* base = (char*)block;
    T* W = (T*)base;
    T* G = (T*)(base + sz_w);
    T* Tb = (T*)(base + sz_w + sz_g);
    int32_t* ipiv = (int32_t*)(base + sz_w + sz_g + sz_t);
    int32_t* perm = (int32_t*)(base + sz_w + sz_g + sz_t + sz_i);
    T* R = t_is_c ? (T*)elem_ptr(t) : (T*)(base + sz_w + sz_g + sz_t + 2 * sz_i);
    int32_t* flag = (int32_t*)(base + sz_w + sz_g + sz_t + 2 * sz_i + sz_r);
    T* Gs = (T*)(base + sz_w + sz_g + sz_t + 2 * sz_i + sz_r + 256);   // sub-panel multipliers (n x sb per matrix, sb <= NB)
    int32_t* rows_a = (int32_t*)(base + sz_w + 2 * sz_g + sz_t + 2 * sz_i + sz_r + 256);
    int32_t* rows_b = (int32_t*)((char*)rows_a + sz_rows);
    T* pinv = (T*)((char*)rows_a + 2 * sz_rows);

    // the side stream of the tournament form (the library's own, default priority), with the two events that order it against `stream`
    hipStream_t side = nullptr;
    hipEvent_t ev_main = nullptr, ev_side = nullptr;
    bool side_busy = false;
    if (tourn && n > 2 * NB) {
        DNH_TRY(side_stream(&side));
        if (hipEventCreateWithFlags(&ev_main, hipEventDisableTiming) != hipSuccess ||
            hipEventCreateWithFlags(&ev_side, hipEventDisableTiming) != hipSuccess) {
            if (ev_main) (void)hipEventDestroy(ev_main);
            (void)dnh_free_async(block, stream);
            return fail(DNH_ERR_HIP, "dnh_batched_invert: cannot create an event");
        }
    }
    int32_t st = DNH_OK;
    auto body = [&]() -> int32_t {
        // src (any layout, broadcast batch dimensions included) -> W, rows padded to ld
        DnhTensor wd = *t;
        wd.base = W;
        wd.offset = 0;
        int64_t acc = 1;
        for (int d = nd - 1; d >= 0; d--) {
            if (d == nd - 1) { wd.stride[d] = 1; acc = ld; }
            else { wd.stride[d] = acc; acc *= t->shape[d]; }
        }
        DNH_TRY(dnh_copy(&wd, src, stream));
        hipLaunchKernelGGL(invert_clear_flag_kernel, dim3(1), dim3(1), 0, stream, flag);
        // threads of the one workgroup that eliminates a (sub-)panel: fewer wavefronts make its four barriers per step cheaper,
        // more of them hide LDS latency.  Measured (1000 / 2000 / 4000 rows): 512 threads are 5-8 % faster than 1024 everywhere
        // except single precision beyond 2048 rows (4 % slower); 256 are slower throughout.
        const int max_threads = (sizeof(T) == 4 && n > 2048) ? kMaxPanelThreads : 512;
        int threads = (n + 63) / 64 * 64;
        if (threads > max_threads) threads = max_threads;
        // widest sub-panel (a power of two <= NB) whose rows fit in the LDS a workgroup may use; 0 = none fits
        int lds_limit = 0, dev = 0;
        DNH_HIP(hipGetDevice(&dev));
        DNH_HIP(hipDeviceGetAttribute(&lds_limit, hipDeviceAttributeMaxSharedMemoryPerBlock, dev));
        auto lds_need = [&](int cw) { return (size_t)n * cw * sizeof(T); };
        int sb = 0;
        for (int cand = NB; cand >= 1; cand >>= 1)
            if (lds_need(cand) + 2048 <= (size_t)lds_limit) { sb = cand; break; }   // 2 KB for the kernel's static arrays
        auto launch_subpanel = [&](int cw, T* g, int cs, int sw, int gld, int pkb, int pwc) -> int32_t {
            const size_t lds = lds_need(cw);
#define DNH_SUBPANEL(CWV)                                                                                                              \
    case CWV:                                                                                                                          \
        if (lds > 32 * 1024)                                                                                                           \
            DNH_HIP(hipFuncSetAttribute((const void*)invert_subpanel_lds_kernel<T, CWV>, hipFuncAttributeMaxDynamicSharedMemorySize,  \
                                        (int)lds));                                                                                    \
        hipLaunchKernelGGL((invert_subpanel_lds_kernel<T, CWV>), dim3((unsigned)batch), dim3(threads), lds, stream, W, g, ipiv, flag, n, ld, \
                           cs, sw, gld, bs_w, bs_g, Tb, pkb, pwc, bs_t);                                                               \
        break;
            switch (cw) {
                DNH_SUBPANEL(32) DNH_SUBPANEL(16) DNH_SUBPANEL(8) DNH_SUBPANEL(4) DNH_SUBPANEL(2) DNH_SUBPANEL(1)
            }
#undef DNH_SUBPANEL
            return DNH_OK;
        };
        for (int kb = 0; kb < n; kb += NB) {
            const int wc = (n - kb < NB) ? n - kb : NB;
            if (tourn) {
                // the tournament of a block: queued for the first block here, for every later one right behind the previous block's
                // own-column work (below), ahead of that block's side-stream launches, so that the device never waits for it
                auto play = [&](int pkb, int pwc) {
                    int count = n - pkb;
                    const int32_t* rows_in = nullptr;
                    int32_t* rows_out = rows_a;
                    while (count > kTournLast) {
                        const int chunks = (int)cdiv(count, kTournRows);
                        hipLaunchKernelGGL((invert_tourn_round_kernel<T>), dim3((unsigned)chunks, (unsigned)batch), dim3(128), 0, stream, W,
                                           rows_in, count, rows_out, ld, pkb, pwc, bs_w, bs_rows);
                        count = chunks * NB;
                        rows_in = rows_out;
                        rows_out = rows_out == rows_a ? rows_b : rows_a;
                    }
                    hipLaunchKernelGGL((invert_tourn_last_kernel<T>), dim3((unsigned)batch), dim3(kTournLastThreads), 0, stream, W, rows_in, count,
                                       ipiv, pinv, flag, n, ld, pkb, pwc, bs_w, bs_rows);
                };
                if (kb == 0) play(kb, wc);
                if (side_busy) {
                    DNH_HIP(hipStreamWaitEvent(stream, ev_side, 0));
                    side_busy = false;
                }
                // The exchange and the update W += (G - I) . T of the block's own columns and of the next block's (all its tournament
                // needs) run here; the columns to their left and right get theirs on the side stream, beside that tournament.  The
                // exchange after it waits for them: it rewrites T, and G is rewritten behind it.
                const int next0 = kb + wc, next1 = (n - next0 < NB) ? n : next0 + NB;
                auto exchange = [&](int c0, int c1, hipStream_t s) {
                    if (c1 > c0)
                        hipLaunchKernelGGL((invert_swap_kernel<T, true>), dim3((unsigned)cdiv(c1 - c0, kSwapCols), (unsigned)batch),
                                           dim3(kSwapThreads), 0, s, W, Tb, ipiv, n, ld, kb, wc, c0, c1, bs_w, bs_t);
                };
                auto update = [&](int c0, int c1, hipStream_t s) -> int32_t {
                    if (c1 <= c0) return DNH_OK;
                    return gemm_accumulate(t->dtype, W + c0, G, Tb + c0, n, c1 - c0, wc, NB, ld, ld, batch, bs_g, bs_t, bs_w, s);
                };
                exchange(0, n, stream);
                hipLaunchKernelGGL((invert_tourn_g_kernel<T>), dim3((unsigned)cdiv(n, kTournGThreads / 4), (unsigned)batch), dim3(kTournGThreads), 0,
                                   stream, W, G, pinv, Tb, n, ld, kb, wc, next0, next1 - next0, bs_w, bs_g, bs_t);
                hipStream_t rest = stream;
                if (side) {
                    DNH_HIP(hipEventRecord(ev_main, stream));
                    if (next0 < n) play(next0, next1 - next0);
                    DNH_HIP(hipStreamWaitEvent(side, ev_main, 0));
                    rest = side;
                }
                DNH_TRY(update(0, kb, rest));
                DNH_TRY(update(next1, n, rest));
                if (side) {
                    DNH_HIP(hipEventRecord(ev_side, side));
                    side_busy = true;
                } else if (next0 < n) {
                    play(next0, next1 - next0);
                }
                continue;
            }
            if (sb == NB) {
                DNH_TRY(launch_subpanel(NB, G, kb, wc, NB, kb, wc));
            } else if (sb > 0) {
                for (int cs = kb; cs < kb + wc; cs += sb) {
                    const int sw = (kb + wc - cs < sb) ? kb + wc - cs : sb;
                    DNH_TRY(launch_subpanel(sb, Gs, cs, sw, sb, kb, wc));   // also exchanges the panel's other columns and fills T
                    if (wc > sw)                                             // the sub-panel's steps applied to those columns
                        hipLaunchKernelGGL((invert_panel_update_kernel<T>), dim3((unsigned)cdiv(n, 256 / NB), (unsigned)batch), dim3(256), 0, stream,
                                           W, Gs, Tb, n, ld, sb, kb, wc, cs, sw, bs_w, bs_g, bs_t);
                }
                hipLaunchKernelGGL((invert_extract_g_kernel<T>), dim3((unsigned)cdiv((int64_t)n * wc, 256), (unsigned)batch), dim3(256), 0, stream,
                                   W, G, n, ld, kb, wc, bs_w, bs_g);
            } else {
                hipLaunchKernelGGL((invert_panel_kernel<T>), dim3((unsigned)batch), dim3(threads), 0, stream, W, G, ipiv, flag, n, ld, kb, wc,
                                   bs_w, bs_g);
            }
            if (n > wc) {
                hipLaunchKernelGGL((invert_swap_kernel<T, false>), dim3((unsigned)cdiv(n, kSwapCols), (unsigned)batch), dim3(kSwapThreads), 0, stream,
                                   W, Tb, ipiv, n, ld, kb, wc, 0, n, bs_w, bs_t);
                DNH_TRY(gemm_accumulate(t->dtype, W, G, Tb, n, n, wc, NB, ld, ld, batch, bs_g, bs_t, bs_w, stream));
            }
        }
        if (side_busy) {
            DNH_HIP(hipStreamWaitEvent(stream, ev_side, 0));
            side_busy = false;
        }
        const int use_lds = (size_t)n * sizeof(int32_t) <= 48 * 1024;
        hipLaunchKernelGGL(invert_perm_kernel, dim3((unsigned)batch), dim3(256), use_lds ? (size_t)n * sizeof(int32_t) : 0, stream, perm, ipiv,
                           n, use_lds);
        hipLaunchKernelGGL((invert_unpermute_kernel<T>), dim3((unsigned)cdiv(n, 256), (unsigned)n, (unsigned)batch), dim3(256), 0, stream, R, W,
                           perm, n, ld, bs_w);
        DNH_LAUNCH_CHECK();
        if (!t_is_c) {
            DnhTensor rd = *t;
            rd.base = R;
            rd.offset = 0;
            int64_t a2 = 1;
            for (int d = nd - 1; d >= 0; d--) { rd.stride[d] = a2; a2 *= t->shape[d]; }
            DNH_TRY(dnh_copy(t, &rd, stream));
        }
        int32_t host_flag = 0;
        DNH_HIP(hipMemcpyAsync(&host_flag, flag, sizeof(int32_t), hipMemcpyDeviceToHost, stream));
        DNH_HIP(hipStreamSynchronize(stream));
        if (host_flag) return fail(DNH_ERR_SINGULAR_MATRIX, "cannot invert singular matrix");
        return DNH_OK;
    };
    st = body();
    if (side_busy) {   // an error left the side stream at work on the block about to be freed
        if (hipStreamWaitEvent(stream, ev_side, 0) != hipSuccess) (void)hipStreamSynchronize(side);
    }
    if (ev_main) (void)hipEventDestroy(ev_main);
    if (ev_side) (void)hipEventDestroy(ev_side);
    (void)dnh_free_async(block, stream);
    return st;
}

}  // namespace

extern "C" int32_t dnh_batched_invert(const DnhTensor* t, const DnhTensor* src, void* stream) {
    DNH_TRY(ensure_init());
    DNH_TRY(check_tensor(t, "dnh_batched_invert"));
    DNH_TRY(check_tensor(src, "dnh_batched_invert"));
    if (t->dtype != src->dtype) return fail(DNH_ERR_INVALID_ARG, "dnh_batched_invert: dtypes differ");
    if (!dtype_is_fp(t->dtype))
        return fail(DNH_ERR_NOT_SUPPORTED, "dnh_batched_invert: this operation is only supported for floating point numbers");
    if (!same_shape(t, src)) return fail(DNH_ERR_INVALID_ARG, "dnh_batched_invert: source is not broadcast to the target's shape");
    if (t->ndims < 2) return fail(DNH_ERR_INVALID_ARG, "dnh_batched_invert: need at least a matrix");
    if (t->shape[t->ndims - 1] != t->shape[t->ndims - 2]) return fail(DNH_ERR_INVALID_ARG, "dnh_batched_invert: matrices are not square");
    if (t->dtype == DNH_F32) return invert_impl<float>(t, src, (hipStream_t)stream);
    return invert_impl<double>(t, src, (hipStream_t)stream);
}
