// dnh_dot: ITensorBackend VecVecDot / MatVecDot / MatMatDot / BatchedMatMatDot (Tensor/Tensor/TensorBackend.fs:137-140;
// dispatch by rank as Tensor.FillDot, Tensor/Tensor/Tensor.fs:2714-2730; Host semantics Host/HostBackend.fs:463-546).
//
// One strided-batched GEMM kernel, C[b] = A[b] * B[b] (alpha 1, beta 0), written for gfx950:
//   - 128x128 block tile, K step 16, 256 threads = 4 wavefronts in a 2x2 arrangement, each owning a 64x64 sub-tile;
//   - fp32: four 32x32 accumulators per wavefront on v_mfma_f32_32x32x2_f32 (A and B operands one dword per lane);
//     fp64: sixteen 16x16 accumulators per wavefront on v_mfma_f64_16x16x4_f64;
//   - A is staged k-major ([k][m]) and B as [k][n] in LDS, double buffered, so every MFMA operand fetch is a
//     conflict-free 4-byte LDS read of consecutive addresses; the next K step's global loads are issued before the
//     MFMAs of the current one; workgroup ids are remapped so that each XCD (own L2) gets a contiguous range of tiles;
//   - operands are addressed straight from the descriptors (any strides, broadcast batch dimensions, row-major
//     target written directly): no pointer arrays, no column-major temporary and transposing copy-back as on the
//     reference's BLAS paths (Tensor/Tensor/BlasSupport.fs:173-190, Cuda/CudaBLAS.fs:28-38).
// The "fast" instantiation (row-major, 16-byte aligned A and B) uses 16-byte global loads on interior tiles and guarded
// scalar loads on edge tiles; every other layout runs the same kernel with guarded scalar loads throughout.
// This kernel is the general form (operands strided in both dimensions, accumulation, K < one step).  Operands that are contiguous
// along one of their dimensions take the kernels further down: gemm_bf16x3_kernel / gemm_bf16x3_big_kernel (single precision on the
// bf16 matrix instructions) and gemm_f64_kernel (double precision), whose K loops have a hand-pinned instruction order.
#include "map_kernels.h"

using namespace dnh;

namespace {

constexpr int BM = 128, BN = 128, PAD = 4;
template <class T> constexpr int kBK = sizeof(T) == 8 ? 8 : 16;  // K step: keeps the double-buffered tiles within 64 KB of LDS

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef double f64x4 __attribute__((ext_vector_type(4)));

struct GemmArgs {
    int64_t M, N, K;
    int64_t sam, sak, sbk, sbn, scm, scn;
    int nbatch;                                   // batch dimensions
    uint32_t bshape[DNH_MAX_DIMS];
    int64_t bsa[DNH_MAX_DIMS], bsb[DNH_MAX_DIMS], bsc[DNH_MAX_DIMS];
    uint32_t tiles_m, tiles_n;
    uint32_t xcd_chunk;                           // total tiles / 8 when divisible, else 0 (identity order)
    uint32_t accumulate;                          // 1: c += a.b (used by the blocked matrix inversion), 0: c = a.b
    int64_t kchunk;                               // > 0: the innermost batch dimension walks K in chunks of this many (split K)
    uint32_t xcd_2d;                              // 1: one matrix whose tiles are dealt to the 8 XCDs as a 2 x 4 grid of regions
};

template <class T, bool FAST, bool ACC, bool SPLIT>
__global__ __launch_bounds__(kBlock, (sizeof(T) == 4 && FAST ? 4 : 2)) void gemm_kernel(T* __restrict__ c, const T* __restrict__ a, const T* __restrict__ b, GemmArgs g) {
    constexpr int BK = kBK<T>;
    __shared__ __align__(16) T As[2][BK][BM + PAD];
    __shared__ __align__(16) T Bs[2][BK][BN + PAD];

    // XCD-aware tile order: consecutive workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.  Remapping
    // id -> (id % 8) * (total / 8) + id / 8 hands every XCD one contiguous range of tiles, so the tiles of one matrix pair
    // (which re-read the same A rows and B columns) share an L2 instead of being spread over all eight.
    uint32_t bid = blockIdx.x;
    if (g.xcd_chunk) bid = (bid % 8u) * g.xcd_chunk + bid / 8u;
    const uint32_t tn = bid % g.tiles_n;
    bid /= g.tiles_n;
    const uint32_t tm = bid % g.tiles_m;
    bid /= g.tiles_m;
    int64_t oa = 0, ob = 0, oc = 0;
    uint32_t chunk_id = 0;
    for (int d = g.nbatch - 1; d >= 0; d--) {
        const uint32_t q = (d == 0) ? 0u : bid / g.bshape[d];
        const uint32_t i = bid - q * g.bshape[d];
        bid = q;
        oa += (int64_t)i * g.bsa[d];
        ob += (int64_t)i * g.bsb[d];
        oc += (int64_t)i * g.bsc[d];
        if (SPLIT && d == g.nbatch - 1) chunk_id = i;
    }
    // this block's extent along k: the whole of K, or one chunk of it (SPLIT: the innermost batch dimension counts the chunks)
    const int64_t K = SPLIT ? min(g.kchunk, g.K - (int64_t)chunk_id * g.kchunk) : g.K;
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
    a += oa;
    b += ob;
    c += oc;

    const int tid = threadIdx.x;
    // global -> register staging
    constexpr int SPT = BM * BK / kBlock;  // elements of each tile per thread
    T ra[SPT], rb[SPT];
    uint32_t amask = 0, bmask = 0;  // element loads: bit i = ra[i] / rb[i] lies inside the matrix (else it is stored as zero)

    const bool full_mn = m0 + BM <= g.M && n0 + BN <= g.N;
    // load_tiles(k0, buf) fetches the tiles of K step k0 and says where they are: kVec / kScalar = in registers (ra/rb, in the
    // vector or the element layout), still to be written to LDS buffer `buf` by store_tiles after the MFMAs of the current step, so
    // that the fetch overlaps them; kDirect = already written to buffer `buf` (nobody reads that buffer during this K step).
    //   FAST kernel (row-major, 16-byte aligned operands): whole K steps of interior tiles use 16-byte loads.
    //     fp32 (LEAN): edge tiles use the same loads with rows of A beyond M and vectors of B beyond N replaced by zeros; only the
    //     K tail (K % BK != 0) or an N that is not a whole number of vectors goes element by element, straight into LDS, in a rolled
    //     loop that keeps no addresses or staging registers alive across the MFMA chain: 128 registers, four wavefronts per SIMD,
    //     and edge-heavy shapes (4000^3) run 37 % faster than with element loads for edge tiles.
    //     fp64: 128 accumulator registers allow two wavefronts per SIMD either way; edge tiles and tails take guarded element
    //     loads staged in registers (measured 5-9 % faster for fp64 than the lean form).
    //   General kernel (any strides): guarded element loads staged in registers.
    enum { kDirect = 0, kVec = 1, kScalar = 2 };
    constexpr bool LEAN = FAST && sizeof(T) == 4;
    const bool n_vec_ok = (g.N % (16 / (int)sizeof(T))) == 0;
    auto load_tiles = [&](int64_t k0, int buf) -> int {
        if (FAST && (LEAN ? n_vec_ok : full_mn) && k0 + BK <= K) {
            constexpr int V = 16 / (int)sizeof(T);           // elements per 16-byte load
            constexpr int APT = (BM * BK) / (kBlock * V);     // loads per thread for A (fp32: 2, fp64: 4)
            constexpr int KV = BK / V;                        // vectors per A row
#pragma unroll
            for (int i = 0; i < APT; i++) {
                const int idx = tid + i * kBlock;
                const int row = idx / KV, kv = (idx % KV) * V;
                Pack<T, V> v;
                if (full_mn || m0 + row < g.M) v = load_pack<T, V>(a + (m0 + row) * g.sam + (k0 + kv));
                else v = splat_pack<T, V>(T(0));
#pragma unroll
                for (int e = 0; e < V; e++) ra[i * V + e] = v.v[e];
            }
            constexpr int NV = BN / V;                        // vectors per B row
#pragma unroll
            for (int i = 0; i < APT; i++) {
                const int idx = tid + i * kBlock;
                const int kk = idx / NV, nv = (idx % NV) * V;
                Pack<T, V> v;
                if (full_mn || n0 + nv < g.N) v = load_pack<T, V>(b + (k0 + kk) * g.sbk + (n0 + nv));
                else v = splat_pack<T, V>(T(0));
#pragma unroll
                for (int e = 0; e < V; e++) rb[i * V + e] = v.v[e];
            }
            return kVec;
        } else if constexpr (LEAN) {
#pragma unroll 1
            for (int i = 0; i < SPT; i++) {
                const int idx = tid + i * kBlock;
                {
                    const int row = idx / BK, kk = idx % BK;
                    const int64_t m = m0 + row, k = k0 + kk;
                    As[buf][kk][row] = (m < g.M && k < K) ? a[m * g.sam + k * g.sak] : T(0);
                }
                {
                    const int kk = idx / BN, col = idx % BN;
                    const int64_t k = k0 + kk, n = n0 + col;
                    Bs[buf][kk][col] = (k < K && n < g.N) ? b[k * g.sbk + n * g.sbn] : T(0);
                }
            }
            return kDirect;
        } else if (full_mn && k0 + BK <= K) {
            // whole K step of an interior tile: every element exists
            amask = ~0u;
            bmask = ~0u;
#pragma unroll
            for (int i = 0; i < SPT; i++) {
                const int idx = tid + i * kBlock;
                ra[i] = a[(m0 + idx / BK) * g.sam + (k0 + idx % BK) * g.sak];
                rb[i] = b[(k0 + idx / BN) * g.sbk + (n0 + idx % BN) * g.sbn];
            }
            return kScalar;
        } else {
            amask = 0;
            bmask = 0;
#pragma unroll
            for (int i = 0; i < SPT; i++) {
                const int idx = tid + i * kBlock;
                {
                    const int row = idx / BK, kk = idx % BK;
                    const int64_t m = m0 + row, k = k0 + kk;
                    // Unconditional load from an address clamped to element (0, 0); whether the element counts is kept as one
                    // bit and applied when the registers go to LDS, after the MFMAs of the current step.  The loads of a thread
                    // are then issued back to back and nothing waits for them before the MFMA chain (`cond ? load : 0` leaves
                    // the compiler free to branch around every load or to select right after it, and which one it picked
                    // changed with unrelated edits: fp64 edge tiles ran 20 % slower when it did).
                    const bool ok = m < g.M && k < K;
                    ra[i] = a[ok ? m * g.sam + k * g.sak : 0];
                    amask |= (uint32_t)ok << i;
                }
                {
                    const int kk = idx / BN, col = idx % BN;
                    const int64_t k = k0 + kk, n = n0 + col;
                    const bool ok = k < K && n < g.N;
                    rb[i] = b[ok ? k * g.sbk + n * g.sbn : 0];
                    bmask |= (uint32_t)ok << i;
                }
            }
            return kScalar;
        }
    };
    auto store_tiles = [&](int buf, int where) {
        if (where == kVec) {
            constexpr int V = 16 / (int)sizeof(T);
            constexpr int APT = (BM * BK) / (kBlock * V);
            constexpr int KV = BK / V;
#pragma unroll
            for (int i = 0; i < APT; i++) {
                const int idx = tid + i * kBlock;
                const int row = idx / KV, kv = (idx % KV) * V;
#pragma unroll
                for (int e = 0; e < V; e++) As[buf][kv + e][row] = ra[i * V + e];
            }
            constexpr int NV = BN / V;
#pragma unroll
            for (int i = 0; i < APT; i++) {
                const int idx = tid + i * kBlock;
                const int kk = idx / NV, nv = (idx % NV) * V;
                // one 16-byte LDS store (element stores of this pattern collide four ways on the banks)
                Pack<T, V> v;
#pragma unroll
                for (int e = 0; e < V; e++) v.v[e] = rb[i * V + e];
                typename RawWord<16>::type w;
                __builtin_memcpy(&w, &v, 16);
                *reinterpret_cast<typename RawWord<16>::type*>(&Bs[buf][kk][nv]) = w;
            }
        } else if (!LEAN && where == kScalar) {
#pragma unroll
            for (int i = 0; i < SPT; i++) {
                const int idx = tid + i * kBlock;
                As[buf][idx % BK][idx / BK] = ((amask >> i) & 1u) ? ra[i] : T(0);
                Bs[buf][idx / BN][idx % BN] = ((bmask >> i) & 1u) ? rb[i] : T(0);
            }
        }
    };

    const int wave = tid >> 6, lane = tid & 63;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;

    if constexpr (std::is_same<T, float>::value) {
        f32x16 acc[2][2];
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    // accumulate mode starts from the target's values, fetched while the first tiles arrive: the epilogue is then a
                    // plain store instead of 64 read-modify-write round trips per lane
                    acc[i][j][r] = 0.f;
                    if constexpr (ACC) {
                        const int64_t m = m0 + wm + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                        const int64_t n = n0 + wn + j * 32 + (lane & 31);
                        if (full_mn || (m < g.M && n < g.N)) acc[i][j][r] = c[m * g.scm + n * g.scn];
                    }
                }

        int vl = kDirect;
        if (FAST || K > 0) {  // (the fast kernel is only launched with K > 0) an empty inner dimension has no element to fetch (not even the clamped one): the target becomes zeros
            vl = load_tiles(0, 0);
            store_tiles(0, vl);
        }
        __syncthreads();
        int cur = 0;
        const int lk = lane >> 5, lm = lane & 31;
        for (int64_t k0 = 0; k0 < K; k0 += BK) {
            const bool more = k0 + BK < K;
            if (more) vl = load_tiles(k0 + BK, cur ^ 1);
            // Operand reads stay interleaved with the MFMAs (four per pair of LDS reads): hoisting all 32 reads of a K step
            // ahead of the MFMA chain costs 27 more registers, drops occupancy from 4 to 3 wavefronts per SIMD and measured
            // 6 % slower; with 4 wavefronts per SIMD the other wavefronts' MFMAs cover each LDS round trip.
#pragma unroll
            for (int kk = 0; kk < BK; kk += 2) {
                const float a0 = As[cur][kk + lk][wm + lm];
                const float a1 = As[cur][kk + lk][wm + 32 + lm];
                const float b0 = Bs[cur][kk + lk][wn + lm];
                const float b1 = Bs[cur][kk + lk][wn + 32 + lm];
                acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
                acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
                acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
                acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
                // FAST kernel: the next step's tiles go to the other LDS buffer inside the MFMA chain (their loads were issued a
                // thousand cycles earlier), so only the barrier is left at the end of the step: +2-7 % (the four wavefronts of
                // a SIMD run in phase, so whatever follows the last MFMA of a step leaves the matrix pipe idle).  The general
                // kernel, whose element loads take longer to arrive, measured 5 % slower that way and stores at the end.
                if (FAST && kk == 4 && more) store_tiles(cur ^ 1, vl);
            }
            if (more) {
                if (!FAST) store_tiles(cur ^ 1, vl);
                __syncthreads();
                cur ^= 1;
            }
        }
        // accumulator register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32 of its 32x32 tile
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int64_t m = m0 + wm + i * 32 + (r >> 2) * 8 + lk * 4 + (r & 3);
                    const int64_t n = n0 + wn + j * 32 + lm;
                    if (full_mn || (m < g.M && n < g.N)) {
                        T* dst = c + m * g.scm + n * g.scn;
                        *dst = acc[i][j][r];
                    }
                }
    } else {
        // fp64: sixteen 16x16 accumulators per wavefront on v_mfma_f64_16x16x4_f64.  Operand lane l supplies A[l%16][l/16] and
        // B[l/16][l%16]; accumulator register r of lane l holds row 4*r + l/16, column l%16 of its 16x16 tile.
        f64x4 acc[4][4];
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    acc[i][j][r] = 0.0;
                    if constexpr (ACC) {   // as for single precision: start from the target's values
                        const int64_t m = m0 + wm + i * 16 + 4 * r + (lane >> 4), n = n0 + wn + j * 16 + (lane & 15);
                        if (full_mn || (m < g.M && n < g.N)) acc[i][j][r] = c[m * g.scm + n * g.scn];
                    }
                }
        int vl = kDirect;
        if (FAST || K > 0) {  // (the fast kernel is only launched with K > 0) an empty inner dimension has no element to fetch (not even the clamped one): the target becomes zeros
            vl = load_tiles(0, 0);
            store_tiles(0, vl);
        }
        __syncthreads();
        int cur = 0;
        const int lk = lane >> 4, lm = lane & 15;
        for (int64_t k0 = 0; k0 < K; k0 += BK) {
            const bool more = k0 + BK < K;
            if (more) vl = load_tiles(k0 + BK, cur ^ 1);
#pragma unroll
            for (int kk = 0; kk < BK; kk += 4) {
                double av[4], bv[4];
#pragma unroll
                for (int i = 0; i < 4; i++) av[i] = As[cur][kk + lk][wm + i * 16 + lm];
#pragma unroll
                for (int j = 0; j < 4; j++) bv[j] = Bs[cur][kk + lk][wn + j * 16 + lm];
#pragma unroll
                for (int i = 0; i < 4; i++)
#pragma unroll
                    for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(av[i], bv[j], acc[i][j], 0, 0, 0);
            }
            if (more) {
                store_tiles(cur ^ 1, vl);   // storing inside the MFMA chain (as the fp32 path does) measured no gain for fp64
                __syncthreads();
                cur ^= 1;
            }
        }
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int64_t m = m0 + wm + i * 16 + 4 * r + lk, n = n0 + wn + j * 16 + lm;
                    if (full_mn || (m < g.M && n < g.N)) {
                        T* dst = c + m * g.scm + n * g.scn;
                        *dst = acc[i][j][r];
                    }
                }
    }
}

// Split K.  A product with few output tiles leaves most of the 256 CUs idle (1000 x 1000 x 1000 has 64 tiles), and the one block a
// CU does get runs a long K loop with nothing to overlap its loads; a tile count just above a multiple of what the chip holds
// (3000^3: 576 tiles on 1024 block slots) wastes most of its last round.  Such a product is cut along K into `splits` chunks
// that run as one more (innermost) batch dimension, each writing an M x N partial to the stream's workspace;
// gemm_split_finish_kernel adds the partials in chunk order (deterministic, no float atomics) and stores, or accumulates into,
// the target through its strides.
//
// The number of chunks minimises a cost model fitted to measurements on MI355X.  A CU that holds r blocks at once takes
// t(r) = t0 + t1 * r microseconds per K step (fp32, K step 16: 1.9 us for one block, 5.2 us for four; fp64, K step 8: 2.0 us and
// 2.5 us for two), a block costs about 2.7 K steps of prologue and epilogue, and the partials cost one launch plus their bytes
// written and read back at about 5 TB/s.  The model reproduces 1000^3, 2000^3 and 3000^3 at 1 to 16 chunks within 6 %.
template <class T>
int64_t choose_k_splits(int64_t blocks, int64_t steps, int64_t out_elems) {
    constexpr int R = sizeof(T) == 4 ? 4 : 2;                      // blocks a CU holds (registers and LDS)
    constexpr double t0 = sizeof(T) == 4 ? 0.8 : 1.44, t1 = sizeof(T) == 4 ? 1.1 : 0.53;
    constexpr int64_t kMinSteps = 4;
    const int64_t cus = device_cus();
    const int64_t max_splits = steps / kMinSteps;
    if (max_splits < 2) return 1;                                  // also the empty inner dimension (no steps)
    auto cost = [&](int64_t sp) {
        const int64_t chunk = (steps + sp - 1) / sp;
        const int64_t real = (steps + chunk - 1) / chunk;          // chunks that are not empty
        const int64_t per_cu = (blocks * real + cus - 1) / cus;
        const int64_t rest = per_cu % R;
        const double step_us = (double)(per_cu / R) * (t0 + t1 * R) + (rest ? t0 + t1 * (double)rest : 0.0);
        double us = step_us * ((double)chunk + 2.7);
        if (real > 1) us += 3.0 + (double)real * (double)out_elems * sizeof(T) * 2.0 / 5.0e6;
        return us;
    };
    int64_t best = 1;
    double best_us = cost(1);
    for (int64_t k = 1; k <= 16; k++) {                            // the largest chunk count that keeps k blocks per CU
        const int64_t sp = std::min(max_splits, cus * k / blocks);
        if (sp < 2) continue;
        const double us = cost(sp);
        if (us < best_us * 0.97) {                                 // a split must pay for itself
            best_us = us;
            best = sp;
        }
    }
    return best;
}

// One wavefront covers 64 consecutive output vectors of VEC elements (coalesced along n); the SG wavefronts of a block take the
// chunks s = w, w + SG, ... of those outputs, and wavefront 0 adds the SG sums in index order: the result depends on
// (splits, SG) only.  VEC > 1 needs N % VEC == 0 and a target whose rows are contiguous and 16-byte aligned.
template <class T, bool ACC, int SG, int VEC>
__global__ __launch_bounds__(64 * SG) void gemm_split_finish_kernel(T* __restrict__ c, const T* __restrict__ ws, GemmArgs g, uint32_t splits, uint32_t total_vecs) {
    __shared__ Pack<T, VEC> red[SG][64];
    const uint32_t lane = threadIdx.x % 64u, w = threadIdx.x / 64u;
    const uint32_t e = blockIdx.x * 64u + lane;
    const uint32_t NV = (uint32_t)g.N / VEC, M = (uint32_t)g.M;
    const uint32_t n = (e % NV) * VEC, r = e / NV, m = r % M;
    uint32_t bl = r / M;
    Pack<T, VEC> sum = splat_pack<T, VEC>(T(0));
    if (e < total_vecs) {
        const size_t mn = (size_t)M * (size_t)g.N;
        const T* p = ws + ((size_t)bl * splits * M + m) * (size_t)g.N + n;
        for (uint32_t s = w; s < splits; s += SG) {
            const Pack<T, VEC> v = load_pack<T, VEC>(p + s * mn);
#pragma unroll
            for (int k = 0; k < VEC; k++) sum.v[k] += v.v[k];
        }
    }
    red[w][lane] = sum;
    __syncthreads();
    if (w != 0 || e >= total_vecs) return;
#pragma unroll
    for (int i = 1; i < SG; i++)
#pragma unroll
        for (int k = 0; k < VEC; k++) sum.v[k] += red[i][lane].v[k];
    int64_t oc = (int64_t)m * g.scm + (int64_t)n * g.scn;
    for (int d = g.nbatch - 1; d >= 0; d--) {
        const uint32_t q = (d == 0) ? 0u : bl / g.bshape[d];
        oc += (int64_t)(bl - q * g.bshape[d]) * g.bsc[d];
        bl = q;
    }
    if constexpr (VEC > 1) {
        if (ACC) {
            const Pack<T, VEC> old = load_pack<T, VEC>(c + oc);
#pragma unroll
            for (int k = 0; k < VEC; k++) sum.v[k] = old.v[k] + sum.v[k];
        }
        store_pack<T, VEC>(c + oc, sum);
    } else {
        c[oc] = ACC ? c[oc] + sum.v[0] : sum.v[0];
    }
}

// ---- single precision on the bf16 matrix instructions ----------------------------------------------------------------------
// v_mfma_f32_32x32x16_bf16 runs 16 times the rate of v_mfma_f32_32x32x2_f32.  A float is the exact sum of three bf16 numbers
// (its 24 significant bits cut into 8 + 8 + 8 by truncation: hi = the upper 16 bits of a, mid = those of a - hi, lo = those of
// a - hi - mid, every difference exact), so a.b = sum of nine bf16 products, each exact in the instruction's fp32 accumulator.
// The six largest are kept: hi.hi, hi.mid, mid.hi, hi.lo, lo.hi, mid.mid; the three dropped (mid.lo, lo.mid, lo.lo) are below
// 2^-21 |a||b|, usually 2^-25, i.e. a few units of the rounding of one fp32 product, against a contract of K of them.  Six bf16
// instructions of K = 16 replace eight fp32 instructions of K = 2 per 32 x 32 x 16 block: 2.7 times fewer matrix-pipe cycles.
// The cut is exact only for finite elements whose parts are representable: an infinite element would give inf - inf = NaN in its
// mid part, and below 2^-109 the lo part (lowest bit 2^(e-23)) falls under the smallest bf16 denormal, 2^-133.  Every staged element
// is therefore classified (one multiply by 2^-17 and one class test: infinite, or denormal after the scaling); a workgroup that has
// met such an element in its rows of A or columns of B recomputes its tile with the fp32 matrix instruction (fp32_tile_fallback:
// IEEE products and sums, inf x finite = inf, inf x 0 = NaN, as the reference's sgemm).  NaN needs no fallback: one part of a NaN is
// a NaN.  Products with K < 16 (no whole K step; worst case 8 u per product from the three dropped terms against 1 u of one
// rounded fp32 product) stay on the fp32 instructions.  The option dot_bf16x3 = 0 keeps every product there.
// Every operand that is contiguous along one of its two dimensions (row-major or transposed; 16-byte aligned rows when k is the
// contiguous one), K splits included; accumulating products and operands strided in both dimensions take gemm_kernel.
// Two forms: 128 x 128 tiles, 256 threads, two workgroups per CU (gemm_bf16x3_kernel: every size, K splits), and 256 x 256 tiles,
// 512 threads, one workgroup per CU (gemm_bf16x3_big_kernel: half the staging and LDS traffic per matrix instruction; taken when
// the product has about a CU's worth of such tiles, use_big_tiles; the option dot_big = 0 / 1 forces the choice).
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr int kX3BK = 16;
constexpr int kX3Row = 24;   // bf16 per LDS row: 16 of data + 8 of padding (48 bytes: 16-byte reads of 16 consecutive rows hit all banks once)

// Splits eight floats into their hi / mid / lo bf16 parts, packed as 8 x bf16 = 16 bytes each.
__device__ __forceinline__ void split3_bf16(const float (&v)[8], u32x4& hi, u32x4& mid, u32x4& lo) {
    uint32_t h[8], m[8], l[8];   // the part sits in the upper 16 bits of each word
#pragma unroll
    for (int e = 0; e < 8; e++) {
        h[e] = __float_as_uint(v[e]);
        const float r1 = v[e] - __uint_as_float(h[e] & 0xFFFF0000u);
        m[e] = __float_as_uint(r1);
        const float r2 = r1 - __uint_as_float(m[e] & 0xFFFF0000u);
        l[e] = __float_as_uint(r2);
    }
    // one byte permute packs the upper halves of two words: result = {x1[31:16], x0[31:16]}
#pragma unroll
    for (int e = 0; e < 4; e++) {
        hi[e] = __builtin_amdgcn_perm(h[2 * e + 1], h[2 * e], 0x07060302u);
        mid[e] = __builtin_amdgcn_perm(m[2 * e + 1], m[2 * e], 0x07060302u);
        lo[e] = __builtin_amdgcn_perm(l[2 * e + 1], l[2 * e], 0x07060302u);
    }
}

// Staging of one operand tile (ROWS rows x 16 k; "row" is m for A and n for B) by 2 * ROWS threads from memory into the three bf16 tiles in LDS.
//   KC: k is the contiguous direction.  Four lanes cover the 16 k of a row with one 16-byte load each (a wavefront reads 16 rows of
//       64 contiguous bytes); a thread takes the same 4 k of rows r and r + ROWS / 2 and writes 8 bytes per part and row.
//   otherwise the rows are contiguous (row-major B, transposed A): a thread takes one row and 8 consecutive k with element loads
//       (the lanes of a wavefront read 256 consecutive bytes) and writes 16 bytes per part.
template <bool KC, int ROWS = BM>
struct X3Stage {
    static constexpr int HALF = ROWS / 2;   // 2 * ROWS threads stage a tile
    int row, kofs;      // first row and first k of this thread inside the tile
    // element (row, k = 0) of this thread's rows (KC: row and row + ROWS / 2).  A row beyond the matrix reads row 0 instead: what it
    // contributes lands in rows (columns) of the tile's result that lie beyond the matrix as well and are never stored.
    const float *p0, *p1;
    int64_t ks;
    bool bad;           // an element staged so far is infinite or too small to cut into bf16 parts
    __device__ __forceinline__ void init(const float* base, int64_t row0, int64_t limit, int64_t rs, int64_t kstride, int tid) {
        row = KC ? tid >> 2 : tid & (ROWS - 1);
        kofs = KC ? (tid & 3) * 4 : (tid / ROWS) * 8;
        p0 = base + (row0 + row < limit ? (row0 + row) * rs : 0);
        p1 = base + (KC && row0 + row + HALF < limit ? (row0 + row + HALF) * rs : 0);
        ks = KC ? 1 : kstride;
        bad = false;
    }
    template <bool TAIL>
    __device__ __forceinline__ void load(int64_t k0, int64_t K, float (&r)[8]) const {
        if (!TAIL || k0 + kX3BK <= K) {
            if constexpr (KC) {
                // plain (temporal) 16-byte loads: the other half of each 128-byte line is wanted at the next K step and by the
                // workgroups of the same tile row (load_pack's non-temporal loads measured 2.5-4 % slower at 4000^3 / 4096^3)
                typedef float f32x4v __attribute__((ext_vector_type(4), aligned(4)));   // any dword address (rows of views that start at odd elements)
                const f32x4v v0 = *reinterpret_cast<const f32x4v*>(p0 + k0 + kofs), v1 = *reinterpret_cast<const f32x4v*>(p1 + k0 + kofs);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    r[e] = v0[e];
                    r[4 + e] = v1[e];
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) r[e] = p0[(k0 + kofs + e) * ks];
            }
        } else {
            // TAIL (K is not a multiple of 16): the last, partial K step takes element loads from addresses clamped into the row, zeros beyond K
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int64_t k = k0 + kofs + (KC ? (e & 3) : e);
                const float* p = (KC && e >= 4) ? p1 : p0;
                const float v = p[(k < K ? k : K - 1) * ks];
                r[e] = k < K ? v : 0.0f;
            }
        }
    }
    // cuts the staged elements into their parts and writes them to tile[part][row][k]
    __device__ __forceinline__ void store(float (&r)[8], __bf16 (*tile)[ROWS][kX3Row]) {
        // +-inf stays infinite under the scaling; 2^-126 <= |x| < 2^-109 becomes denormal; zero stays zero.  An element that is
        // denormal already is tested as it is: scaled, the smallest ones (|x| <= 2^-133) would round to zero and pass for zeros.
        constexpr int kClassInfOrDenormal = (1 << 2) | (1 << 4) | (1 << 7) | (1 << 9), kClassDenormal = (1 << 4) | (1 << 7);
#pragma unroll
        for (int e = 0; e < 8; e++)
            bad |= __builtin_amdgcn_classf(r[e] * 0x1p-17f, kClassInfOrDenormal) | __builtin_amdgcn_classf(r[e], kClassDenormal);
        u32x4 part[3];
        split3_bf16(r, part[0], part[1], part[2]);
#pragma unroll
        for (int s = 0; s < 3; s++) {
            if constexpr (KC) {
                typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
                *reinterpret_cast<u32x2*>(&tile[s][row][kofs]) = u32x2{part[s][0], part[s][1]};
                *reinterpret_cast<u32x2*>(&tile[s][row + HALF][kofs]) = u32x2{part[s][2], part[s][3]};
            } else {
                *reinterpret_cast<u32x4*>(&tile[s][row][kofs]) = part[s];
            }
        }
    }
    // The same work as store() in 16 pieces of a few instructions each, for a caller that places them between its matrix instructions:
    // piece 2e cuts element e, piece 2e + 1 classifies it, packs a finished pair and writes finished groups to LDS.
    uint32_t hw[2], mw[2], lw[2];
    u32x4 part[3];
    template <int Q>
    __device__ __forceinline__ void piece(float (&r)[8], __bf16 (*tile)[ROWS][kX3Row]) {
        constexpr int e = Q / 2;
        if constexpr (Q % 2 == 0) {
            const float v = r[e];
            const uint32_t h = __float_as_uint(v);
            const float r1 = v - __uint_as_float(h & 0xFFFF0000u);
            const uint32_t m = __float_as_uint(r1);
            const float r2 = r1 - __uint_as_float(m & 0xFFFF0000u);
            hw[e & 1] = h;
            mw[e & 1] = m;
            lw[e & 1] = __float_as_uint(r2);
        } else {
            constexpr int kClassInfOrDenormal = (1 << 2) | (1 << 4) | (1 << 7) | (1 << 9), kClassDenormal = (1 << 4) | (1 << 7);
            bad |= __builtin_amdgcn_classf(r[e] * 0x1p-17f, kClassInfOrDenormal) | __builtin_amdgcn_classf(r[e], kClassDenormal);
            if constexpr (e % 2 == 1) {
                part[0][e / 2] = __builtin_amdgcn_perm(hw[1], hw[0], 0x07060302u);
                part[1][e / 2] = __builtin_amdgcn_perm(mw[1], mw[0], 0x07060302u);
                part[2][e / 2] = __builtin_amdgcn_perm(lw[1], lw[0], 0x07060302u);
            }
            if constexpr (KC && e % 4 == 3) {
                typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
#pragma unroll
                for (int s = 0; s < 3; s++)
                    *reinterpret_cast<u32x2*>(&tile[s][row + (e / 4) * HALF][kofs]) = u32x2{part[s][e / 2 - 1], part[s][e / 2]};
            }
            if constexpr (!KC && e == 7) {
#pragma unroll
                for (int s = 0; s < 3; s++) *reinterpret_cast<u32x4*>(&tile[s][row][kofs]) = part[s];
            }
        }
    }
};

template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) { (f(std::integral_constant<int, I>()), ...); }
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) { static_for_impl(f, std::make_integer_sequence<int, N>()); }

// One 128 x 128 tile of c = a . b over k in [0, K) on v_mfma_f32_32x32x2_f32, operands fetched element by element through their
// strides: the slow, IEEE-faithful path of a workgroup of gemm_bf16x3_kernel whose operands hold infinite or very small elements.
// A32 / B32: [16][BM + PAD] floats of LDS each; every thread of the block calls it.
// tid: 0..255, the thread's number among the 256 that share this tile (a larger workgroup runs several tiles side by side, each group
// with its own A32 / B32; the barriers are the whole workgroup's, so every group must make the same number of K steps).
__device__ __forceinline__ void fp32_tile_fallback(float* c, const float* a, const float* b, const GemmArgs& g, int64_t m0, int64_t n0, int64_t K,
                                                float (*A32)[BM + PAD], float (*B32)[BN + PAD], int tid) {
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64, lk = lane >> 5, lm = lane & 31;
    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;
    for (int64_t k0 = 0; k0 < K; k0 += 16) {
        __syncthreads();   // the previous step's operand reads (and, on entry, the caller's use of the memory) are over
#pragma unroll 2
        for (int i = 0; i < BM * 16 / kBlock; i++) {
            const int idx = tid + i * kBlock;
            {
                const int row = idx / 16, kk = idx % 16;
                const int64_t m = m0 + row, k = k0 + kk;
                A32[kk][row] = (m < g.M && k < K) ? a[m * g.sam + k * g.sak] : 0.0f;
            }
            {
                const int kk = idx / BN, col = idx % BN;
                const int64_t k = k0 + kk, n = n0 + col;
                B32[kk][col] = (k < K && n < g.N) ? b[k * g.sbk + n * g.sbn] : 0.0f;
            }
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 16; kk += 2) {
            const float a0 = A32[kk + lk][wm + lm], a1 = A32[kk + lk][wm + 32 + lm];
            const float b0 = B32[kk + lk][wn + lm], b1 = B32[kk + lk][wn + 32 + lm];
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
        }
    }
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int64_t m = m0 + wm + i * 32 + (r >> 2) * 8 + lk * 4 + (r & 3);
                const int64_t n = n0 + wn + j * 32 + lm;
                if (m < g.M && n < g.N) c[m * g.scm + n * g.scn] = acc[i][j][r];
            }
}

template <bool SPLIT, bool TAIL, bool A_KC, bool B_KC>
__global__ __launch_bounds__(kBlock, 2) void gemm_bf16x3_kernel(float* __restrict__ c, const float* __restrict__ a, const float* __restrict__ b, GemmArgs g) {
    __shared__ __align__(16) __bf16 As[2][3][BM][kX3Row];
    __shared__ __align__(16) __bf16 Bs[2][3][BN][kX3Row];

    uint32_t bid = blockIdx.x, tm, tn;
    if (g.xcd_2d) {
        // one matrix: XCD x (workgroup ids are dealt round-robin) takes region (x / 4, x % 4) of a 2 x 4 grid of regions, row-major inside,
        // so that the workgroups running together on an XCD share few A and B panels (a region of 16 x 8 tiles: 8 + 8 panels for 64
        // workgroups instead of 2 + 32 with whole tile rows)
        const uint32_t xcd = bid % 8u, local = bid / 8u, regw = g.tiles_n / 4u, regh = g.tiles_m / 2u;
        tm = (xcd / 4u) * regh + local / regw;
        tn = (xcd % 4u) * regw + local % regw;
        bid = 0;
    } else {
        if (g.xcd_chunk) bid = (bid % 8u) * g.xcd_chunk + bid / 8u;
        tn = bid % g.tiles_n;
        bid /= g.tiles_n;
        tm = bid % g.tiles_m;
        bid /= g.tiles_m;
    }
    int64_t oa = 0, ob = 0, oc = 0;
    uint32_t chunk_id = 0;
    for (int d = g.nbatch - 1; d >= 0; d--) {
        const uint32_t q = (d == 0) ? 0u : bid / g.bshape[d];
        const uint32_t i = bid - q * g.bshape[d];
        bid = q;
        oa += (int64_t)i * g.bsa[d];
        ob += (int64_t)i * g.bsb[d];
        oc += (int64_t)i * g.bsc[d];
        if (SPLIT && d == g.nbatch - 1) chunk_id = i;
    }
    // this block's extent along k: the whole of K, or one chunk of it (SPLIT: the innermost batch dimension counts the chunks)
    const int64_t K = SPLIT ? min(g.kchunk, g.K - (int64_t)chunk_id * g.kchunk) : g.K;
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
    a += oa;
    b += ob;
    c += oc;
    const int tid = threadIdx.x;

    X3Stage<A_KC> sa;
    X3Stage<B_KC> sb;
    sa.init(a, m0, g.M, g.sam, g.sak, tid);
    sb.init(b, n0, g.N, g.sbn, g.sbk, tid);
    float ra[8], rb[8];

    const int wave = tid >> 6, lane = tid & 63;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
    const int lm = lane & 31, lk = lane >> 5;
    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    // One K step: the 24 matrix instructions of the tiles in LDS buffer cur and, when NEXT, the fetch of the next step's elements
    // (first), their cutting into parts and the writes to the other buffer (32 pieces, X3Stage::piece, two behind each of the last 16
    // matrix instructions).  The order is pinned by scheduling barriers: left alone, the compiler puts the fetches after most of the
    // matrix instructions and the cutting after all of them, and each wavefront waits for memory with the matrix pipe idle.
    int cur = 0;
    auto k_step = [&](auto next_tag, auto tail_tag, int64_t k_next) {
        constexpr bool NEXT = decltype(next_tag)::value, TL = decltype(tail_tag)::value;
        if constexpr (NEXT) {
            sa.template load<TL>(k_next, K, ra);
            sb.template load<TL>(k_next, K, rb);
        }
        __builtin_amdgcn_sched_barrier(0);
        bf16x8 av[2][3], bv[2][3];
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int s = 0; s < 3; s++) bv[j][s] = *reinterpret_cast<const bf16x8*>(&Bs[cur][s][wn + j * 32 + lm][lk * 8]);
#pragma unroll
        for (int s = 0; s < 3; s++) av[0][s] = *reinterpret_cast<const bf16x8*>(&As[cur][s][wm + lm][lk * 8]);
        __builtin_amdgcn_sched_barrier(0);
        static_for<24>([&](auto tt) {
            constexpr int t = decltype(tt)::value, i = t / 12, j = (t % 12) / 6, p = t % 6;
            constexpr int pa = p == 0 ? 1 : p == 1 ? 0 : p == 2 ? 2 : p == 3 ? 0 : p == 4 ? 1 : 0;   // smallest products first
            constexpr int pb = p == 0 ? 1 : p == 1 ? 2 : p == 2 ? 0 : p == 3 ? 1 : p == 4 ? 0 : 0;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[i][pa], bv[j][pb], acc[i][j], 0, 0, 0);
            if constexpr (t < 3) av[1][t] = *reinterpret_cast<const bf16x8*>(&As[cur][t][wm + 32 + lm][lk * 8]);
            if constexpr (NEXT && t >= 8) {
                constexpr int q = (t - 8) * 2;
                if constexpr (q < 16) {
                    sa.template piece<q>(ra, As[cur ^ 1]);
                    sa.template piece<q + 1>(ra, As[cur ^ 1]);
                } else {
                    sb.template piece<q - 16>(rb, Bs[cur ^ 1]);
                    sb.template piece<q - 15>(rb, Bs[cur ^ 1]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        if constexpr (NEXT) {
            __syncthreads();
            cur ^= 1;
        }
    };
    const int64_t nsteps = (K + kX3BK - 1) / kX3BK;
    sa.template load<TAIL>(0, K, ra);
    sb.template load<TAIL>(0, K, rb);
    sa.store(ra, As[0]);
    sb.store(rb, Bs[0]);
    __syncthreads();
    // K steps 1 .. nsteps - 2 are whole; the last one may be partial (TAIL)
    for (int64_t s = 0; s + 2 < nsteps; s++) k_step(std::true_type(), std::false_type(), (s + 1) * kX3BK);
    if (nsteps >= 2) k_step(std::true_type(), std::integral_constant<bool, TAIL>(), (nsteps - 1) * kX3BK);
    k_step(std::false_type(), std::false_type(), 0);
    // an element that cannot be cut into bf16 parts was staged by some thread: the whole tile is redone on the fp32 instruction
    if (__syncthreads_or((int)(sa.bad | sb.bad))) {
        fp32_tile_fallback(c, a, b, g, m0, n0, K, reinterpret_cast<float (*)[BM + PAD]>(&As[0][0][0][0]),
                           reinterpret_cast<float (*)[BN + PAD]>(&Bs[0][0][0][0]), tid);
        return;
    }
    // accumulator register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32 of its 32x32 tile
    const bool full_mn = m0 + BM <= g.M && n0 + BN <= g.N;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int64_t m = m0 + wm + i * 32 + (r >> 2) * 8 + lk * 4 + (r & 3);
                const int64_t n = n0 + wn + j * 32 + lm;
                if (full_mn || (m < g.M && n < g.N)) c[m * g.scm + n * g.scn] = acc[i][j][r];
            }
}

// The same product on 256 x 256 tiles: 512 threads = 8 wavefronts in a 2 x 4 arrangement, each owning 128 x 64 (eight 32 x 32
// accumulators).  Against the 128 x 128 kernel every staged element (cut into parts once per workgroup that needs it) and every LDS
// operand fetch feeds twice as many matrix instructions: 48 per wavefront and K step against 18 LDS reads and 16 staged elements.
// One workgroup per CU (144 KB of LDS, two wavefronts per SIMD); choose_plan picks the form (and the chunks along K) per product.
// The K loop keeps one shape per iteration (no branch inside: the last K step and the K tail are peeled), so that the cutting of the
// next step's elements can be scheduled between the matrix instructions of the current one.
constexpr int XBM = 256, XBN = 256, kBigThreads = 512;
constexpr size_t kBigLdsBytes = (size_t)2 * 2 * 3 * XBM * kX3Row * sizeof(__bf16);

template <bool SPLIT, bool TAIL, bool A_KC, bool B_KC>
__global__ __launch_bounds__(kBigThreads) void gemm_bf16x3_big_kernel(float* c, const float* a, const float* b, GemmArgs g) {
    extern __shared__ __align__(16) unsigned char x3_lds[];
    typedef __bf16 (*Tiles)[3][XBM][kX3Row];                      // [buffer][part][row][k]
    Tiles As = reinterpret_cast<Tiles>(x3_lds);
    Tiles Bs = reinterpret_cast<Tiles>(x3_lds + kBigLdsBytes / 2);

    uint32_t bid = blockIdx.x, tm, tn;
    if (g.xcd_2d) {
        const uint32_t xcd = bid % 8u, local = bid / 8u, regw = g.tiles_n / 4u, regh = g.tiles_m / 2u;
        tm = (xcd / 4u) * regh + local / regw;
        tn = (xcd % 4u) * regw + local % regw;
        bid = 0;
    } else {
        if (g.xcd_chunk) bid = (bid % 8u) * g.xcd_chunk + bid / 8u;
        tn = bid % g.tiles_n;
        bid /= g.tiles_n;
        tm = bid % g.tiles_m;
        bid /= g.tiles_m;
    }
    int64_t oa = 0, ob = 0, oc = 0;
    uint32_t chunk_id = 0;
    for (int d = g.nbatch - 1; d >= 0; d--) {
        const uint32_t q = (d == 0) ? 0u : bid / g.bshape[d];
        const uint32_t i = bid - q * g.bshape[d];
        bid = q;
        oa += (int64_t)i * g.bsa[d];
        ob += (int64_t)i * g.bsb[d];
        oc += (int64_t)i * g.bsc[d];
        if (SPLIT && d == g.nbatch - 1) chunk_id = i;
    }
    // this block's extent along k: the whole of K, or one chunk of it (SPLIT: the innermost batch dimension counts the chunks)
    const int64_t K = SPLIT ? min(g.kchunk, g.K - (int64_t)chunk_id * g.kchunk) : g.K;
    const int64_t m0 = (int64_t)tm * XBM, n0 = (int64_t)tn * XBN;
    a += oa;
    b += ob;
    c += oc;
    const int tid = threadIdx.x;

    X3Stage<A_KC, XBM> sa;
    X3Stage<B_KC, XBN> sb;
    sa.init(a, m0, g.M, g.sam, g.sak, tid);
    sb.init(b, n0, g.N, g.sbn, g.sbk, tid);
    float ra[8], rb[8];

    const int wave = tid >> 6, lane = tid & 63;
    const int wm = (wave >> 2) * 128, wn = (wave & 3) * 64;
    const int lm = lane & 31, lk = lane >> 5;
    f32x16 acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    // the matrix instructions of one K step on LDS buffer `buf`
    auto compute = [&](int buf) {
        bf16x8 bv[2][3];
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int s = 0; s < 3; s++) bv[j][s] = *reinterpret_cast<const bf16x8*>(&Bs[buf][s][wn + j * 32 + lm][lk * 8]);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            bf16x8 av[3];
#pragma unroll
            for (int s = 0; s < 3; s++) av[s] = *reinterpret_cast<const bf16x8*>(&As[buf][s][wm + i * 32 + lm][lk * 8]);
#pragma unroll
            for (int j = 0; j < 2; j++) {
                // smallest products first
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[1], bv[j][1], acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[0], bv[j][2], acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[2], bv[j][0], acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[0], bv[j][1], acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[1], bv[j][0], acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[0], bv[j][0], acc[i][j], 0, 0, 0);
            }
        }
    };

    // Elements are fetched two K steps ahead of the step that multiplies them: those of step s + 2 are requested in the middle of step s
    // (A) and near its end (B), cut into parts and written to the other LDS buffer during step s + 1, and multiplied in step s + 2, so
    // that a fetch has two thirds of a step (about 3000 cycles) to arrive before its first use.  The barrier at the end of a step
    // therefore has fetches in flight across it: it orders the LDS accesses only (lds_barrier), never the global ones.
    auto lds_barrier = [] {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    };
    const int64_t nsteps = (K + kX3BK - 1) / kX3BK;
    if (nsteps == 1) {
        sa.template load<TAIL>(0, K, ra);
        sb.template load<TAIL>(0, K, rb);
    } else {
        sa.template load<false>(0, K, ra);
        sb.template load<false>(0, K, rb);
    }
    sa.store(ra, As[0]);
    sb.store(rb, Bs[0]);
    if (nsteps == 2) {
        sa.template load<TAIL>(kX3BK, K, ra);
        sb.template load<TAIL>(kX3BK, K, rb);
    } else if (nsteps > 2) {
        sa.template load<false>(kX3BK, K, ra);
        sb.template load<false>(kX3BK, K, rb);
    }
    lds_barrier();
    int cur = 0;
    // One K step: multiply the current step's tiles, cut the elements fetched during the previous step into parts and write them to the
    // other buffer, request the elements of the step after the next (FETCH: 0 none, 1 whole K step, 2 the partial last one).  The
    // instruction order is pinned by scheduling barriers (left alone, the compiler puts the fetches after most of the matrix instructions
    // and the cutting after all of them: each wavefront then waits for memory with the matrix pipe idle): the LDS reads of B and of the
    // first 32 rows of A; then the 48 matrix instructions, the remaining LDS reads behind the first nine, the 16 pieces of cutting A
    // (X3Stage::piece) behind instructions 8-23, the request for A's next elements behind the 24th, B's pieces behind 24-39 and its
    // request behind the 40th.
    auto k_step = [&](auto fetch_tag, int64_t k_fetch) {
        constexpr int FETCH = decltype(fetch_tag)::value;
        __builtin_amdgcn_sched_barrier(0);
        bf16x8 av[4][3], bv[2][3];
        // In the order of first use (the first matrix instruction multiplies the mid parts, the second hi by lo, the third lo by hi),
        // the order pinned pair by pair: the eight wavefronts leave the barrier together and queue 72 reads of 1 KB at the LDS, so a
        // first instruction that needs two of its wavefront's reads starts some 400 cycles before one that needs eight.
        av[0][1] = *reinterpret_cast<const bf16x8*>(&As[cur][1][wm + lm][lk * 8]);
        bv[0][1] = *reinterpret_cast<const bf16x8*>(&Bs[cur][1][wn + lm][lk * 8]);
        __builtin_amdgcn_sched_barrier(0);
        av[0][0] = *reinterpret_cast<const bf16x8*>(&As[cur][0][wm + lm][lk * 8]);
        bv[0][2] = *reinterpret_cast<const bf16x8*>(&Bs[cur][2][wn + lm][lk * 8]);
        __builtin_amdgcn_sched_barrier(0);
        av[0][2] = *reinterpret_cast<const bf16x8*>(&As[cur][2][wm + lm][lk * 8]);
        bv[0][0] = *reinterpret_cast<const bf16x8*>(&Bs[cur][0][wn + lm][lk * 8]);
        __builtin_amdgcn_sched_barrier(0);
        bv[1][1] = *reinterpret_cast<const bf16x8*>(&Bs[cur][1][wn + 32 + lm][lk * 8]);
        bv[1][2] = *reinterpret_cast<const bf16x8*>(&Bs[cur][2][wn + 32 + lm][lk * 8]);
        bv[1][0] = *reinterpret_cast<const bf16x8*>(&Bs[cur][0][wn + 32 + lm][lk * 8]);
        __builtin_amdgcn_sched_barrier(0);
        static_for<48>([&](auto tt) {
            constexpr int t = decltype(tt)::value, i = t / 12, j = (t % 12) / 6, p = t % 6;
            constexpr int pa = p == 0 ? 1 : p == 1 ? 0 : p == 2 ? 2 : p == 3 ? 0 : p == 4 ? 1 : 0;   // smallest products first
            constexpr int pb = p == 0 ? 1 : p == 1 ? 2 : p == 2 ? 0 : p == 3 ? 1 : p == 4 ? 0 : 0;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[i][pa], bv[j][pb], acc[i][j], 0, 0, 0);
            if constexpr (t < 9) av[1 + t / 3][t % 3] = *reinterpret_cast<const bf16x8*>(&As[cur][t % 3][wm + (1 + t / 3) * 32 + lm][lk * 8]);
            if constexpr (t >= 8 && t < 24) sa.template piece<t - 8>(ra, As[cur ^ 1]);
            if constexpr (t >= 24 && t < 40) sb.template piece<t - 24>(rb, Bs[cur ^ 1]);
            if constexpr (t == 24 && FETCH != 0) sa.template load<FETCH == 2>(k_fetch, K, ra);
            if constexpr (t == 40 && FETCH != 0) sb.template load<FETCH == 2>(k_fetch, K, rb);
            __builtin_amdgcn_sched_barrier(0);
        });
        lds_barrier();
        cur ^= 1;
    };
    // step s (0 <= s <= nsteps - 2) cuts the elements of step s + 1 and requests those of step s + 2; the last request may be a partial step
    for (int64_t s = 0; s + 3 < nsteps; s++) k_step(std::integral_constant<int, 1>(), (s + 2) * kX3BK);
    if (nsteps >= 3) k_step(std::integral_constant<int, TAIL ? 2 : 1>(), (nsteps - 1) * kX3BK);
    if (nsteps >= 2) k_step(std::integral_constant<int, 0>(), 0);
    compute(cur);

    // an element that cannot be cut into bf16 parts was staged by some thread: the four 128 x 128 quarters of the tile are redone on the
    // fp32 instruction, two at a time (threads 0-255 take the upper two, threads 256-511 the lower two)
    if (__syncthreads_or((int)(sa.bad | sb.bad))) {
        const int grp = tid >> 8;
        float* lds = reinterpret_cast<float*>(x3_lds) + grp * 2 * 16 * (BM + PAD);
        for (int q = 0; q < 2; q++)
            fp32_tile_fallback(c, a, b, g, m0 + grp * 128, n0 + q * 128, K, reinterpret_cast<float (*)[BM + PAD]>(lds),
                               reinterpret_cast<float (*)[BN + PAD]>(lds + 16 * (BM + PAD)), tid & 255);
        return;
    }
    const bool full_mn = m0 + XBM <= g.M && n0 + XBN <= g.N;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int64_t m = m0 + wm + i * 32 + (r >> 2) * 8 + lk * 4 + (r & 3);
                const int64_t n = n0 + wn + j * 32 + lm;
                if (full_mn || (m < g.M && n < g.N)) c[m * g.scm + n * g.scn] = acc[i][j][r];
            }
}

bool use_bf16x3() {
    return option(OPT_DOT_BF16X3) != 0;
}

// ---- double precision with a pinned instruction order ------------------------------------------------------------------------
// The 128 x 128 tile of gemm_kernel<double> (K step 8, sixteen 16 x 16 accumulators per wavefront on v_mfma_f64_16x16x4_f64) for
// operands that are each contiguous along one of their two dimensions, with the loop written as the bf16-parts kernels write theirs:
// branch-free fetches of the next K step first (rows beyond the matrix read row 0; their products are never stored), then the 32
// matrix instructions with the second half's LDS reads behind the first eight and the LDS writes of the fetched elements behind the
// last sixteen, one barrier per step.  gemm_kernel keeps the other layouts and the accumulating form.
constexpr int kF64BK = 8;

// Staging of one operand tile (128 rows x 8 k) by 256 threads: four doubles per thread.
//   KC (k contiguous, 16-byte aligned rows): four lanes cover the 8 k of a row with one 16-byte load each; a thread takes rows r, r + 64.
//   otherwise (rows contiguous): a thread takes one row and 4 consecutive k with element loads (a wavefront reads 512 contiguous bytes).
template <bool KC>
struct F64Stage {
    int row, kofs;
    const double *p0, *p1;   // a row beyond the matrix reads row 0: its products land beyond the matrix too and are never stored
    int64_t ks;
    __device__ __forceinline__ void init(const double* base, int64_t row0, int64_t limit, int64_t rs, int64_t kstride, int tid) {
        row = KC ? tid >> 2 : tid & 127;
        kofs = KC ? (tid & 3) * 2 : (tid >> 7) * 4;
        p0 = base + (row0 + row < limit ? (row0 + row) * rs : 0);
        p1 = base + (KC && row0 + row + 64 < limit ? (row0 + row + 64) * rs : 0);
        ks = KC ? 1 : kstride;
    }
    template <bool TAIL>
    __device__ __forceinline__ void load(int64_t k0, int64_t K, double (&r)[4]) const {
        if (!TAIL || k0 + kF64BK <= K) {
            if constexpr (KC) {
                // (non-temporal loads; plain ones measured the same here)
                const Pack<double, 2> v0 = load_pack<double, 2>(p0 + k0 + kofs), v1 = load_pack<double, 2>(p1 + k0 + kofs);
                r[0] = v0.v[0];
                r[1] = v0.v[1];
                r[2] = v1.v[0];
                r[3] = v1.v[1];
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) r[e] = p0[(k0 + kofs + e) * ks];
            }
        } else {
            // the partial last K step: element loads from addresses clamped into the row, zeros beyond K
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int64_t k = k0 + kofs + (KC ? (e & 1) : e);
                const double* p = (KC && e >= 2) ? p1 : p0;
                const double v = p[(k < K ? k : K - 1) * ks];
                r[e] = k < K ? v : 0.0;
            }
        }
    }
    // element e of the staged four goes to tile[k][row]
    template <int E>
    __device__ __forceinline__ void put(const double (&r)[4], double (*tile)[BM + PAD]) const {
        const double v = r[E];
        if constexpr (KC) tile[kofs + (E & 1)][row + (E >> 1) * 64] = v;
        else tile[kofs + E][row] = v;
    }
    __device__ __forceinline__ void store(const double (&r)[4], double (*tile)[BM + PAD]) const {
        put<0>(r, tile);
        put<1>(r, tile);
        put<2>(r, tile);
        put<3>(r, tile);
    }
};

template <bool SPLIT, bool TAIL, bool A_KC, bool B_KC>
__global__ __launch_bounds__(kBlock, 2) void gemm_f64_kernel(double* c, const double* a, const double* b, GemmArgs g) {
    __shared__ __align__(16) double As[2][kF64BK][BM + PAD];
    __shared__ __align__(16) double Bs[2][kF64BK][BN + PAD];

    uint32_t bid = blockIdx.x;
    if (g.xcd_chunk) bid = (bid % 8u) * g.xcd_chunk + bid / 8u;
    const uint32_t tn = bid % g.tiles_n;
    bid /= g.tiles_n;
    const uint32_t tm = bid % g.tiles_m;
    bid /= g.tiles_m;
    int64_t oa = 0, ob = 0, oc = 0;
    uint32_t chunk_id = 0;
    for (int d = g.nbatch - 1; d >= 0; d--) {
        const uint32_t q = (d == 0) ? 0u : bid / g.bshape[d];
        const uint32_t i = bid - q * g.bshape[d];
        bid = q;
        oa += (int64_t)i * g.bsa[d];
        ob += (int64_t)i * g.bsb[d];
        oc += (int64_t)i * g.bsc[d];
        if (SPLIT && d == g.nbatch - 1) chunk_id = i;
    }
    const int64_t K = SPLIT ? min(g.kchunk, g.K - (int64_t)chunk_id * g.kchunk) : g.K;
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
    a += oa;
    b += ob;
    c += oc;
    const int tid = threadIdx.x;

    F64Stage<A_KC> sa;
    F64Stage<B_KC> sb;
    sa.init(a, m0, g.M, g.sam, g.sak, tid);
    sb.init(b, n0, g.N, g.sbn, g.sbk, tid);
    double ra[4], rb[4];

    // operand lane l supplies A[l % 16][l / 16] and B[l / 16][l % 16]; accumulator register r of lane l holds row 4 r + l / 16,
    // column l % 16 of its 16 x 16 tile
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
    const int lk = lane >> 4, lm = lane & 15;
    f64x4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int r = 0; r < 4; r++) acc[i][j][r] = 0.0;

    int cur = 0;
    auto k_step = [&](auto next_tag, auto tail_tag, int64_t k_next) {
        constexpr bool NEXT = decltype(next_tag)::value, TL = decltype(tail_tag)::value;
        if constexpr (NEXT) {
            sa.template load<TL>(k_next, K, ra);
            sb.template load<TL>(k_next, K, rb);
        }
        __builtin_amdgcn_sched_barrier(0);
        double av[2][4], bv[2][4];
#pragma unroll
        for (int i = 0; i < 4; i++) av[0][i] = As[cur][lk][wm + i * 16 + lm];
#pragma unroll
        for (int j = 0; j < 4; j++) bv[0][j] = Bs[cur][lk][wn + j * 16 + lm];
        __builtin_amdgcn_sched_barrier(0);
        static_for<32>([&](auto tt) {
            constexpr int t = decltype(tt)::value, h = t / 16, i = (t % 16) / 4, j = t % 4;
            acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(av[h][i], bv[h][j], acc[i][j], 0, 0, 0);
            if constexpr (t < 4) av[1][t] = As[cur][4 + lk][wm + t * 16 + lm];
            else if constexpr (t < 8) bv[1][t - 4] = Bs[cur][4 + lk][wn + (t - 4) * 16 + lm];
            if constexpr (NEXT && t >= 16 && t < 32 && t % 2 == 0) {
                constexpr int q = (t - 16) / 2;   // eight elements: four of A, four of B
                if constexpr (q < 4) sa.template put<q>(ra, As[cur ^ 1]);
                else sb.template put<q - 4>(rb, Bs[cur ^ 1]);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        if constexpr (NEXT) {
            __syncthreads();
            cur ^= 1;
        }
    };
    const int64_t nsteps = (K + kF64BK - 1) / kF64BK;
    sa.template load<TAIL>(0, K, ra);
    sb.template load<TAIL>(0, K, rb);
    sa.store(ra, As[0]);
    sb.store(rb, Bs[0]);
    __syncthreads();
    for (int64_t s = 0; s + 2 < nsteps; s++) k_step(std::true_type(), std::false_type(), (s + 1) * kF64BK);
    if (nsteps >= 2) k_step(std::true_type(), std::integral_constant<bool, TAIL>(), (nsteps - 1) * kF64BK);
    k_step(std::false_type(), std::false_type(), 0);

    const bool full_mn = m0 + BM <= g.M && n0 + BN <= g.N;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int64_t m = m0 + wm + i * 16 + 4 * r + lk, n = n0 + wn + j * 16 + lm;
                if (full_mn || (m < g.M && n < g.N)) c[m * g.scm + n * g.scn] = acc[i][j][r];
            }
}

bool use_f64_pinned() {
    return option(OPT_DOT_F64_PINNED) != 0;   // 0: gemm_kernel<double> for every layout
}

// Tile form and number of K chunks of a product on the kernels with a pinned instruction order: the cheapest of the available forms
// at 1 .. 32 chunks under a model fitted to measurements (1000^3 .. 4096^3, 512 x 8192 x 512, 2048 x 512 x 2048, 4 .. 64 x 512^3 /
// 1024^3: the model's pick is the measured best or within 9 % of it).  Per K step, in microseconds:
//   bf16 parts (K step 16), 128 x 128 tiles: 1.56 with two workgroups on a CU, 1.09 - 1.29 with one (the more CUs are busy, the
//       lower the clock); 256 x 256 tiles, one per CU: 1.75 - 2.5;
//   double precision (K step 8), 128 x 128 tiles: 2.05 with two workgroups on a CU, 1.10 - 1.26 with one.
// A round of workgroups costs 8 / 10 / 13 us on top (launch, first fetch, epilogue), the summing launch 5 us plus its traffic at
// 5 TB/s.  The options dot_big = 0 / 1 and dot_splits = n force either choice (for measurements and tests).
void choose_plan(bool f64, int64_t M, int64_t N, int64_t batch, int64_t steps, bool can_split, bool* big, int64_t* want) {
    const int force_big = option(OPT_DOT_BIG), force_splits = option(OPT_DOT_SPLITS);
    const int64_t cus = device_cus();
    const int64_t nbig = cdiv(M, (int64_t)XBM) * cdiv(N, (int64_t)XBN) * batch, nsmall = cdiv(M, (int64_t)BM) * cdiv(N, (int64_t)BN) * batch;
    const double out_bytes = (double)batch * (double)M * (double)N * (f64 ? 8.0 : 4.0);
    auto cost = [&](bool bg, int64_t sp) {
        const int64_t chunk = cdiv(steps, sp), real = cdiv(steps, chunk);
        const int64_t n = (bg ? nbig : nsmall) * real;
        double us;
        if (bg) {
            const int64_t full = n / cus, rem = n % cus;
            us = (double)full * ((double)chunk * 2.5 + 10.0) + (rem ? (double)chunk * (1.75 + 0.75 * (double)rem / (double)cus) + 10.0 : 0.0);
        } else {
            const int64_t full = n / (2 * cus), rem = n % (2 * cus);
            const double r = (double)rem / (double)cus;
            const double ts2 = f64 ? 2.05 : 1.56, fix = f64 ? 13.0 : 8.0;
            const double ts = f64 ? (rem <= cus ? 1.10 + 0.16 * r : 1.26 + 0.79 * (r - 1.0)) : (rem <= cus ? 1.09 + 0.2 * r : 1.29 + 0.27 * (r - 1.0));
            us = (double)full * ((double)chunk * ts2 + fix) + (rem ? (double)chunk * ts + fix : 0.0);
        }
        if (real > 1) us = (us + 5.0 + (double)(real + 1) * out_bytes / 5.0e6) * 1.03;   // a split must pay for itself
        return us;
    };
    // chunks of at least 4 steps; the partial sums of a split stay below 32 x 64 (128) MB
    const int64_t max_sp = (can_split && nsmall <= 4 * cus) ? std::min<int64_t>(32, steps / 4) : 1;
    bool best_big = false;
    int64_t best_sp = 1;
    double best = -1.0;
    for (int form = 0; form < (f64 ? 1 : 2); form++) {
        if (!f64 && force_big >= 0 && form != (force_big ? 1 : 0)) continue;
        for (int64_t sp = 1; sp <= std::max<int64_t>(max_sp, 1); sp++) {
            const double us = cost(form == 1, sp);
            if (best < 0.0 || us < best) {
                best = us;
                best_big = form == 1;
                best_sp = sp;
            }
        }
    }
    if (force_splits > 0 && can_split && batch * M * N < (1ll << 31)) best_sp = std::min<int64_t>(force_splits, std::max<int64_t>(steps / 2, 1));
    *big = best_big;
    *want = best_sp;
}

template <class T>
int32_t launch_gemm(GemmArgs g, T* c, const T* a, const T* b, int64_t batch, hipStream_t stream) {
    int64_t blocks = (int64_t)g.tiles_m * g.tiles_n * batch;
    if (blocks == 0) return DNH_OK;
    if (blocks > 0x7FFFFFFF) return fail(DNH_ERR_NOT_SUPPORTED, "dnh_dot: too many output tiles");
    constexpr int V = 16 / (int)sizeof(T);
    bool fast = g.sak == 1 && g.sbn == 1 && g.K > 0 &&
                (g.sam % V) == 0 && (g.sbk % V) == 0 && aligned_to(a, 16) && aligned_to(b, 16);
    for (int d = 0; d < g.nbatch && fast; d++) fast = (g.bsa[d] % V) == 0 && (g.bsb[d] % V) == 0;

    const GemmArgs orig = g;
    WorkspaceLease lease;   // covers the product and its finishing launch
    T* target = c;
    int64_t splits = 1;
    const int64_t steps = (g.K + kBK<T> - 1) / kBK<T>;
    bool x3 = false, big = false;
    bool a_kc = false, b_kc = false;
    if constexpr (sizeof(T) == 4) {
        // each operand either k-contiguous (its 16-byte fetches are declared at element alignment: any offset and pitch), or
        // contiguous along its other dimension
        a_kc = g.sak == 1;
        b_kc = g.sbk == 1;
        x3 = g.K >= kX3BK && (a_kc || g.sam == 1) && (b_kc || g.sbn == 1) && !g.accumulate && use_bf16x3();
    }
    bool f64p = false;   // double precision on gemm_f64_kernel: each operand contiguous along one of its dimensions
    if constexpr (sizeof(T) == 8) {
        a_kc = g.sak == 1;
        b_kc = g.sbk == 1;
        f64p = g.K >= kF64BK && (a_kc || g.sam == 1) && (b_kc || g.sbn == 1) && !g.accumulate && use_f64_pinned();
    }
    int64_t want = 1;
    if (x3 || f64p) {
        choose_plan(f64p, g.M, g.N, batch, steps, g.nbatch < DNH_MAX_DIMS, &big, &want);
        if (big) {
            g.tiles_m = (uint32_t)cdiv(g.M, (int64_t)XBM);
            g.tiles_n = (uint32_t)cdiv(g.N, (int64_t)XBN);
            blocks = (int64_t)g.tiles_m * g.tiles_n * batch;
        }
    } else if (g.nbatch < DNH_MAX_DIMS && blocks <= 4 * (int64_t)device_cus()) {
        want = choose_k_splits<T>(blocks, steps, batch * g.M * g.N);
        const int force_splits = option(OPT_DOT_SPLITS);
        if (force_splits > 0) want = std::min<int64_t>(force_splits, std::max<int64_t>(steps / 2, 1));
    }
    if (want > 1) {   // the choosers keep chunks of at least 2 steps: the chunk below is not empty
        const int64_t kchunk = ((steps + want - 1) / want) * kBK<T>;
        splits = (g.K + kchunk - 1) / kchunk;
        if (splits > 1) {
            T* ws = nullptr;
            DNH_TRY(workspace(stream, sizeof(T) * (size_t)batch * splits * g.M * g.N, (void**)&ws, lease));
            int64_t inner = splits * g.M * g.N;       // workspace layout [batch...][split][M][N]
            for (int d = g.nbatch - 1; d >= 0; d--) {
                g.bsc[d] = inner;
                inner *= g.bshape[d];
            }
            g.bshape[g.nbatch] = (uint32_t)splits;
            g.bsa[g.nbatch] = kchunk * g.sak;
            g.bsb[g.nbatch] = kchunk * g.sbk;
            g.bsc[g.nbatch] = g.M * g.N;
            g.nbatch++;
            g.kchunk = kchunk;
            g.scm = g.N;
            g.scn = 1;
            g.accumulate = 0;
            c = ws;
            blocks *= splits;
        }
    }
    g.xcd_chunk = (blocks % 8 == 0 && blocks >= 64) ? (uint32_t)(blocks / 8) : 0u;
#define DNH_X3_LAUNCH(SP, TL, AK, BK_) hipLaunchKernelGGL((gemm_bf16x3_kernel<SP, TL, AK, BK_>), dim3((unsigned)blocks), dim3(kBlock), 0, stream, c, a, b, g)
#define DNH_X3_AB(SP, TL) do { if (a_kc) { if (b_kc) DNH_X3_LAUNCH(SP, TL, true, true); else DNH_X3_LAUNCH(SP, TL, true, false); } \
                               else { if (b_kc) DNH_X3_LAUNCH(SP, TL, false, true); else DNH_X3_LAUNCH(SP, TL, false, false); } } while (0)
#define DNH_X3(SP) do { if (g.K % kX3BK) DNH_X3_AB(SP, true); else DNH_X3_AB(SP, false); } while (0)
#define DNH_GEMM(FASTF, ACCF, SPLITF) hipLaunchKernelGGL((gemm_kernel<T, FASTF, ACCF, SPLITF>), dim3((unsigned)blocks), dim3(kBlock), 0, stream, c, a, b, g)
    g.xcd_2d = (x3 && g.nbatch == 0 && (g.tiles_m % 2u) == 0 && (g.tiles_n % 4u) == 0 && blocks >= 64) ? 1u : 0u;
#define DNH_BIG_LAUNCH(SP, TL, AK, BK_) do { \
        static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_bf16x3_big_kernel<SP, TL, AK, BK_>), \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)kBigLdsBytes); \
        if (attr != hipSuccess) return fail(DNH_ERR_HIP, "dnh_dot: %s", hipGetErrorString(attr)); \
        hipLaunchKernelGGL((gemm_bf16x3_big_kernel<SP, TL, AK, BK_>), dim3((unsigned)blocks), dim3(kBigThreads), kBigLdsBytes, stream, c, a, b, g); } while (0)
#define DNH_BIG_AB(SP, TL) do { if (a_kc) { if (b_kc) DNH_BIG_LAUNCH(SP, TL, true, true); else DNH_BIG_LAUNCH(SP, TL, true, false); } \
                                else { if (b_kc) DNH_BIG_LAUNCH(SP, TL, false, true); else DNH_BIG_LAUNCH(SP, TL, false, false); } } while (0)
#define DNH_BIG(SP) do { if (g.K % kX3BK) DNH_BIG_AB(SP, true); else DNH_BIG_AB(SP, false); } while (0)
    if constexpr (sizeof(T) == 4) {
        if (big) {
            if (splits > 1) DNH_BIG(true); else DNH_BIG(false);
        }
    }
#define DNH_F64_LAUNCH(SP, TL, AK, BK_) hipLaunchKernelGGL((gemm_f64_kernel<SP, TL, AK, BK_>), dim3((unsigned)blocks), dim3(kBlock), 0, stream, (double*)c, (const double*)a, (const double*)b, g)
#define DNH_F64_AB(SP, TL) do { if (a_kc) { if (b_kc) DNH_F64_LAUNCH(SP, TL, true, true); else DNH_F64_LAUNCH(SP, TL, true, false); } \
                                else { if (b_kc) DNH_F64_LAUNCH(SP, TL, false, true); else DNH_F64_LAUNCH(SP, TL, false, false); } } while (0)
#define DNH_F64(SP) do { if (g.K % kF64BK) DNH_F64_AB(SP, true); else DNH_F64_AB(SP, false); } while (0)
    if constexpr (sizeof(T) == 8) {
        if (f64p) {
            if (splits > 1) DNH_F64(true); else DNH_F64(false);
        }
    }
#undef DNH_F64
#undef DNH_F64_AB
#undef DNH_F64_LAUNCH
    if (big || f64p) {
        // launched above
    } else if (splits > 1) {
        if (x3) {
            if constexpr (sizeof(T) == 4) DNH_X3(true);
        } else if (fast) DNH_GEMM(true, false, true);
        else DNH_GEMM(false, false, true);
    } else if (g.accumulate) {
        if (fast) DNH_GEMM(true, true, false); else DNH_GEMM(false, true, false);
    } else {
        if (x3) {
            if constexpr (sizeof(T) == 4) DNH_X3(false);
        } else if (fast) DNH_GEMM(true, false, false);
        else DNH_GEMM(false, false, false);
    }
#undef DNH_GEMM
#undef DNH_BIG
#undef DNH_BIG_AB
#undef DNH_BIG_LAUNCH
#undef DNH_X3
#undef DNH_X3_AB
#undef DNH_X3_LAUNCH
    DNH_LAUNCH_CHECK();
    if (splits > 1) {
        constexpr int FV = 16 / (int)sizeof(T);
        bool vec = orig.scn == 1 && (orig.N % FV) == 0 && (orig.scm % FV) == 0 && aligned_to(target, 16);
        for (int d = 0; d < orig.nbatch && vec; d++) vec = (orig.bsc[d] % FV) == 0;
        const uint32_t total = (uint32_t)(batch * orig.M * orig.N / (vec ? FV : 1));   // at most 4 tiles per CU: fits 32 bits
        const unsigned fb = (unsigned)cdiv((int64_t)total, 64);
#define DNH_FINISH(ACCF, SGV, VV) hipLaunchKernelGGL((gemm_split_finish_kernel<T, ACCF, SGV, VV>), dim3(fb), dim3(64 * SGV), 0, stream, target, (const T*)c, orig, (uint32_t)splits, total)
#define DNH_FINISH_V(ACCF, SGV) do { if (vec) DNH_FINISH(ACCF, SGV, FV); else DNH_FINISH(ACCF, SGV, 1); } while (0)
        if (splits >= 32) {
            if (orig.accumulate) DNH_FINISH_V(true, 16); else DNH_FINISH_V(false, 16);
        } else {
            if (orig.accumulate) DNH_FINISH_V(true, 4); else DNH_FINISH_V(false, 4);
        }
#undef DNH_FINISH_V
#undef DNH_FINISH
        DNH_LAUNCH_CHECK();
    }
    return DNH_OK;
}

// ---- vector forms -------------------------------------------------------------------------------------------------------------
// VecVecDot and MatVecDot are bandwidth-bound reductions, not tile problems: y[m] = sum_k A[m,k] * x[k].
//   gemv_rows : A's k dimension has stride 1 — TPR threads share a row, 16-byte loads of A and x, shuffle tree; a long K with few
//               rows (the vector-vector case is M = 1) is split over gridDim.y into partials.
//   gemv_cols : A's m dimension has stride 1 (a transposed view) — one lane per m, coalesced along m, K split over gridDim.y.
// Partials are summed by gemv_finish in index order (deterministic, no float atomics).

template <class T, int VEC, int TPR>
__global__ __launch_bounds__(kBlock) void gemv_rows_kernel(T* y, T* partial, const T* a, const T* x, uint32_t M, int64_t K, int64_t sam,
                                                           int64_t sak, int64_t sxk, int64_t sym, int64_t chunk, uint32_t splits) {
    constexpr int RPB = kBlock / TPR;
    const uint32_t m = blockIdx.x * RPB + threadIdx.x / TPR;
    const uint32_t lane = threadIdx.x % TPR;
    const int64_t k0 = (int64_t)blockIdx.y * chunk;
    const int64_t k1 = (k0 + chunk < K) ? k0 + chunk : K;
    T acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++) acc[e] = T(0);
    if (m < M) {
        const T* row = a + (int64_t)m * sam;
        if constexpr (VEC > 1) {
            int64_t k = k0 + (int64_t)lane * VEC;
            for (; k + VEC <= k1; k += (int64_t)TPR * VEC) {
                const Pack<T, VEC> va = load_pack<T, VEC>(row + k);
                const Pack<T, VEC> vx = *(const Pack<T, VEC>*)(x + k);
#pragma unroll
                for (int e = 0; e < VEC; e++) acc[e] += va.v[e] * vx.v[e];
            }
            const int64_t t0 = k0 + ((k1 - k0) / VEC) * VEC + lane;
            if (t0 < k1) acc[0] += row[t0] * x[t0];
        } else {
            for (int64_t k = k0 + lane; k < k1; k += TPR) acc[0] += row[k * sak] * x[k * sxk];
        }
    }
    T s = acc[0];
#pragma unroll
    for (int e = 1; e < VEC; e++) s += acc[e];
#pragma unroll
    for (int w = (TPR < 64 ? TPR : 64) / 2; w >= 1; w >>= 1) s += __shfl_xor(s, w, 64);
    if constexpr (TPR > 64) {
        __shared__ T sh[TPR / 64];
        if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = s;
        __syncthreads();
        if (threadIdx.x == 0)
#pragma unroll
            for (int w = 1; w < TPR / 64; w++) s += sh[w];
    }
    if (m < M && lane == 0) {
        if (splits == 1) y[(int64_t)m * sym] = s;
        else partial[(int64_t)m * splits + blockIdx.y] = s;
    }
}

template <class T, int VEC>
__global__ __launch_bounds__(kBlock) void gemv_cols_kernel(T* y, T* partial, const T* a, const T* x, uint32_t M, int64_t K, int64_t sak,
                                                           int64_t sxk, int64_t sym, int64_t chunk, uint32_t splits, uint32_t mblocks,
                                                           uint32_t xcd_chunk) {
    // one workgroup per (split, block of m), the m block fastest; xcd_chunk re-numbers the workgroups so that every XCD takes one
    // contiguous range of that order (with 8 m blocks the plain order would pin each XCD to one 4 KB-wide strip of the matrix)
    uint32_t bid = blockIdx.x;
    if (xcd_chunk) bid = (bid % 8u) * xcd_chunk + bid / 8u;
    const uint32_t split = bid / mblocks, mb = bid - split * mblocks;
    const uint32_t m = (mb * kBlock + threadIdx.x) * VEC;
    if (m >= M) return;
    const int64_t k0 = (int64_t)split * chunk;
    const int64_t k1 = (k0 + chunk < K) ? k0 + chunk : K;
    T acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++) acc[e] = T(0);
    const T* p = a + m;
    int64_t k = k0;
    for (; k + 1 < k1; k += 2) {
        const Pack<T, VEC> v0 = load_pack<T, VEC>(p + k * sak);
        const Pack<T, VEC> v1 = load_pack<T, VEC>(p + (k + 1) * sak);
        const T x0 = x[k * sxk], x1 = x[(k + 1) * sxk];
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[e] += v0.v[e] * x0;
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[e] += v1.v[e] * x1;
    }
    if (k < k1) {
        const Pack<T, VEC> v0 = load_pack<T, VEC>(p + k * sak);
        const T x0 = x[k * sxk];
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[e] += v0.v[e] * x0;
    }
    if (splits == 1) {
#pragma unroll
        for (int e = 0; e < VEC; e++) y[(int64_t)(m + e) * sym] = acc[e];
    } else {
        // partials [split][m]: the VEC sums of a thread leave as one vector store (VEC > 1 implies M % VEC == 0)
        Pack<T, VEC> v;
#pragma unroll
        for (int e = 0; e < VEC; e++) v.v[e] = acc[e];
        store_pack<T, VEC>(partial + (int64_t)split * M + m, v);
    }
}

// Sums the [split][m] partials of gemv_cols in split order inside each of the 16 groups, then the groups in order (deterministic).
template <class T>
__global__ __launch_bounds__(kBlock) void gemv_cols_finish_kernel(T* y, const T* partial, uint32_t M, uint32_t splits, int64_t sym) {
    constexpr int WX = 16, NY = kBlock / WX;
    const uint32_t x = threadIdx.x % WX, g = threadIdx.x / WX;
    const uint32_t m = blockIdx.x * WX + x;
    T s = T(0);
    if (m < M)
        for (uint32_t i = g; i < splits; i += NY) s += partial[(int64_t)i * M + m];
    __shared__ T sh[NY][WX];
    sh[g][x] = s;
    __syncthreads();
    if (g == 0 && m < M) {
        for (int w = 1; w < NY; w++) s += sh[w][x];
        y[(int64_t)m * sym] = s;
    }
}

template <class T>
__global__ __launch_bounds__(kBlock) void gemv_finish_kernel(T* y, const T* partial, uint32_t M, uint32_t splits, int64_t sym) {
    const uint32_t m = blockIdx.x;
    T s = T(0);
    for (uint32_t i = threadIdx.x; i < splits; i += kBlock) s += partial[(int64_t)m * splits + i];
#pragma unroll
    for (int w = 32; w >= 1; w >>= 1) s += __shfl_xor(s, w, 64);
    __shared__ T sh[kBlock / 64];
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kBlock / 64; w++) s += sh[w];
        y[(int64_t)m * sym] = s;
    }
}

// Returns false when neither vector kernel fits the strides (the tile kernel then handles the call).
template <class T>
bool try_gemv(const GemmArgs& g, T* y, const T* a, const T* x, hipStream_t stream, int32_t* status) {
    if (g.N != 1 || g.nbatch != 0 || g.M > (int64_t)kMaxItems) return false;
    *status = DNH_OK;
    if (g.K == 0) return false;
    const uint32_t M = (uint32_t)g.M;
    const int cus = device_cus();
    constexpr int V = 16 / (int)sizeof(T);
    T* partial = nullptr;
    WorkspaceLease lease;
    if (g.sak == 1 || g.M == 1) {
        // (vectors of 4- and 8-byte elements are fetched at element alignment: any row pitch and start)
        const bool vec = g.sak == 1 && g.sbk == 1 && vector_stride(g.sam, V, sizeof(T)) && vector_address(a, V, sizeof(T)) && vector_address(x, V, sizeof(T));
        const int v = vec ? V : 1;
        const int tpr = g.K >= (int64_t)256 * v * 2 ? 256 : (g.K >= (int64_t)64 * v ? 64 : 16);
        const int64_t row_blocks = (M + kBlock / tpr - 1) / (kBlock / tpr);
        uint32_t splits = 1;
        int64_t chunk = g.K;
        if (tpr == 256 && row_blocks < (int64_t)cus * 4) {
            const int64_t min_chunk = (int64_t)256 * v * 8;
            int64_t sp = ((int64_t)cus * 8 + row_blocks - 1) / row_blocks;
            const int64_t maxs = (g.K + min_chunk - 1) / min_chunk;
            if (sp > maxs) sp = maxs;
            if (sp > 1) {
                chunk = (g.K + sp - 1) / sp;
                chunk = ((chunk + 256 * v - 1) / (256 * v)) * (256 * v);
                splits = (uint32_t)((g.K + chunk - 1) / chunk);
            }
        }
        if (splits > 1 && (*status = workspace(stream, sizeof(T) * (size_t)M * splits, (void**)&partial, lease)) != DNH_OK) return true;
        const dim3 grid((unsigned)row_blocks, splits);
#define DNH_GEMV(VV, TPR) hipLaunchKernelGGL((gemv_rows_kernel<T, VV, TPR>), grid, dim3(kBlock), 0, stream, y, partial, a, x, M, g.K, g.sam, g.sak, g.sbk, g.scm, chunk, splits)
        if (vec) { if (tpr == 256) DNH_GEMV(V, 256); else if (tpr == 64) DNH_GEMV(V, 64); else DNH_GEMV(V, 16); }
        else { if (tpr == 256) DNH_GEMV(1, 256); else if (tpr == 64) DNH_GEMV(1, 64); else DNH_GEMV(1, 16); }
#undef DNH_GEMV
        if (splits > 1) hipLaunchKernelGGL(gemv_finish_kernel<T>, dim3(M), dim3(kBlock), 0, stream, y, (const T*)partial, M, splits, g.scm);
    } else if (g.sam == 1) {
        const bool vec = (M % V) == 0 && vector_stride(g.sak, V, sizeof(T)) && vector_address(a, V, sizeof(T));
        const int v = vec ? V : 1;
        const int64_t mblocks = (M / v + kBlock - 1) / kBlock;
        uint32_t splits = 1;
        int64_t chunk = g.K;
        if (mblocks < (int64_t)cus * 4) {
            int64_t sp = ((int64_t)cus * 4 + mblocks - 1) / mblocks;
            const int64_t maxs = (g.K + 63) / 64;
            if (sp > maxs) sp = maxs;
            if (sp > 1) {
                chunk = (g.K + sp - 1) / sp;
                splits = (uint32_t)((g.K + chunk - 1) / chunk);
            }
        }
        if (splits > 65535) return false;
        if (splits > 1 && (*status = workspace(stream, sizeof(T) * (size_t)M * splits, (void**)&partial, lease)) != DNH_OK) return true;
        const int64_t total = mblocks * splits;
        if (total > 0x7FFFFFFF) return false;
        // measured: +4 % when the m blocks map one-to-one onto the XCDs (8 blocks), -2 % with 16 blocks, so only the former is re-numbered
        const uint32_t xcd_chunk = (mblocks <= 8 && total % 8 == 0 && total >= 64) ? (uint32_t)(total / 8) : 0u;
        if (vec) hipLaunchKernelGGL((gemv_cols_kernel<T, V>), dim3((unsigned)total), dim3(kBlock), 0, stream, y, partial, a, x, M, g.K, g.sak, g.sbk, g.scm, chunk, splits, (uint32_t)mblocks, xcd_chunk);
        else hipLaunchKernelGGL((gemv_cols_kernel<T, 1>), dim3((unsigned)total), dim3(kBlock), 0, stream, y, partial, a, x, M, g.K, g.sak, g.sbk, g.scm, chunk, splits, (uint32_t)mblocks, xcd_chunk);
        if (splits > 1) hipLaunchKernelGGL(gemv_cols_finish_kernel<T>, dim3((M + 15) / 16), dim3(kBlock), 0, stream, y, (const T*)partial, M, splits, g.scm);
    } else {
        return false;
    }
    if (hipGetLastError() != hipSuccess) *status = fail(DNH_ERR_HIP, "gemv launch failed");
    return true;
}

// ---- integer types ------------------------------------------------------------------------------------------------------------
// The reference's host backend computes dot for the types BLAS does not cover as multiply + sumAxis in the element type
// (Host/HostBackend.fs:544-546), i.e. with wrapping arithmetic; its CUDA backend has no such path.  Wrapping is a ring
// homomorphism, so products and sums are formed in the unsigned type of at least 32 bits and truncated once at the end:
// bit-identical to wrapping at every step.  No matrix cores for 32/64-bit integers: a 64 x 64 tile per workgroup, a 4 x 4
// block of outputs per thread, operands staged through LDS.
template <class T>
__global__ __launch_bounds__(256) void gemm_int_kernel(T* __restrict__ c, const T* __restrict__ a, const T* __restrict__ b, GemmArgs g) {
    using U = typename std::conditional<sizeof(T) == 8, uint64_t, uint32_t>::type;
    constexpr int TM = 64, TN = 64, TK = 16;
    __shared__ U As[TK][TM + 4];
    __shared__ U Bs[TK][TN + 4];
    uint32_t bid = blockIdx.x;
    const uint32_t tn = bid % g.tiles_n;
    bid /= g.tiles_n;
    const uint32_t tm = bid % g.tiles_m;
    bid /= g.tiles_m;
    int64_t oa = 0, ob = 0, oc = 0;
    for (int d = g.nbatch - 1; d >= 0; d--) {
        const uint32_t q = (d == 0) ? 0u : bid / g.bshape[d];
        const uint32_t i = bid - q * g.bshape[d];
        bid = q;
        oa += (int64_t)i * g.bsa[d];
        ob += (int64_t)i * g.bsb[d];
        oc += (int64_t)i * g.bsc[d];
    }
    a += oa;
    b += ob;
    c += oc;
    const int64_t m0 = (int64_t)tm * TM, n0 = (int64_t)tn * TN;
    const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
    U acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = 0;
    for (int64_t k0 = 0; k0 < g.K; k0 += TK) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int idx = tid + i * 256;
            {
                const int row = idx / TK, kk = idx % TK;
                const int64_t m = m0 + row, k = k0 + kk;
                As[kk][row] = (m < g.M && k < g.K) ? (U)a[m * g.sam + k * g.sak] : U(0);
            }
            {
                const int kk = idx / TN, col = idx % TN;
                const int64_t k = k0 + kk, n = n0 + col;
                Bs[kk][col] = (k < g.K && n < g.N) ? (U)b[k * g.sbk + n * g.sbn] : U(0);
            }
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < TK; kk++) {
            U av[4], bv[4];
#pragma unroll
            for (int i = 0; i < 4; i++) av[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; j++) bv[j] = Bs[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] += av[i] * bv[j];
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int64_t m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
            if (m < g.M && n < g.N) c[m * g.scm + n * g.scn] = (T)acc[i][j];
        }
}

// 32-bit integers on the int8 matrix instruction.  Modulo 2^32 an element is the sum of four signed bytes d_i 2^(8 i) (the bytes of
// (u + 0x80808080) ^ 0x80808080: adding 128 to every byte with carries, then taking 128 off each byte), so a.b = sum over i, j of
// 2^(8 (i + j)) sum_k da_i db_j, of which the ten terms with i + j <= 3 survive the modulus.  v_mfma_i32_32x32x32_i8 forms the byte
// products exactly and adds them in int32, whose wrap-around is the modulus itself: one accumulator per shift i + j, combined at the
// end as acc0 + (acc1 << 8) + (acc2 << 16) + (acc3 << 24).  Bit-identical to the wrapping multiply + sum of the host backend for any
// K.  128 x 128 tile, K step 32, 512 threads = 8 wavefronts 2 x 4, each owning 64 x 32 (two 32 x 32 sub-tiles x four shifts); the four
// byte planes of both operands lie in LDS k-contiguous, [plane][row][32 + 16 bytes], double buffered.  20 matrix instructions per
// wavefront and K step replace 64 x 32 x 32 / 64 lanes = 1024 integer multiply-adds per lane.
typedef int i32x4v __attribute__((ext_vector_type(4)));
typedef int i32x16v __attribute__((ext_vector_type(16)));
constexpr int kI8BK = 32, kI8Row = 48, kI8Threads = 512;
constexpr size_t kI8LdsBytes = (size_t)2 * 2 * 4 * BM * kI8Row;

// four elements (consecutive k) -> one dword of each byte plane
__device__ __forceinline__ void cut4_i8(const uint32_t (&w)[4], uint32_t (&plane)[4]) {
    uint32_t d[4];
#pragma unroll
    for (int e = 0; e < 4; e++) d[e] = (w[e] + 0x80808080u) ^ 0x80808080u;
    const uint32_t lo01 = __builtin_amdgcn_perm(d[1], d[0], 0x05010400u), hi01 = __builtin_amdgcn_perm(d[1], d[0], 0x07030602u);
    const uint32_t lo23 = __builtin_amdgcn_perm(d[3], d[2], 0x05010400u), hi23 = __builtin_amdgcn_perm(d[3], d[2], 0x07030602u);
    plane[0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
    plane[1] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
    plane[2] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
    plane[3] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
}

// Staging of one operand tile (128 rows x 32 k) by 512 threads, eight elements per thread.
//   KC (k contiguous, 16-byte aligned rows): eight lanes cover the 32 k of a row with one 16-byte load each; a thread takes rows r, r + 64.
//   otherwise (rows contiguous): a thread takes one row and 8 consecutive k with element loads.
template <bool KC>
struct I8Stage {
    int row, kofs;
    const uint32_t *p0, *p1;   // a row beyond the matrix reads row 0: its products land beyond the matrix too and are never stored
    int64_t ks;
    __device__ __forceinline__ void init(const uint32_t* base, int64_t row0, int64_t limit, int64_t rs, int64_t kstride, int tid) {
        row = KC ? tid >> 3 : tid & 127;
        kofs = KC ? (tid & 7) * 4 : (tid >> 7) * 8;
        p0 = base + (row0 + row < limit ? (row0 + row) * rs : 0);
        p1 = base + (KC && row0 + row + 64 < limit ? (row0 + row + 64) * rs : 0);
        ks = KC ? 1 : kstride;
    }
    template <bool TAIL>
    __device__ __forceinline__ void load(int64_t k0, int64_t K, uint32_t (&r)[8]) const {
        if (!TAIL || k0 + kI8BK <= K) {
            if constexpr (KC) {
                typedef uint32_t u32x4v __attribute__((ext_vector_type(4), aligned(4)));
                const u32x4v v0 = *reinterpret_cast<const u32x4v*>(p0 + k0 + kofs), v1 = *reinterpret_cast<const u32x4v*>(p1 + k0 + kofs);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    r[e] = v0[e];
                    r[4 + e] = v1[e];
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) r[e] = p0[(k0 + kofs + e) * ks];
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int64_t k = k0 + kofs + (KC ? (e & 3) : e);
                const uint32_t* p = (KC && e >= 4) ? p1 : p0;
                const uint32_t v = p[(k < K ? k : K - 1) * ks];
                r[e] = k < K ? v : 0u;
            }
        }
    }
    // half of store(): elements 4 H .. 4 H + 3
    template <int H>
    __device__ __forceinline__ void piece(const uint32_t (&r)[8], unsigned char (*tile)[BM][kI8Row]) const {
        const uint32_t w[4] = {r[4 * H], r[4 * H + 1], r[4 * H + 2], r[4 * H + 3]};
        uint32_t q[4];
        cut4_i8(w, q);
#pragma unroll
        for (int s = 0; s < 4; s++) {
            if constexpr (KC) *reinterpret_cast<uint32_t*>(&tile[s][row + 64 * H][kofs]) = q[s];
            else *reinterpret_cast<uint32_t*>(&tile[s][row][kofs + 4 * H]) = q[s];
        }
    }
    __device__ __forceinline__ void store(const uint32_t (&r)[8], unsigned char (*tile)[BM][kI8Row]) const {
        uint32_t w0[4] = {r[0], r[1], r[2], r[3]}, w1[4] = {r[4], r[5], r[6], r[7]}, q0[4], q1[4];
        cut4_i8(w0, q0);
        cut4_i8(w1, q1);
#pragma unroll
        for (int s = 0; s < 4; s++) {
            if constexpr (KC) {
                *reinterpret_cast<uint32_t*>(&tile[s][row][kofs]) = q0[s];
                *reinterpret_cast<uint32_t*>(&tile[s][row + 64][kofs]) = q1[s];
            } else {
                typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
                *reinterpret_cast<u32x2*>(&tile[s][row][kofs]) = u32x2{q0[s], q1[s]};
            }
        }
    }
};

template <bool TAIL, bool A_KC, bool B_KC>
__global__ __launch_bounds__(kI8Threads) void gemm_i32_i8parts_kernel(uint32_t* c, const uint32_t* a, const uint32_t* b, GemmArgs g) {
    extern __shared__ __align__(16) unsigned char i8_lds[];
    typedef unsigned char (*Tiles)[4][BM][kI8Row];                 // [buffer][plane][row][k]
    Tiles As = reinterpret_cast<Tiles>(i8_lds);
    Tiles Bs = reinterpret_cast<Tiles>(i8_lds + kI8LdsBytes / 2);

    uint32_t bid = blockIdx.x;
    if (g.xcd_chunk) bid = (bid % 8u) * g.xcd_chunk + bid / 8u;
    const uint32_t tn = bid % g.tiles_n;
    bid /= g.tiles_n;
    const uint32_t tm = bid % g.tiles_m;
    bid /= g.tiles_m;
    int64_t oa = 0, ob = 0, oc = 0;
    for (int d = g.nbatch - 1; d >= 0; d--) {
        const uint32_t q = (d == 0) ? 0u : bid / g.bshape[d];
        const uint32_t i = bid - q * g.bshape[d];
        bid = q;
        oa += (int64_t)i * g.bsa[d];
        ob += (int64_t)i * g.bsb[d];
        oc += (int64_t)i * g.bsc[d];
    }
    const int64_t K = g.K;
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
    a += oa;
    b += ob;
    c += oc;
    const int tid = threadIdx.x;

    I8Stage<A_KC> sa;
    I8Stage<B_KC> sb;
    sa.init(a, m0, g.M, g.sam, g.sak, tid);
    sb.init(b, n0, g.N, g.sbn, g.sbk, tid);
    uint32_t ra[8], rb[8];

    // operand lane l supplies 16 consecutive k (16 (l / 32) ...) of row l % 32; accumulator register r of lane l holds row
    // 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32 of its 32 x 32 tile (as the other 32 x 32 matrix instructions)
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = (wave >> 2) * 64, wn = (wave & 3) * 32;
    const int lm = lane & 31, lk = lane >> 5;
    i32x16v acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int s = 0; s < 4; s++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][s][r] = 0;

    // One K step, the instruction order pinned as in the bf16-parts kernels: the fetch of the next step (NEXT), the LDS reads of B and of
    // the first 32 rows of A, then the 20 matrix instructions with the remaining LDS reads behind the first four and the four pieces of
    // the cutting (one cut4_i8 each with its LDS writes) behind numbers 8, 11, 14 and 17.
    int cur = 0;
    auto k_step = [&](auto next_tag, auto tail_tag, int64_t k_next) {
        constexpr bool NEXT = decltype(next_tag)::value, TL = decltype(tail_tag)::value;
        if constexpr (NEXT) {
            sa.template load<TL>(k_next, K, ra);
            sb.template load<TL>(k_next, K, rb);
        }
        __builtin_amdgcn_sched_barrier(0);
        i32x4v av[2][4], bv[4];
#pragma unroll
        for (int s = 0; s < 4; s++) bv[s] = *reinterpret_cast<const i32x4v*>(&Bs[cur][s][wn + lm][lk * 16]);
#pragma unroll
        for (int s = 0; s < 4; s++) av[0][s] = *reinterpret_cast<const i32x4v*>(&As[cur][s][wm + lm][lk * 16]);
        __builtin_amdgcn_sched_barrier(0);
        static_for<20>([&](auto tt) {
            // products in the order (sub-tile i, shift sh, plane pa of A): 1 + 2 + 3 + 4 per sub-tile
            constexpr int t = decltype(tt)::value, i = t / 10, u = t % 10;
            constexpr int sh = u < 1 ? 0 : u < 3 ? 1 : u < 6 ? 2 : 3;
            constexpr int pa = u - (sh == 0 ? 0 : sh == 1 ? 1 : sh == 2 ? 3 : 6);
            acc[i][sh] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[i][pa], bv[sh - pa], acc[i][sh], 0, 0, 0);
            if constexpr (t < 4) av[1][t] = *reinterpret_cast<const i32x4v*>(&As[cur][t][wm + 32 + lm][lk * 16]);
            if constexpr (NEXT && (t == 8 || t == 11)) sa.template piece<(t - 8) / 3>(ra, As[cur ^ 1]);
            if constexpr (NEXT && (t == 14 || t == 17)) sb.template piece<(t - 14) / 3>(rb, Bs[cur ^ 1]);
            __builtin_amdgcn_sched_barrier(0);
        });
        if constexpr (NEXT) {
            __syncthreads();
            cur ^= 1;
        }
    };

    const int64_t nsteps = (K + kI8BK - 1) / kI8BK;
    sa.template load<TAIL>(0, K, ra);
    sb.template load<TAIL>(0, K, rb);
    sa.store(ra, As[0]);
    sb.store(rb, Bs[0]);
    __syncthreads();
    for (int64_t s = 0; s + 2 < nsteps; s++) k_step(std::true_type(), std::false_type(), (s + 1) * kI8BK);
    if (nsteps >= 2) k_step(std::true_type(), std::integral_constant<bool, TAIL>(), (nsteps - 1) * kI8BK);
    k_step(std::false_type(), std::false_type(), 0);

    const bool full_mn = m0 + BM <= g.M && n0 + BN <= g.N;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int64_t m = m0 + wm + i * 32 + (r >> 2) * 8 + lk * 4 + (r & 3);
            const int64_t n = n0 + wn + lm;
            const uint32_t v = (uint32_t)acc[i][0][r] + ((uint32_t)acc[i][1][r] << 8) + ((uint32_t)acc[i][2][r] << 16) + ((uint32_t)acc[i][3][r] << 24);
            if (full_mn || (m < g.M && n < g.N)) c[m * g.scm + n * g.scn] = v;
        }
}

// 64-bit integers the same way: eight signed byte planes per operand, the 36 byte products with i + j <= 7, one int32 accumulator
// per shift.  Modulo 2^64 the accumulators of the low shifts must not wrap (shift s needs its sum modulo 2^(64 - 8 s)): 8 (s + 1)
// byte products of at most 2^14 per K step of 32 stay below 2^31 for 256 steps, so every 256 steps (and at the end) the accumulators are
// added into the 64-bit result, each shifted by its 8 s, and cleared.  64 x 128 tile, 512 threads = 8 wavefronts 2 x 4, 32 x 32 each.
constexpr int kI64BM = 64, kI64BN = 128, kI64FoldSteps = 256;
constexpr size_t kI64LdsBytes = (size_t)2 * 8 * (kI64BM + kI64BN) * kI8Row;

// four elements (consecutive k) -> one dword of each of the eight byte planes
__device__ __forceinline__ void cut4_i8x8(const uint64_t (&w)[4], uint32_t (&plane)[8]) {
    uint32_t lo[4], hi[4], q[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const uint64_t d = (w[e] + 0x8080808080808080ull) ^ 0x8080808080808080ull;
        lo[e] = (uint32_t)d;
        hi[e] = (uint32_t)(d >> 32);
    }
    // (the byte transposition of cut4_i8, without its digit step)
    auto transpose = [](const uint32_t (&d)[4], uint32_t (&out)[4]) {
        const uint32_t lo01 = __builtin_amdgcn_perm(d[1], d[0], 0x05010400u), hi01 = __builtin_amdgcn_perm(d[1], d[0], 0x07030602u);
        const uint32_t lo23 = __builtin_amdgcn_perm(d[3], d[2], 0x05010400u), hi23 = __builtin_amdgcn_perm(d[3], d[2], 0x07030602u);
        out[0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
        out[1] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
        out[2] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
        out[3] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
    };
    transpose(lo, q);
#pragma unroll
    for (int s = 0; s < 4; s++) plane[s] = q[s];
    transpose(hi, q);
#pragma unroll
    for (int s = 0; s < 4; s++) plane[4 + s] = q[s];
}

// Staging of one operand tile (ROWS rows x 32 k of 64-bit elements) by 512 threads: NG = ROWS / 64 groups of four consecutive k per thread.
//   KC (k contiguous, 16-byte aligned rows): eight lanes cover the 32 k of a row, 32 bytes each; group i is row r + 64 i.
//   otherwise (rows contiguous): a thread takes one row and 4 NG consecutive k with element loads.
template <bool KC, int ROWS>
struct I64Stage {
    static constexpr int NG = ROWS / 64;
    int row, kofs;
    const uint64_t* p[NG];   // KC: the rows of the groups (a row beyond the matrix reads row 0: its products are never stored)
    int64_t ks;
    __device__ __forceinline__ void init(const uint64_t* base, int64_t row0, int64_t limit, int64_t rs, int64_t kstride, int tid) {
        row = KC ? tid >> 3 : tid & (ROWS - 1);
        kofs = KC ? (tid & 7) * 4 : (tid / ROWS) * 4 * NG;
#pragma unroll
        for (int i = 0; i < NG; i++) {
            const int64_t rr = row0 + row + (KC ? 64 * i : 0);
            p[i] = base + (rr < limit ? rr * rs : 0);
        }
        ks = KC ? 1 : kstride;
    }
    template <bool TAIL>
    __device__ __forceinline__ void load(int64_t k0, int64_t K, uint64_t (&r)[4 * NG]) const {
#pragma unroll
        for (int i = 0; i < NG; i++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int64_t k = k0 + kofs + (KC ? e : 4 * i + e);
                if (!TAIL || k0 + kI8BK <= K) {
                    r[4 * i + e] = p[i][k * ks];   // (KC: the four loads of a group are 32 contiguous bytes: two 16-byte loads)
                } else {
                    const uint64_t v = p[i][(k < K ? k : K - 1) * ks];
                    r[4 * i + e] = k < K ? v : 0ull;
                }
            }
    }
    __device__ __forceinline__ void store(const uint64_t (&r)[4 * NG], unsigned char (*tile)[ROWS][kI8Row]) const {
        uint32_t q[NG][8];
#pragma unroll
        for (int i = 0; i < NG; i++) {
            const uint64_t w[4] = {r[4 * i], r[4 * i + 1], r[4 * i + 2], r[4 * i + 3]};
            cut4_i8x8(w, q[i]);
        }
#pragma unroll
        for (int s = 0; s < 8; s++)
#pragma unroll
            for (int i = 0; i < NG; i++) {
                if constexpr (KC) *reinterpret_cast<uint32_t*>(&tile[s][row + 64 * i][kofs]) = q[i][s];
                else *reinterpret_cast<uint32_t*>(&tile[s][row][kofs + 4 * i]) = q[i][s];
            }
    }
};

template <bool TAIL, bool A_KC, bool B_KC>
__global__ __launch_bounds__(kI8Threads) void gemm_i64_i8parts_kernel(uint64_t* c, const uint64_t* a, const uint64_t* b, GemmArgs g) {
    extern __shared__ __align__(16) unsigned char i8_lds[];
    typedef unsigned char (*TilesA)[8][kI64BM][kI8Row];            // [buffer][plane][row][k]
    typedef unsigned char (*TilesB)[8][kI64BN][kI8Row];
    TilesA As = reinterpret_cast<TilesA>(i8_lds);
    TilesB Bs = reinterpret_cast<TilesB>(i8_lds + (size_t)2 * 8 * kI64BM * kI8Row);

    uint32_t bid = blockIdx.x;
    if (g.xcd_chunk) bid = (bid % 8u) * g.xcd_chunk + bid / 8u;
    const uint32_t tn = bid % g.tiles_n;
    bid /= g.tiles_n;
    const uint32_t tm = bid % g.tiles_m;
    bid /= g.tiles_m;
    int64_t oa = 0, ob = 0, oc = 0;
    for (int d = g.nbatch - 1; d >= 0; d--) {
        const uint32_t q = (d == 0) ? 0u : bid / g.bshape[d];
        const uint32_t i = bid - q * g.bshape[d];
        bid = q;
        oa += (int64_t)i * g.bsa[d];
        ob += (int64_t)i * g.bsb[d];
        oc += (int64_t)i * g.bsc[d];
    }
    const int64_t K = g.K;
    const int64_t m0 = (int64_t)tm * kI64BM, n0 = (int64_t)tn * kI64BN;
    a += oa;
    b += ob;
    c += oc;
    const int tid = threadIdx.x;

    I64Stage<A_KC, kI64BM> sa;
    I64Stage<B_KC, kI64BN> sb;
    sa.init(a, m0, g.M, g.sam, g.sak, tid);
    sb.init(b, n0, g.N, g.sbn, g.sbk, tid);
    uint64_t ra[4], rb[8];

    const int wave = tid >> 6, lane = tid & 63;
    const int wm = (wave >> 2) * 32, wn = (wave & 3) * 32;
    const int lm = lane & 31, lk = lane >> 5;
    i32x16v acc[8];
    uint64_t tot[16];
#pragma unroll
    for (int r = 0; r < 16; r++) tot[r] = 0;
    auto clear = [&]() {
#pragma unroll
        for (int s = 0; s < 8; s++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[s][r] = 0;
    };
    auto fold = [&]() {
#pragma unroll
        for (int s = 0; s < 8; s++)
#pragma unroll
            for (int r = 0; r < 16; r++) tot[r] += (uint64_t)(int64_t)acc[s][r] << (8 * s);
    };
    clear();

    int cur = 0;
    auto compute = [&]() {
        i32x4v bv[8];
#pragma unroll
        for (int s = 0; s < 8; s++) bv[s] = *reinterpret_cast<const i32x4v*>(&Bs[cur][s][wn + lm][lk * 16]);
#pragma unroll
        for (int pa = 0; pa < 8; pa++) {
            const i32x4v av = *reinterpret_cast<const i32x4v*>(&As[cur][pa][wm + lm][lk * 16]);
#pragma unroll
            for (int pb = 0; pa + pb < 8; pb++) acc[pa + pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, bv[pb], acc[pa + pb], 0, 0, 0);
        }
    };

    const int64_t nsteps = (K + kI8BK - 1) / kI8BK;
    sa.template load<TAIL>(0, K, ra);
    sb.template load<TAIL>(0, K, rb);
    sa.store(ra, As[0]);
    sb.store(rb, Bs[0]);
    __syncthreads();
    for (int64_t s = 0; s + 1 < nsteps; s++) {
        sa.template load<TAIL>((s + 1) * kI8BK, K, ra);
        sb.template load<TAIL>((s + 1) * kI8BK, K, rb);
        __builtin_amdgcn_sched_barrier(0);   // the fetches stay in front of the matrix instructions
        compute();
        if ((s + 1) % kI64FoldSteps == 0) {
            fold();
            clear();
        }
        sa.store(ra, As[cur ^ 1]);
        sb.store(rb, Bs[cur ^ 1]);
        __syncthreads();
        cur ^= 1;
    }
    compute();
    fold();

    const bool full_mn = m0 + kI64BM <= g.M && n0 + kI64BN <= g.N;
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int64_t m = m0 + wm + (r >> 2) * 8 + lk * 4 + (r & 3);
        const int64_t n = n0 + wn + lm;
        if (full_mn || (m < g.M && n < g.N)) c[m * g.scm + n * g.scn] = tot[r];
    }
}

bool use_int_mfma() {
    return option(OPT_DOT_INT_MFMA) != 0;   // 0: every integer product on gemm_int_kernel
}

template <class T>
int32_t launch_gemm_int(GemmArgs g, T* c, const T* a, const T* b, int64_t batch, hipStream_t stream) {
    if constexpr (sizeof(T) == 4) {
        // each operand either k-contiguous with 16-byte aligned rows, or contiguous along its other dimension
        bool a_kc = g.sak == 1, b_kc = g.sbk == 1;   // (k-contiguous rows are fetched at element alignment)
        if (g.K >= kI8BK && (a_kc || g.sam == 1) && (b_kc || g.sbn == 1) && use_int_mfma()) {
            g.tiles_m = (uint32_t)cdiv(g.M, (int64_t)BM);
            g.tiles_n = (uint32_t)cdiv(g.N, (int64_t)BN);
            const int64_t blocks = (int64_t)g.tiles_m * g.tiles_n * batch;
            if (blocks > 0x7FFFFFFF) return fail(DNH_ERR_NOT_SUPPORTED, "dnh_dot: too many output tiles");
            g.xcd_chunk = (blocks % 8 == 0 && blocks >= 64) ? (uint32_t)(blocks / 8) : 0u;
#define DNH_I8_LAUNCH(TL, AK, BK_) do { \
                static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_i32_i8parts_kernel<TL, AK, BK_>), \
                                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)kI8LdsBytes); \
                if (attr != hipSuccess) return fail(DNH_ERR_HIP, "dnh_dot: %s", hipGetErrorString(attr)); \
                hipLaunchKernelGGL((gemm_i32_i8parts_kernel<TL, AK, BK_>), dim3((unsigned)blocks), dim3(kI8Threads), kI8LdsBytes, stream, \
                                   (uint32_t*)c, (const uint32_t*)a, (const uint32_t*)b, g); } while (0)
#define DNH_I8_AB(TL) do { if (a_kc) { if (b_kc) DNH_I8_LAUNCH(TL, true, true); else DNH_I8_LAUNCH(TL, true, false); } \
                           else { if (b_kc) DNH_I8_LAUNCH(TL, false, true); else DNH_I8_LAUNCH(TL, false, false); } } while (0)
            if (g.K % kI8BK) DNH_I8_AB(true); else DNH_I8_AB(false);
#undef DNH_I8_AB
#undef DNH_I8_LAUNCH
            DNH_LAUNCH_CHECK();
            return DNH_OK;
        }
    }
    if constexpr (sizeof(T) == 8) {
        bool a_kc = g.sak == 1, b_kc = g.sbk == 1;
        if (g.K >= kI8BK && (a_kc || g.sam == 1) && (b_kc || g.sbn == 1) && use_int_mfma()) {
            g.tiles_m = (uint32_t)cdiv(g.M, (int64_t)kI64BM);
            g.tiles_n = (uint32_t)cdiv(g.N, (int64_t)kI64BN);
            const int64_t blocks = (int64_t)g.tiles_m * g.tiles_n * batch;
            if (blocks > 0x7FFFFFFF) return fail(DNH_ERR_NOT_SUPPORTED, "dnh_dot: too many output tiles");
            g.xcd_chunk = (blocks % 8 == 0 && blocks >= 64) ? (uint32_t)(blocks / 8) : 0u;
#define DNH_I64_LAUNCH(TL, AK, BK_) do { \
                static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_i64_i8parts_kernel<TL, AK, BK_>), \
                                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)kI64LdsBytes); \
                if (attr != hipSuccess) return fail(DNH_ERR_HIP, "dnh_dot: %s", hipGetErrorString(attr)); \
                hipLaunchKernelGGL((gemm_i64_i8parts_kernel<TL, AK, BK_>), dim3((unsigned)blocks), dim3(kI8Threads), kI64LdsBytes, stream, \
                                   (uint64_t*)c, (const uint64_t*)a, (const uint64_t*)b, g); } while (0)
#define DNH_I64_AB(TL) do { if (a_kc) { if (b_kc) DNH_I64_LAUNCH(TL, true, true); else DNH_I64_LAUNCH(TL, true, false); } \
                            else { if (b_kc) DNH_I64_LAUNCH(TL, false, true); else DNH_I64_LAUNCH(TL, false, false); } } while (0)
            if (g.K % kI8BK) DNH_I64_AB(true); else DNH_I64_AB(false);
#undef DNH_I64_AB
#undef DNH_I64_LAUNCH
            DNH_LAUNCH_CHECK();
            return DNH_OK;
        }
    }

    g.tiles_m = cdiv(g.M, 64);
    g.tiles_n = cdiv(g.N, 64);
    const int64_t blocks = (int64_t)g.tiles_m * g.tiles_n * batch;
    if (blocks > 0x7FFFFFFF) return fail(DNH_ERR_NOT_SUPPORTED, "dnh_dot: too many output tiles");
    hipLaunchKernelGGL((gemm_int_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream, c, a, b, g);
    DNH_LAUNCH_CHECK();
    return DNH_OK;
}

}  // namespace

namespace dnh {
// c[b] (M x N, row stride ldc) += a[b] (M x K, row stride lda) . b[b] (K x N, row stride ldb) for b < batch; all row-major.
int32_t gemm_accumulate(int32_t dtype, void* c, const void* a, const void* b, int64_t M, int64_t N, int64_t K, int64_t lda,
                        int64_t ldb, int64_t ldc, int64_t batch, int64_t bsa, int64_t bsb, int64_t bsc, hipStream_t stream) {
    if (M == 0 || N == 0 || K == 0 || batch == 0) return DNH_OK;
    if (batch > 0xFFFFFFFFLL) return fail(DNH_ERR_NOT_SUPPORTED, "gemm_accumulate: batch too large");
    GemmArgs g;
    memset(&g, 0, sizeof(g));
    g.M = M; g.N = N; g.K = K;
    g.sam = lda; g.sak = 1; g.sbk = ldb; g.sbn = 1; g.scm = ldc; g.scn = 1;
    g.accumulate = 1;
    if (batch > 1) {
        g.nbatch = 1;
        g.bshape[0] = (uint32_t)batch;
        g.bsa[0] = bsa; g.bsb[0] = bsb; g.bsc[0] = bsc;
    }
    g.tiles_m = cdiv(M, BM);
    g.tiles_n = cdiv(N, BN);
    if (dtype == DNH_F32) return launch_gemm<float>(g, (float*)c, (const float*)a, (const float*)b, batch, stream);
    if (dtype == DNH_F64) return launch_gemm<double>(g, (double*)c, (const double*)a, (const double*)b, batch, stream);
    return fail(DNH_ERR_NOT_SUPPORTED, "gemm_accumulate: only single and double");
}
}  // namespace dnh

extern "C" int32_t dnh_dot(const DnhTensor* t, const DnhTensor* a, const DnhTensor* b, void* stream) {
    DNH_TRY(ensure_init());
    DNH_TRY(check_tensor(t, "dnh_dot"));
    DNH_TRY(check_tensor(a, "dnh_dot"));
    DNH_TRY(check_tensor(b, "dnh_dot"));
    if (t->dtype != a->dtype || t->dtype != b->dtype) return fail(DNH_ERR_INVALID_ARG, "dnh_dot: dtypes differ");
    if (t->dtype == DNH_BOOL) return fail(DNH_ERR_NOT_SUPPORTED, "dnh_dot: multiplication is not defined for bool");
    const int nt = t->ndims, na = a->ndims, nb = b->ndims;
    GemmArgs g;
    memset(&g, 0, sizeof(g));
    int64_t batch = 1;
    if (nt == 0 && na == 1 && nb == 1) {
        if (a->shape[0] != b->shape[0]) return fail(DNH_ERR_INVALID_ARG, "dnh_dot: vector lengths differ");
        g.M = 1; g.N = 1; g.K = a->shape[0];
        g.sak = a->stride[0]; g.sbk = b->stride[0];
    } else if (nt == 1 && na == 2 && nb == 1) {
        if (t->shape[0] != a->shape[0] || a->shape[1] != b->shape[0]) return fail(DNH_ERR_INVALID_ARG, "dnh_dot: matrix-vector shapes do not agree");
        g.M = a->shape[0]; g.N = 1; g.K = a->shape[1];
        g.sam = a->stride[0]; g.sak = a->stride[1]; g.sbk = b->stride[0]; g.scm = t->stride[0];
    } else if (nt >= 2 && na == nt && nb == nt) {
        g.M = a->shape[na - 2]; g.K = a->shape[na - 1]; g.N = b->shape[nb - 1];
        if (b->shape[nb - 2] != g.K || t->shape[nt - 2] != g.M || t->shape[nt - 1] != g.N)
            return fail(DNH_ERR_INVALID_ARG, "dnh_dot: matrix shapes do not agree");
        g.sam = a->stride[na - 2]; g.sak = a->stride[na - 1];
        g.sbk = b->stride[nb - 2]; g.sbn = b->stride[nb - 1];
        g.scm = t->stride[nt - 2]; g.scn = t->stride[nt - 1];
        for (int d = 0; d < nt - 2; d++) {
            if (a->shape[d] != t->shape[d] || b->shape[d] != t->shape[d]) return fail(DNH_ERR_INVALID_ARG, "dnh_dot: batch dimensions are not broadcast to the target's");
            if (t->shape[d] == 1) continue;
            if (t->shape[d] > 0xFFFFFFFFLL) return fail(DNH_ERR_NOT_SUPPORTED, "dnh_dot: batch extent too large");
            g.bshape[g.nbatch] = (uint32_t)t->shape[d];
            g.bsa[g.nbatch] = a->stride[d];
            g.bsb[g.nbatch] = b->stride[d];
            g.bsc[g.nbatch] = t->stride[d];
            g.nbatch++;
            batch *= t->shape[d];
        }
    } else {
        return fail(DNH_ERR_INVALID_ARG, "dnh_dot: ranks (%d, %d, %d) match no dot variant", nt, na, nb);
    }
    if (g.M == 0 || g.N == 0 || batch == 0) return DNH_OK;
    g.tiles_m = cdiv(g.M, BM);
    g.tiles_n = cdiv(g.N, BN);
    hipStream_t s = (hipStream_t)stream;
    int32_t st = DNH_OK;
    if (!dtype_is_fp(t->dtype)) {
        if (g.N == 1 && g.nbatch == 0 && g.K > 0) {
            // vector forms: element-wise product into a temporary, then its fold along k: both at memory speed, whatever M and K are
            const int es = dtype_size(t->dtype);
            void* tmp = nullptr;
            DNH_TRY(dnh_alloc_async((size_t)g.M * (size_t)g.K * es, s, &tmp));
            DnhTensor pd, ad, bd;
            memset(&pd, 0, sizeof(pd));
            pd.base = tmp; pd.ndims = 2; pd.dtype = t->dtype;
            pd.shape[0] = g.M; pd.shape[1] = g.K; pd.stride[0] = g.K; pd.stride[1] = 1;
            ad = pd; ad.base = a->base; ad.offset = a->offset; ad.stride[0] = g.sam; ad.stride[1] = g.sak;
            bd = pd; bd.base = b->base; bd.offset = b->offset; bd.stride[0] = 0; bd.stride[1] = g.sbk;
            DnhTensor td = *t;
            td.ndims = 1; td.shape[0] = g.M; td.stride[0] = g.scm;
            st = dnh_binary(DNH_MULTIPLY, &pd, &ad, &bd, stream);
            if (st == DNH_OK) st = dnh_reduce_last_axis(DNH_SUM, &td, &pd, stream);
            (void)dnh_free_async(tmp, s);
            return st;
        }
#define DNH_INT_DOT(DT, CT) case DT: return launch_gemm_int<CT>(g, (CT*)elem_ptr(t), (const CT*)elem_ptr(a), (const CT*)elem_ptr(b), batch, s);
        switch (t->dtype) {
            DNH_INT_DOT(DNH_U8, uint8_t) DNH_INT_DOT(DNH_I8, int8_t) DNH_INT_DOT(DNH_I16, int16_t) DNH_INT_DOT(DNH_U16, uint16_t) DNH_INT_DOT(DNH_I32, int32_t) DNH_INT_DOT(DNH_U32, uint32_t)
            DNH_INT_DOT(DNH_I64, int64_t) DNH_INT_DOT(DNH_U64, uint64_t)
        }
#undef DNH_INT_DOT
        return fail(DNH_ERR_NOT_SUPPORTED, "dnh_dot: unsupported element type");
    }
    if (t->dtype == DNH_F32 && try_gemv<float>(g, (float*)elem_ptr(t), (const float*)elem_ptr(a), (const float*)elem_ptr(b), s, &st)) return st;
    if (t->dtype == DNH_F64 && try_gemv<double>(g, (double*)elem_ptr(t), (const double*)elem_ptr(a), (const double*)elem_ptr(b), s, &st)) return st;
    if (t->dtype == DNH_F32) return launch_gemm<float>(g, (float*)elem_ptr(t), (const float*)elem_ptr(a), (const float*)elem_ptr(b), batch, s);
    return launch_gemm<double>(g, (double*)elem_ptr(t), (const double*)elem_ptr(a), (const double*)elem_ptr(b), batch, s);
}
