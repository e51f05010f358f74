// dnh_batched_svd, dnh_symmetric_eig: ITensorBackend BatchedSVD and SymmetricEigenDecomposition (Tensor/Tensor/TensorBackend.fs:143,
// 145).  The reference's host backend calls LAPACK gesdd / syevd (Tensor/Tensor/Host/HostBackend.fs:579-628); its CUDA backend
// does not implement either (Tensor/Tensor/Cuda/CudaBackend.fs:486-492).
//
// Both run on one-sided Jacobi (Hestenes) rotations: for two columns x_p, x_q of a work matrix X (R rows, C <= R columns, every
// column contiguous) a plane rotation makes them orthogonal, and the same rotation is applied to the columns of W, which starts
// as the identity.  When a sweep over all pairs rotates nothing, X = A W has orthogonal columns: their norms are the singular
// values, the normalised columns the left vectors, W the right vectors.  The sweeps run on blocks of 16 columns (see "block
// rounds" below): the rotations of a pair of blocks are found from its 32 x 32 Gram matrix and applied as one 32 x 32 factor.
//
//   SVD of A (M x N):  the side with fewer vectors plays W (it comes out complete); the taller side's vectors are the
//     normalised columns of X for the singular values above 4 eps * sigma_max, and an orthonormal basis of their
//     complement for the rest: the Householder QR of the columns found so far, Q^T U1 = [D; 0], and Q applied to the unit
//     vectors that remain.
//   Symmetric eigendecomposition:  the chosen triangle is mirrored, the matrix shifted by mu = its Frobenius norm so that it is
//     positive semidefinite (equal magnitudes of opposite sign would otherwise share a singular subspace); then the singular
//     values are lambda + mu and W holds the eigenvectors.  Absolute error of the eigenvalues: a few eps * |A|, as syevd's.
#include "common.h"
#include "wave_argmax.h"

#include <algorithm>
#include <limits>
#include <vector>

using namespace dnh;

namespace {

constexpr int kPairThreads = 256;
constexpr int kMaxSweeps = 60;

// Players a, b of pair k in round r of the round-robin schedule for an even number `ce` of players: player ce - 1 stays, the
// others rotate.  Players >= c are byes (c odd).
__device__ __forceinline__ void pair_of(int ce, int r, int k, int* a, int* b) {
    const int m = ce - 1;
    if (k == 0) {
        *a = m;
        *b = r % m;
    } else {
        *a = (r + k) % m;
        *b = (r - k + m) % m;
    }
}

// Sum of one value per thread over the workgroup (kPairThreads threads).
__device__ __forceinline__ double block_sum(double v, double* red) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    __syncthreads();   // red may still be read from the previous call
    if (lane == 0) red[w] = v;
    __syncthreads();
    double s = 0;
#pragma unroll
    for (int i = 0; i < kPairThreads / 64; i++) s += red[i];
    return s;
}

// ---- block rounds ---------------------------------------------------------------------------------------------------------
// Blocks of 16 columns are paired by the round-robin schedule (blocks / 2 disjoint pairs per round, blocks - 1 rounds per sweep).
// For a pair of blocks (32 columns B) the 32 x 32 Gram matrix G = B^T B is formed on the matrix cores, G is diagonalised by
// cyclic two-sided Jacobi rotations in LDS while the rotations accumulate in Q (G <- J^T G J, Q <- Q J), and the columns are
// replaced by B Q (the same columns of W by W Q), again on the matrix cores.  The entries of G are the sums
// alpha = |x_p|^2, beta = |x_q|^2, gamma = x_p . x_q that define the rotation of columns p, q (a pair is rotated when
// |gamma| > tol sqrt(alpha beta), tol = sqrt(rows) eps as in LAPACK's xGESVJ); one round moves the matrices once for
// 16 x 16 + 2 * 120 column pairs.  A sweep in which no workgroup finds an entry of its G above the threshold ends the iteration.  There are only C / 32 pairs, too few workgroups for the two passes over the rows, so a round
// is three launches: the partial Gram matrices of every (pair, piece of the rows); per pair the sum of the pieces and the
// diagonalisation (Q to memory); Q applied to every (pair, piece of the rows of X and of W).
typedef double f64x4 __attribute__((ext_vector_type(4)));
constexpr int kBlockCols = 16;

// Four consecutive elements p[i .. i+3] of a column of `n` elements, raw: the caller converts (and zeroes what `ok4` excludes)
// when it uses them, so that the loads of the next step stay in flight during the matrix instructions of the current one.
template <class T>
struct Raw4 {
    T v[4];
};
template <class T>
__device__ __forceinline__ Raw4<T> load4_raw(const T* __restrict__ p, int i, int n, bool ok, bool vec) {
    Raw4<T> r;
    if (vec && i + 4 <= n) {
        typedef T V4 __attribute__((ext_vector_type(4), aligned(16)));
        const V4 v = *reinterpret_cast<const V4*>(p + i);
#pragma unroll
        for (int j = 0; j < 4; j++) r.v[j] = v[j];
    } else {
#pragma unroll
        for (int j = 0; j < 4; j++) r.v[j] = p[(ok && i + j < n) ? i + j : 0];
    }
    return r;
}

// Rows of M (`n` per column, columns of the two blocks at pcol / qcol) times Q: one wavefront per 16 rows.  Computed as
// (Q^T M^T): operand lane l supplies Q[4s + l/16][16t + l%16] and M[row0 + l%16][column 4s + l/16]; accumulator register r
// holds row l%16 of column 16t + 4r + l/16, so a store instruction writes 16 consecutive rows of four columns.
template <class T, int NW>
__device__ __forceinline__ void apply_block_rotation(T* __restrict__ m, int n, int begin, int end, int c, int pcol, int qcol, const double* __restrict__ Q, int wave,
                                                     int lane) {
    constexpr int STEP = NW * 16;
    const int lc = lane & 15, lk = lane >> 4;
    double qa[8][2];
#pragma unroll
    for (int s = 0; s < 8; s++) {
        qa[s][0] = Q[(4 * s + lk) * 32 + lc];
        qa[s][1] = Q[(4 * s + lk) * 32 + 16 + lc];
    }
    int64_t off[8];
    unsigned col_ok = 0;
#pragma unroll
    for (int s = 0; s < 8; s++) {
        const int col = (s < 4 ? pcol : qcol - 16) + 4 * s + lk;
        if (col < c) col_ok |= 1u << s;
        off[s] = col < c ? (int64_t)col * n : 0;
    }
    T cur[8], nxt[8];
    int r0 = begin + wave * 16;
    if (r0 < end) {
        const int row = r0 + lc < n ? r0 + lc : 0;
#pragma unroll
        for (int s = 0; s < 8; s++) cur[s] = m[off[s] + row];
    }
    for (; r0 < end; r0 += STEP) {
        const int rn = r0 + STEP;
        if (rn < end) {
            const int row = rn + lc < n ? rn + lc : 0;
#pragma unroll
            for (int s = 0; s < 8; s++) nxt[s] = m[off[s] + row];
        }
        const int row = r0 + lc;
        const bool row_ok = row < n;
        f64x4 acc0 = {0, 0, 0, 0}, acc1 = {0, 0, 0, 0};
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const double xs = (row_ok && ((col_ok >> s) & 1u)) ? (double)cur[s] : 0.0;
            acc0 = __builtin_amdgcn_mfma_f64_16x16x4f64(qa[s][0], xs, acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f64_16x16x4f64(qa[s][1], xs, acc1, 0, 0, 0);
        }
        if (row_ok) {
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int cp = pcol + 4 * r + lk, cq = qcol + 4 * r + lk;
                if (cp < c) m[(int64_t)cp * n + row] = (T)acc0[r];
                if (cq < c) m[(int64_t)cq * n + row] = (T)acc1[r];
            }
        }
#pragma unroll
        for (int s = 0; s < 8; s++) cur[s] = nxt[s];
    }
}

// Partial Gram matrices: workgroup (pair, piece, matrix) covers rows [piece * chunk, (piece + 1) * chunk) (chunk a multiple of 16)
// and writes G_pp, G_pq, G_qq (3 x 256 doubles) to partial[((matrix * pairs + pair) * pieces + piece) * 768].
constexpr int kGramThreads = 256;
template <class T>
__global__ __launch_bounds__(kGramThreads) void jacobi_block_gram_kernel(const T* __restrict__ x, double* __restrict__ partial, int rows, int chunk, int c, int nbe,
                                                                         int round, int64_t bsx) {
    constexpr int NW = kGramThreads / 64;
    __shared__ double part[NW][3][256];
    int ba, bb;
    pair_of(nbe, round, blockIdx.x, &ba, &bb);
    const int nb = (c + kBlockCols - 1) / kBlockCols;
    if (ba >= nb && bb >= nb) return;   // a block paired with the bye still rotates its own columns (the other 16 read as zero)
    const int pcol = (ba < bb ? ba : bb) * kBlockCols, qcol = (ba < bb ? bb : ba) * kBlockCols;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lc = lane & 15, lk = lane >> 4;
    const T* xb = x + (int64_t)blockIdx.z * bsx;
    const int begin = (int)blockIdx.y * chunk, end = begin + chunk < rows ? begin + chunk : rows;
    // operand lane l supplies rows r0 + 4 (l/16) + j (j = 0..3 over four MFMAs) of column l%16 of each block
    const bool okp = pcol + lc < c, okq = qcol + lc < c;
    const T* xp = xb + (int64_t)(okp ? pcol + lc : 0) * rows;
    const T* xq = xb + (int64_t)(okq ? qcol + lc : 0) * rows;
    const bool vec = (rows & 3) == 0;
    f64x4 gpp = {0, 0, 0, 0}, gpq = {0, 0, 0, 0}, gqq = {0, 0, 0, 0};
    Raw4<T> ca, cb, na, nb4;
    int r0 = begin + wave * 16;
    if (r0 < end) {
        ca = load4_raw(xp, r0 + 4 * lk, rows, okp, vec);
        cb = load4_raw(xq, r0 + 4 * lk, rows, okq, vec);
    }
    for (; r0 < end; r0 += NW * 16) {
        const int rn = r0 + NW * 16;
        if (rn < end) {
            na = load4_raw(xp, rn + 4 * lk, rows, okp, vec);
            nb4 = load4_raw(xq, rn + 4 * lk, rows, okq, vec);
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const bool in = r0 + 4 * lk + j < rows;
            const double a = (in && okp) ? (double)ca.v[j] : 0.0;
            const double b = (in && okq) ? (double)cb.v[j] : 0.0;
            gpp = __builtin_amdgcn_mfma_f64_16x16x4f64(a, a, gpp, 0, 0, 0);
            gpq = __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, gpq, 0, 0, 0);
            gqq = __builtin_amdgcn_mfma_f64_16x16x4f64(b, b, gqq, 0, 0, 0);
        }
        ca = na;
        cb = nb4;
    }
#pragma unroll
    for (int r = 0; r < 4; r++) {
        part[wave][0][(4 * r + lk) * 16 + lc] = gpp[r];
        part[wave][1][(4 * r + lk) * 16 + lc] = gpq[r];
        part[wave][2][(4 * r + lk) * 16 + lc] = gqq[r];
    }
    __syncthreads();
    double* out = partial + (((int64_t)blockIdx.z * gridDim.x + blockIdx.x) * gridDim.y + blockIdx.y) * 768;
    const int t = threadIdx.x;
    if (t < 256)
#pragma unroll
    for (int s = 0; s < 3; s++) {
        double v = 0;
#pragma unroll
        for (int k = 0; k < NW; k++) v += part[k][s][t];
        out[s * 256 + t] = v;
    }
}

// Single precision: the same two passes on v_mfma_f32_32x32x2_f32, whose accumulator is the whole 32 x 32 matrix.  Rounding
// the sums of a piece to single precision perturbs gamma by about eps * |x_p| |x_q|, well below the rotation threshold
// sqrt(rows) * eps * |x_p| |x_q|; the pieces are added in double precision.
typedef float f32x16 __attribute__((ext_vector_type(16)));
__device__ __forceinline__ int block_pair_column(int k, int pcol, int qcol) { return k < 16 ? pcol + k : qcol + k - 16; }

__global__ __launch_bounds__(kGramThreads) void jacobi_block_gram_f32_kernel(const float* __restrict__ x, double* __restrict__ partial, int rows, int chunk, int c,
                                                                             int nbe, int round, int64_t bsx) {
    constexpr int NW = kGramThreads / 64;
    __shared__ float part[NW][3][256];
    int ba, bb;
    pair_of(nbe, round, blockIdx.x, &ba, &bb);
    const int nb = (c + kBlockCols - 1) / kBlockCols;
    if (ba >= nb && bb >= nb) return;   // a block paired with the bye still rotates its own columns (the other 16 read as zero)
    const int pcol = (ba < bb ? ba : bb) * kBlockCols, qcol = (ba < bb ? bb : ba) * kBlockCols;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lm = lane & 31, lk = lane >> 5;
    const int begin = (int)blockIdx.y * chunk, end = begin + chunk < rows ? begin + chunk : rows;
    // operand lane l supplies rows r0 + 8 h + 4 (l/32) + j (h = 0, 1; j = 0..3: eight MFMAs per 16 rows) of column l%32 of the pair
    const int col = block_pair_column(lm, pcol, qcol);
    const bool ok = col < c;
    const float* xc = x + (int64_t)blockIdx.z * bsx + (int64_t)(ok ? col : 0) * rows;
    const bool vec = (rows & 3) == 0;
    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.0f;
    Raw4<float> c0, c1, n0, n1;
    int r0 = begin + wave * 16;
    if (r0 < end) {
        c0 = load4_raw(xc, r0 + 4 * lk, rows, ok, vec);
        c1 = load4_raw(xc, r0 + 8 + 4 * lk, rows, ok, vec);
    }
    for (; r0 < end; r0 += NW * 16) {
        const int rn = r0 + NW * 16;
        if (rn < end) {
            n0 = load4_raw(xc, rn + 4 * lk, rows, ok, vec);
            n1 = load4_raw(xc, rn + 8 + 4 * lk, rows, ok, vec);
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float a = (ok && r0 + 4 * lk + j < rows) ? c0.v[j] : 0.0f;
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, a, acc, 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float a = (ok && r0 + 8 + 4 * lk + j < rows) ? c1.v[j] : 0.0f;
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, a, acc, 0, 0, 0);
        }
        c0 = n0;
        c1 = n1;
    }
    // accumulator register r of lane l holds G[8 (r/4) + 4 (l/32) + r%4][l%32]; the lower left block is the transpose of the upper right
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int row = 8 * (r >> 2) + 4 * lk + (r & 3);
        if (row < 16) part[wave][lm < 16 ? 0 : 1][row * 16 + (lm & 15)] = acc[r];
        else if (lm >= 16) part[wave][2][(row - 16) * 16 + lm - 16] = acc[r];
    }
    __syncthreads();
    double* out = partial + (((int64_t)blockIdx.z * gridDim.x + blockIdx.x) * gridDim.y + blockIdx.y) * 768;
    const int t = threadIdx.x;
    if (t < 256)
#pragma unroll
    for (int s = 0; s < 3; s++) {
        double v = 0;
#pragma unroll
        for (int k = 0; k < NW; k++) v += (double)part[k][s][t];
        out[s * 256 + t] = v;
    }
}

// Rows [begin, end) of M times Q in single precision, 32 rows per wavefront step: operand lane l supplies Q[2s + l/32][l%32] and
// M[row0 + l%32][column 2s + l/32]; accumulator register r holds row l%32 of column 8 (r/4) + 4 (l/32) + r%4: a store
// instruction writes 32 consecutive rows (a whole 128-byte line) of two columns.
template <int NW>
__device__ __forceinline__ void apply_block_rotation_f32(float* __restrict__ m, int n, int begin, int end, int c, int pcol, int qcol, const double* __restrict__ Q,
                                                         int wave, int lane) {
    constexpr int STEP = NW * 32;
    const int lm = lane & 31, lk = lane >> 5;
    float qa[16];
    int64_t off[16];
    unsigned col_ok = 0;
#pragma unroll
    for (int s = 0; s < 16; s++) {
        qa[s] = (float)Q[(2 * s + lk) * 32 + lm];
        const int col = block_pair_column(2 * s + lk, pcol, qcol);
        if (col < c) col_ok |= 1u << s;
        off[s] = col < c ? (int64_t)col * n : 0;
    }
    float cur[16], nxt[16];
    int r0 = begin + wave * 32;
    if (r0 < end) {
        const int row = r0 + lm < n ? r0 + lm : 0;
#pragma unroll
        for (int s = 0; s < 16; s++) cur[s] = m[off[s] + row];
    }
    for (; r0 < end; r0 += STEP) {
        const int rn = r0 + STEP;
        if (rn < end) {
            const int row = rn + lm < n ? rn + lm : 0;
#pragma unroll
            for (int s = 0; s < 16; s++) nxt[s] = m[off[s] + row];
        }
        const int row = r0 + lm;
        const bool row_ok = row < n;
        f32x16 acc;
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = 0.0f;
#pragma unroll
        for (int s = 0; s < 16; s++) {
            const float xs = (row_ok && ((col_ok >> s) & 1u)) ? cur[s] : 0.0f;
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(qa[s], xs, acc, 0, 0, 0);
        }
        if (row_ok) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int col = block_pair_column(8 * (r >> 2) + 4 * lk + (r & 3), pcol, qcol);
                if (col < c) m[(int64_t)col * n + row] = acc[r];
            }
        }
#pragma unroll
        for (int s = 0; s < 16; s++) cur[s] = nxt[s];
    }
}

// The second launch of a round, one workgroup per pair: G from the pieces, its diagonalisation; Q goes to qbuf[pair][32][32] and
// flag[pair] says whether anything was rotated (the third launch skips the pair otherwise).  `full`: one cyclic sweep over all
// 496 column pairs of the 32 (31 steps of 16 disjoint pairs); otherwise only the 256 pairs between the two blocks (16 steps): the
// pairs inside a block were made orthogonal when the block last had its full round (one round of every sweep, a different one
// each sweep so that the block that sits out changes) and are disturbed by the other rotations only to second order.
constexpr int kSolveThreads = 256;
template <class T>
__global__ __launch_bounds__(kSolveThreads) void jacobi_block_solve_kernel(const double* __restrict__ partial, int pieces, double* __restrict__ qbuf,
                                                                           int* __restrict__ flag, int c, int nbe, int round, int full, double tol,
                                                                           int* rotations) {
    __shared__ double G[32][33];
    __shared__ double Q[32][33];
    __shared__ double H[32][33];
    __shared__ int above;
    int ba, bb;
    pair_of(nbe, round, blockIdx.x, &ba, &bb);
    const int nb = (c + kBlockCols - 1) / kBlockCols;
    if (ba >= nb && bb >= nb) return;   // a block paired with the bye still rotates its own columns (the other 16 read as zero)
    const int64_t pair_id = (int64_t)blockIdx.y * gridDim.x + blockIdx.x;
    const double* part = partial + pair_id * pieces * 768;
    if (threadIdx.x == 0) above = 0;
    __syncthreads();
    if (threadIdx.x < 256) {
        const int t = threadIdx.x, i = t >> 4, j = t & 15;
        double pp = 0, pq = 0, qq = 0;
        for (int k = 0; k < pieces; k++) {
            pp += part[k * 768 + t];
            pq += part[k * 768 + 256 + t];
            qq += part[k * 768 + 512 + t];
        }
        G[i][j] = pp;
        G[i][16 + j] = pq;
        G[16 + j][i] = pq;
        G[16 + i][16 + j] = qq;
    }
    for (int e = threadIdx.x; e < 1024; e += kSolveThreads) Q[e >> 5][e & 31] = (e >> 5) == (e & 31) ? 1.0 : 0.0;
    __syncthreads();
    // anything to rotate at all?
    for (int e = threadIdx.x; e < 1024; e += kSolveThreads) {
        const int i = e >> 5, j = e & 31;
        if (i < j) {
            const double g = G[i][j];
            if (g != 0.0 && fabs(g) > tol * sqrt(G[i][i] * G[j][j])) above = 1;
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) flag[pair_id] = above;
    if (!above) return;   // uniform
    if (threadIdx.x == 0) *rotations = 1;

    // Two tasks per thread and step: pair k of the step and the indices i, i + 16.  Every thread derives its pair's rotation
    // itself from the three entries of G (same inputs, same instructions: the same bits in every thread), rotates columns p, q
    // of rows i, i + 16 of G into H and of Q in place, and after the barrier rows p, q of columns i, i + 16 of H back into G.
    static_assert(kSolveThreads == 256, "two (pair, index) tasks per thread");
    {
        const int k = threadIdx.x & 15, i = threadIdx.x >> 4;
        const double tol2 = tol * tol;
        const int steps = full ? 31 : 16;
        for (int r = 0; r < steps; r++) {
            int p, q;
            if (full) {
                // pair k of round r among 32 players (pair_of without its divisions: r < 31, k < 16)
                int a = k == 0 ? 31 : r + k, b = k == 0 ? r : r - k;
                if (k != 0 && a >= 31) a -= 31;
                if (b < 0) b += 31;
                p = a < b ? a : b;
                q = a < b ? b : a;
            } else {
                p = k;
                q = 16 + ((k + r) & 15);
            }
            const double alpha = G[p][p], beta = G[q][q], gamma = G[p][q];
            double cs = 1.0, sn = 0.0;
            if (gamma * gamma > tol2 * alpha * beta) {
                // tan of the rotation angle to single precision on operands scaled into [-1, 1] (an angle that is off by 1e-7 of
                // itself leaves 1e-7 of gamma behind, far below what the next visit removes anyway); cos and sin from it in
                // double precision, so that the rotation is orthogonal to working accuracy: 1 / sqrt(1 + t^2) by two Newton steps.
                const double d = beta - alpha, g2 = 2.0 * gamma;
                const double big = fabs(d) > fabs(g2) ? fabs(d) : fabs(g2);
                const int e = __builtin_amdgcn_frexp_exp(big);
                const float df = (float)ldexp(d, -e), gf = (float)ldexp(g2, -e);
                const float hf = __builtin_sqrtf(df * df + gf * gf);
                const float tf = gf * __builtin_amdgcn_rcpf(df >= 0.0f ? df + hf : df - hf);
                double t = (double)tf;
                if (tf == 0.0f) {   // |gamma| below single precision's range next to |beta - alpha|: the same formula in double precision
                    const double zeta = d / g2;
                    t = (zeta >= 0.0 ? 1.0 : -1.0) / (fabs(zeta) + sqrt(1.0 + zeta * zeta));
                }
                const double x = 1.0 + t * t;
                double y = (double)__builtin_amdgcn_rsqf((float)x);
                y = y * (1.5 - 0.5 * x * y * y);
                y = y * (1.5 - 0.5 * x * y * y);
                cs = y;
                sn = y * t;
            }
#pragma unroll
            for (int ii = i; ii < 32; ii += 16) {
                const double u = G[ii][p], v = G[ii][q];
                H[ii][p] = cs * u - sn * v;
                H[ii][q] = sn * u + cs * v;
                if (sn != 0.0) {
                    const double qu = Q[ii][p], qv = Q[ii][q];
                    Q[ii][p] = cs * qu - sn * qv;
                    Q[ii][q] = sn * qu + cs * qv;
                }
            }
            __syncthreads();
#pragma unroll
            for (int ii = i; ii < 32; ii += 16) {
                const double u = H[p][ii], v = H[q][ii];
                G[p][ii] = cs * u - sn * v;
                G[q][ii] = sn * u + cs * v;
            }
            __syncthreads();
        }
    }
    for (int e = threadIdx.x; e < 1024; e += kSolveThreads) qbuf[pair_id * 1024 + e] = Q[e >> 5][e & 31];
}

// The third launch: workgroup (pair, piece, matrix) applies its pair's Q to its piece of the rows of X (pieces 0 .. xpieces - 1) or
// of W (the pieces after those).
constexpr int kApplyThreads = 256;
template <class T>
__global__ __launch_bounds__(kApplyThreads) void jacobi_block_apply_kernel(T* __restrict__ x, T* __restrict__ w, const double* __restrict__ qbuf,
                                                                           const int* __restrict__ flag, int rows, int chunk, int xpieces, int wrows, int wchunk,
                                                                           int c, int nbe, int round, int64_t bsx, int64_t bsw) {
    int ba, bb;
    pair_of(nbe, round, blockIdx.x, &ba, &bb);
    const int nb = (c + kBlockCols - 1) / kBlockCols;
    if (ba >= nb && bb >= nb) return;   // a block paired with the bye still rotates its own columns (the other 16 read as zero)
    const int64_t pair_id = (int64_t)blockIdx.z * gridDim.x + blockIdx.x;
    if (!flag[pair_id]) return;
    const int pcol = (ba < bb ? ba : bb) * kBlockCols, qcol = (ba < bb ? bb : ba) * kBlockCols;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const double* Q = qbuf + pair_id * 1024;
    if ((int)blockIdx.y < xpieces) {
        const int begin = (int)blockIdx.y * chunk, end = begin + chunk < rows ? begin + chunk : rows;
        if constexpr (sizeof(T) == 4) apply_block_rotation_f32<kApplyThreads / 64>(x + (int64_t)blockIdx.z * bsx, rows, begin, end, c, pcol, qcol, Q, wave, lane);
        else apply_block_rotation<T, kApplyThreads / 64>(x + (int64_t)blockIdx.z * bsx, rows, begin, end, c, pcol, qcol, Q, wave, lane);
    } else {
        const int begin = ((int)blockIdx.y - xpieces) * wchunk, end = begin + wchunk < wrows ? begin + wchunk : wrows;
        if constexpr (sizeof(T) == 4) apply_block_rotation_f32<kApplyThreads / 64>(w + (int64_t)blockIdx.z * bsw, wrows, begin, end, c, pcol, qcol, Q, wave, lane);
        else apply_block_rotation<T, kApplyThreads / 64>(w + (int64_t)blockIdx.z * bsw, wrows, begin, end, c, pcol, qcol, Q, wave, lane);
    }
}

// identity matrices [batch][n][n]
template <class T>
__global__ __launch_bounds__(256) void identity_kernel(T* w, int n, int64_t total) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int64_t e = i % ((int64_t)n * n);
    w[i] = (e / n == e % n) ? T(1) : T(0);
}

// norm[b][j] = |column j|
template <class T>
__global__ __launch_bounds__(kPairThreads) void column_norm_kernel(const T* __restrict__ x, double* __restrict__ norm, int rows, int c, int64_t bsx) {
    __shared__ double red[kPairThreads / 64];
    const T* xc = x + (int64_t)blockIdx.y * bsx + (int64_t)blockIdx.x * rows;
    double s = 0;
    for (int i = threadIdx.x; i < rows; i += kPairThreads) {
        const double u = (double)xc[i];
        s += u * u;
    }
    s = block_sum(s, red);
    if (threadIdx.x == 0) norm[(int64_t)blockIdx.y * c + blockIdx.x] = sqrt(s);
}

// order[b][rank] = j with the keys in descending (or ascending) order; equal keys keep their index order
__global__ __launch_bounds__(256) void rank_kernel(const double* __restrict__ key, int* __restrict__ order, int c, int descending) {
    const int j = blockIdx.x * 256 + threadIdx.x;
    if (j >= c) return;
    const double* k = key + (int64_t)blockIdx.y * c;
    const double mine = k[j];
    int rank = 0;
    for (int i = 0; i < c; i++) {
        const double o = k[i];
        rank += (descending ? o > mine : o < mine) || (o == mine && i < j);
    }
    order[(int64_t)blockIdx.y * c + rank] = j;
}

// largest key of every matrix -> kmax[b]
__global__ __launch_bounds__(256) void max_key_kernel(const double* __restrict__ key, double* __restrict__ kmax, int c) {
    __shared__ double red[4];
    double m = 0;
    for (int i = threadIdx.x; i < c; i += 256) m = fmax(m, key[(int64_t)blockIdx.x * c + i]);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) m = fmax(m, __shfl_xor(m, off, 64));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) kmax[blockIdx.x] = fmax(fmax(red[0], red[1]), fmax(red[2], red[3]));
}

// Scaling by a power of two (exact): every matrix is brought to a largest magnitude in [0.5, 1) before the sweeps, so that the
// squares summed in the Gram entries neither overflow nor vanish whatever the magnitude of the input (single precision sums
// them on the matrix cores in single precision); the values are scaled back when they are written.
__global__ __launch_bounds__(64) void clear_scale_kernel(unsigned long long* maxbits, int count) {
    const int i = blockIdx.x * 64 + threadIdx.x;
    if (i < count) maxbits[i] = 0ull;
}
template <class T>
__global__ __launch_bounds__(256) void max_abs_kernel(const T* __restrict__ x, unsigned long long* __restrict__ maxbits, int64_t per_matrix) {
    __shared__ double red[4];
    const T* xb = x + (int64_t)blockIdx.y * per_matrix;
    double m = 0.0;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < per_matrix; i += (int64_t)gridDim.x * 256) {
        const double v = fabs((double)xb[i]);
        m = v > m ? v : m;   // NaN never enters
    }
    for (int o = 32; o > 0; o >>= 1) {
        const double other = __shfl_xor(m, o);
        m = other > m ? other : m;
    }
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int k = 1; k < 4; k++) m = red[k] > m ? red[k] : m;
        atomicMax(maxbits + blockIdx.y, (unsigned long long)__double_as_longlong(m));   // non-negative doubles order like their bits
    }
}
__device__ __forceinline__ int scale_exponent(unsigned long long bits) {
    const double m = __longlong_as_double((long long)bits);
    return (m > 0.0 && m <= 1.7976931348623157e308) ? __builtin_amdgcn_frexp_exp(m) : 0;
}
template <class T>
__global__ __launch_bounds__(256) void scale_down_kernel(T* __restrict__ x, const unsigned long long* __restrict__ maxbits, int* __restrict__ exps,
                                                         int64_t per_matrix) {
    const int e = scale_exponent(maxbits[blockIdx.y]);
    if (blockIdx.x == 0 && threadIdx.x == 0) exps[blockIdx.y] = e;
    if (e == 0) return;
    T* xb = x + (int64_t)blockIdx.y * per_matrix;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < per_matrix; i += (int64_t)gridDim.x * 256) xb[i] = (T)ldexp((double)xb[i], -e);
}

// out[b][k] = (T)(key[b][order[b][k]] + shift[b] * sign) for k < count
template <class T>
__global__ __launch_bounds__(256) void pick_values_kernel(T* __restrict__ out, const double* __restrict__ key, const int* __restrict__ order,
                                                          const double* __restrict__ shift, double sign, const int* __restrict__ exps, int c, int count) {
    const int k = blockIdx.x * 256 + threadIdx.x;
    if (k >= count) return;
    const int64_t b = blockIdx.y;
    const double v = key[b * c + order[b * c + k]] + (shift ? sign * shift[b] : 0.0);
    out[b * count + k] = (T)ldexp(v, exps[b]);
}

// Row-major output matrix [b][n][n] whose column k is column order[k] of the column-major work matrix src ([b][c][n]),
// divided by its norm when norms are given; columns k with norm <= rel * kmax (or k >= c) are left alone (they come from the
// complement) and counted in missing[b] by thread (0, 0).
template <class T>
__global__ __launch_bounds__(256) void scatter_columns_kernel(T* __restrict__ out, const T* __restrict__ src, const int* __restrict__ order,
                                                              const double* __restrict__ norm, const double* __restrict__ kmax, double rel,
                                                              int n, int c, int64_t bs_src) {
    const int i = blockIdx.x * 256 + threadIdx.x;   // row
    const int k = blockIdx.y;                        // output column
    const int64_t b = blockIdx.z;
    if (i >= n) return;
    const int j = order[b * c + k];
    double scale = 1.0;
    if (norm) {
        const double nj = norm[b * c + j];
        if (!(nj > rel * kmax[b]) || nj == 0.0) return;
        scale = 1.0 / nj;
    }
    out[(b * n + i) * (int64_t)n + k] = (T)((double)src[b * bs_src + (int64_t)j * n + i] * scale);
}

// rank[b] = number of columns whose norm exceeds rel * kmax[b]
__global__ __launch_bounds__(256) void numeric_rank_kernel(const double* __restrict__ norm, const double* __restrict__ kmax, double rel, int c,
                                                           int* __restrict__ rank) {
    __shared__ int red[4];
    int n = 0;
    for (int i = threadIdx.x; i < c; i += 256) {
        const double v = norm[(int64_t)blockIdx.x * c + i];
        n += (v > rel * kmax[blockIdx.x]) && v != 0.0;
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) n += __shfl_xor(n, off, 64);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = n;
    __syncthreads();
    if (threadIdx.x == 0) rank[blockIdx.x] = red[0] + red[1] + red[2] + red[3];
}

// ---- orthonormal completion of the taller side -----------------------------------------------------------------------------------
// U1 = the first rank[b] columns of the row-major u[b] (n x n) is orthonormal.  Its Householder QR, Q^T U1 = [D; 0] with D = diag(+-1),
// gives Q = H_0 H_1 ... H_{r-1} whose columns r .. n-1 span the complement: they are Q applied to the unit vectors e_r .. e_{n-1}.
// h[b][k][i] keeps column k (contiguous); below its diagonal it ends up holding the Householder vector v_k (v_k[k] = 1 implied).

// h[b][k][i] = u[b][i][k] for k < rank[b]
template <class T>
__global__ __launch_bounds__(256) void gather_u1_kernel(T* __restrict__ h, const T* __restrict__ u, const int* __restrict__ rank, int n, int c) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    const int k = blockIdx.y;
    const int64_t b = blockIdx.z;
    if (i >= n || k >= rank[b]) return;
    h[(b * c + k) * (int64_t)n + i] = u[(b * n + i) * (int64_t)n + k];
}

// Householder vector of column k (rows k .. n-1), one workgroup per matrix: tau[b][k], the vector scaled so that v[k] = 1
template <class T>
__global__ __launch_bounds__(kPairThreads) void house_vector_kernel(T* __restrict__ h, double* __restrict__ tau, const int* __restrict__ rank, int n,
                                                                    int c, int k) {
    __shared__ double red[kPairThreads / 64];
    const int64_t b = blockIdx.x;
    if (k >= rank[b]) return;
    T* col = h + (b * c + k) * (int64_t)n;
    double s = 0;
    for (int i = k + 1 + threadIdx.x; i < n; i += kPairThreads) {
        const double v = (double)col[i];
        s += v * v;
    }
    const double alpha = (double)col[k];   // read by everyone before the barriers of the sum; thread 0 overwrites it at the end
    const double sigma = block_sum(s, red);
    if (sigma == 0.0) {   // already a multiple of e_k: H_k = I
        if (threadIdx.x == 0) tau[b * c + k] = 0.0;
        return;
    }
    const double beta = -copysign(sqrt(alpha * alpha + sigma), alpha);
    const double scale = 1.0 / (alpha - beta);
    for (int i = k + 1 + threadIdx.x; i < n; i += kPairThreads) col[i] = (T)((double)col[i] * scale);
    if (threadIdx.x == 0) {
        tau[b * c + k] = (beta - alpha) / beta;
        col[k] = (T)beta;
    }
}

// y <- (I - tau v v^T) y for the columns y = first + blockIdx.x of `m` (column stride n, `mc` columns per matrix, `limit[b]` of them
// in use, counted from the rank when from_rank is set), v = Householder vector k of h
template <class T>
__global__ __launch_bounds__(kPairThreads) void house_apply_kernel(T* __restrict__ m, const T* __restrict__ h, const double* __restrict__ tau,
                                                                   const int* __restrict__ rank, int n, int c, int mc, int k, int first, int from_rank) {
    __shared__ double red[kPairThreads / 64];
    const int64_t b = blockIdx.y;
    const int r = rank[b];
    const int j = first + blockIdx.x;
    if (k >= r || j >= (from_rank ? n - r : r)) return;
    const double t = tau[b * c + k];
    if (t == 0.0) return;
    const T* v = h + (b * c + k) * (int64_t)n;
    T* y = m + (b * mc + j) * (int64_t)n;
    double s = threadIdx.x == 0 ? (double)y[k] : 0.0;
    for (int i = k + 1 + threadIdx.x; i < n; i += kPairThreads) s += (double)v[i] * (double)y[i];
    const double w = t * block_sum(s, red);
    if (threadIdx.x == 0) y[k] = (T)((double)y[k] - w);
    for (int i = k + 1 + threadIdx.x; i < n; i += kPairThreads) y[i] = (T)((double)y[i] - w * (double)v[i]);
}

// e[b][j] = unit vector e_{rank[b] + j} for j < n - rank[b]
template <class T>
__global__ __launch_bounds__(256) void complement_seed_kernel(T* __restrict__ e, const int* __restrict__ rank, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    const int j = blockIdx.y;
    const int64_t b = blockIdx.z;
    const int r = rank[b];
    if (i >= n || j >= n - r) return;
    e[(b * n + j) * (int64_t)n + i] = (i == r + j) ? T(1) : T(0);
}

// u[b][i][rank[b] + j] = e[b][j][i]
template <class T>
__global__ __launch_bounds__(256) void complement_store_kernel(T* __restrict__ u, const T* __restrict__ e, const int* __restrict__ rank, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    const int j = blockIdx.y;
    const int64_t b = blockIdx.z;
    const int r = rank[b];
    if (i >= n || j >= n - r) return;
    u[(b * n + i) * (int64_t)n + r + j] = e[(b * n + j) * (int64_t)n + i];
}

// symmetric work matrix from one triangle of the row-major a[b] (n x n), plus fro[b] = its Frobenius norm (second kernel adds it
// to the diagonal): x[i][j] = a[min,max] (upper) or a[max,min] (lower)
template <class T>
__global__ __launch_bounds__(256) void symmetrize_kernel(T* __restrict__ x, const T* __restrict__ a, int n, int lower) {
    const int j = blockIdx.x * 256 + threadIdx.x;
    const int i = blockIdx.y;
    if (j >= n) return;
    const int lo = i < j ? i : j, hi = i < j ? j : i;
    x[(int64_t)i * n + j] = lower ? a[(int64_t)hi * n + lo] : a[(int64_t)lo * n + hi];
}
// fro = sqrt(sum of the squared column norms)
__global__ __launch_bounds__(256) void frobenius_kernel(const double* __restrict__ norm, double* __restrict__ fro, int c) {
    __shared__ double red[4];
    double s = 0;
    for (int i = threadIdx.x; i < c; i += 256) s += norm[i] * norm[i];
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off, 64);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) fro[0] = sqrt(red[0] + red[1] + red[2] + red[3]);
}
template <class T>
__global__ __launch_bounds__(256) void shift_diagonal_kernel(T* __restrict__ x, const double* __restrict__ mu, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) x[(int64_t)i * n + i] = (T)((double)x[(int64_t)i * n + i] + mu[0]);
}

__global__ void clear_int_kernel(int* p) { *p = 0; }

size_t align_up(size_t b) { return (b + 255) / 256 * 256; }

// Scales every matrix of x ([batch][per_matrix]) to a largest magnitude in [0.5, 1); exps[b] receives the exponent taken out.
template <class T>
void prescale(T* x, int64_t batch, int64_t per_matrix, unsigned long long* maxbits, int* exps, hipStream_t stream) {
    const unsigned blocks = (unsigned)std::max<int64_t>(1, std::min<int64_t>(cdiv(per_matrix, 256 * 8), 1024));
    hipLaunchKernelGGL(clear_scale_kernel, dim3(cdiv(batch, 64)), dim3(64), 0, stream, maxbits, (int)batch);
    hipLaunchKernelGGL((max_abs_kernel<T>), dim3(blocks, (unsigned)batch), dim3(256), 0, stream, x, maxbits, per_matrix);
    hipLaunchKernelGGL((scale_down_kernel<T>), dim3(blocks, (unsigned)batch), dim3(256), 0, stream, x, maxbits, exps, per_matrix);
}

// Sweeps until a sweep rotates nothing.  x: [batch][c][rows], w: [batch][c][wrows] or null.
template <class T>
int32_t jacobi_run(T* x, T* w, int64_t batch, int rows, int c, int wrows, int* counter, hipStream_t stream, const char* what) {
    if (c < 2 || batch == 0 || rows == 0) return DNH_OK;
    constexpr int64_t kMaxGridZ = 65535;
    if (batch > kMaxGridZ) {
        for (int64_t b0 = 0; b0 < batch; b0 += kMaxGridZ) {
            const int64_t nbatch = std::min<int64_t>(kMaxGridZ, batch - b0);
            DNH_TRY(jacobi_run<T>(x + b0 * c * rows, w ? w + b0 * c * wrows : nullptr, nbatch, rows, c, wrows, counter, stream, what));
        }
        return DNH_OK;
    }
    const double tol = sqrt((double)rows) * (double)std::numeric_limits<T>::epsilon();   // as LAPACK's Jacobi SVD (xGESVJ)
    // Three launches per round.  Rows are cut into pieces (multiples of 32 rows, at least 128) so that the Gram and the apply
    // launches bring about four workgroups per CU.
    const int nb = (c + kBlockCols - 1) / kBlockCols, nbe = nb + (nb & 1), pairs = nbe / 2;
    int xpieces = 1, chunk = rows, wpieces = 0, wchunk = 32;
    const int64_t want = std::max<int64_t>(1, (int64_t)4 * device_cus() / ((int64_t)pairs * batch));
    xpieces = (int)std::max<int64_t>(1, std::min<int64_t>(want, rows / 128));
    chunk = (int)cdiv(cdiv(rows, xpieces), 32) * 32;
    xpieces = (int)cdiv(rows, chunk);
    if (w && wrows > 0) {
        wpieces = (int)std::max<int64_t>(1, std::min<int64_t>(want, wrows / 128));
        wchunk = (int)cdiv(cdiv(wrows, wpieces), 32) * 32;
        wpieces = (int)cdiv(wrows, wchunk);
    }
    const size_t sz_part = align_up(sizeof(double) * 768 * (size_t)xpieces * pairs * batch);
    const size_t sz_q = align_up(sizeof(double) * 1024 * (size_t)pairs * batch);
    void* block_ws = nullptr;
    DNH_TRY(dnh_alloc_async(sz_part + sz_q + sizeof(int) * (size_t)pairs * batch, stream, &block_ws));
    double* partial = (double*)block_ws;
    double* qbuf = (double*)((char*)block_ws + sz_part);
    int* flag = (int*)((char*)block_ws + sz_part + sz_q);
    struct Release {
        void* p;
        hipStream_t s;
        ~Release() { (void)dnh_free_async(p, s); }
    } release{block_ws, stream};
    for (int sweep = 0; sweep < kMaxSweeps; sweep++) {
        hipLaunchKernelGGL(clear_int_kernel, dim3(1), dim3(1), 0, stream, counter);
        for (int r = 0; r < nbe - 1; r++) {
            if constexpr (sizeof(T) == 4)
                hipLaunchKernelGGL(jacobi_block_gram_f32_kernel, dim3((unsigned)pairs, (unsigned)xpieces, (unsigned)batch), dim3(kGramThreads), 0, stream, x, partial,
                                   rows, chunk, c, nbe, r, (int64_t)c * rows);
            else
                hipLaunchKernelGGL((jacobi_block_gram_kernel<T>), dim3((unsigned)pairs, (unsigned)xpieces, (unsigned)batch), dim3(kGramThreads), 0, stream, x, partial,
                                   rows, chunk, c, nbe, r, (int64_t)c * rows);
            hipLaunchKernelGGL((jacobi_block_solve_kernel<T>), dim3((unsigned)pairs, (unsigned)batch), dim3(kSolveThreads), 0, stream, partial, xpieces, qbuf, flag, c,
                               nbe, r, (r == sweep % (nbe - 1)) ? 1 : 0, tol, counter);
            hipLaunchKernelGGL((jacobi_block_apply_kernel<T>), dim3((unsigned)pairs, (unsigned)(xpieces + wpieces), (unsigned)batch), dim3(kApplyThreads), 0, stream, x,
                               w, qbuf, flag, rows, chunk, xpieces, wrows, wchunk, c, nbe, r, (int64_t)c * rows, (int64_t)c * wrows);
        }
        DNH_LAUNCH_CHECK();
        int rotated = 0;
        DNH_HIP(hipMemcpyAsync(&rotated, counter, sizeof(int), hipMemcpyDeviceToHost, stream));
        DNH_HIP(hipStreamSynchronize(stream));
        if (rotated == 0) return DNH_OK;
    }
    return fail(DNH_ERR_NO_CONVERGENCE, "%s did not converge in %d sweeps", what, kMaxSweeps);
}


// Fills a dense row-major descriptor of `t`'s shape over `base`.
DnhTensor dense_like(const DnhTensor* t, void* base) {
    DnhTensor d = *t;
    d.base = base;
    d.offset = 0;
    int64_t acc = 1;
    for (int k = t->ndims - 1; k >= 0; k--) {
        d.stride[k] = acc;
        acc *= t->shape[k];
    }
    return d;
}

template <class T>
int32_t svd_impl(const DnhTensor* s, const DnhTensor* u, const DnhTensor* v, const DnhTensor* src, hipStream_t stream) {
    const int nd = src->ndims;
    const int64_t M64 = src->shape[nd - 2], N64 = src->shape[nd - 1];
    if (M64 > 0x7FFFFFF || N64 > 0x7FFFFFF) return fail(DNH_ERR_NOT_SUPPORTED, "dnh_batched_svd: matrix too large");
    const int M = (int)M64, N = (int)N64, K = M < N ? M : N;
    int64_t batch = 1;
    for (int d = 0; d < nd - 2; d++) batch *= src->shape[d];
    if (batch == 0 || K == 0) {
        // no singular values; the unitary matrices of an empty product are identities
        if (u && batch > 0 && M > 0) {
            const int64_t total = batch * M * M;
            void* tmp = nullptr;
            DNH_TRY(dnh_alloc_async(sizeof(T) * total, stream, &tmp));
            hipLaunchKernelGGL((identity_kernel<T>), dim3(cdiv(total, 256)), dim3(256), 0, stream, (T*)tmp, M, total);
            DnhTensor dd = dense_like(u, tmp);
            int32_t st = dnh_copy(u, &dd, stream);
            (void)dnh_free_async(tmp, stream);
            DNH_TRY(st);
        }
        if (v && batch > 0 && N > 0) {
            const int64_t total = batch * N * N;
            void* tmp = nullptr;
            DNH_TRY(dnh_alloc_async(sizeof(T) * total, stream, &tmp));
            hipLaunchKernelGGL((identity_kernel<T>), dim3(cdiv(total, 256)), dim3(256), 0, stream, (T*)tmp, N, total);
            DnhTensor dd = dense_like(v, tmp);
            int32_t st = dnh_copy(v, &dd, stream);
            (void)dnh_free_async(tmp, stream);
            DNH_TRY(st);
        }
        return DNH_OK;
    }
    // The work matrix has the K columns of the shorter side, each R = max(M, N) long: for M >= N the columns of A (W -> V, the
    // normalised columns -> U), for M < N the columns of A^T, i.e. the rows of A (W -> U, the normalised columns -> V).
    const bool tall = M >= N;
    const int R = tall ? M : N, Cn = K;
    const bool want_uv = u != nullptr;
    const size_t sz_x = align_up(sizeof(T) * (size_t)batch * Cn * R);
    const size_t sz_w = want_uv ? align_up(sizeof(T) * (size_t)batch * Cn * Cn) : 0;
    const size_t sz_big = want_uv ? align_up(sizeof(T) * (size_t)batch * R * R) : 0;      // the tall side's vectors, row-major
    const size_t sz_small = want_uv ? align_up(sizeof(T) * (size_t)batch * Cn * Cn) : 0;   // the short side's vectors, row-major
    const size_t sz_z = want_uv ? sz_big : 0;                                              // the complement's columns
    const size_t sz_h = want_uv ? sz_x : 0;                                                // Householder vectors of the completion
    const size_t sz_tau = want_uv ? align_up(sizeof(double) * (size_t)batch * Cn) : 0;
    const size_t sz_norm = align_up(sizeof(double) * (size_t)batch * R);
    const size_t sz_ord = align_up(sizeof(int) * (size_t)batch * R);
    const size_t sz_misc = align_up(sizeof(double) * (size_t)batch) + align_up(sizeof(int) * (size_t)batch) + 256 + align_up(sizeof(unsigned long long) * (size_t)batch) +
                           align_up(sizeof(int) * (size_t)batch);
    void* block = nullptr;
    DNH_TRY(dnh_alloc_async(sz_x + sz_w + sz_big + sz_small + sz_z + sz_h + sz_tau + sz_norm + sz_ord + sz_misc + align_up(sizeof(T) * (size_t)batch * K), stream,
                            &block));
    char* base = (char*)block;
    T* X = (T*)base;                       base += sz_x;
    T* W = want_uv ? (T*)base : nullptr;   base += sz_w;
    T* Big = (T*)base;                     base += sz_big;
    T* Small = (T*)base;                   base += sz_small;
    T* Z = (T*)base;                       base += sz_z;
    T* Hh = (T*)base;                      base += sz_h;
    double* tau = (double*)base;           base += sz_tau;
    double* norm = (double*)base;          base += sz_norm;
    int* order = (int*)base;               base += sz_ord;
    double* kmax = (double*)base;          base += align_up(sizeof(double) * (size_t)batch);
    int* rank = (int*)base;                base += align_up(sizeof(int) * (size_t)batch);
    int* counter = (int*)base;             base += 256;
    unsigned long long* maxbits = (unsigned long long*)base;   base += align_up(sizeof(unsigned long long) * (size_t)batch);
    int* exps = (int*)base;                base += align_up(sizeof(int) * (size_t)batch);
    T* Sv = (T*)base;

    auto body = [&]() -> int32_t {
        // X[b][j][i]: for M >= N element (i, j) of A, else element (j, i) of A: a dense view of X with A's index order
        DnhTensor xd = *src;
        xd.base = X;
        xd.offset = 0;
        {
            int64_t acc = (int64_t)Cn * R;
            for (int d = nd - 3; d >= 0; d--) { xd.stride[d] = acc; acc *= src->shape[d]; }
            if (tall) { xd.stride[nd - 2] = 1; xd.stride[nd - 1] = R; }   // A[i][j] -> X[j][i], R = M
            else      { xd.stride[nd - 2] = R; xd.stride[nd - 1] = 1; }   // A[i][j] -> X[i][j], R = N: column i of X = row i of A
        }
        DNH_TRY(dnh_copy(&xd, src, stream));
        prescale<T>(X, batch, (int64_t)Cn * R, maxbits, exps, stream);
        if (want_uv) {
            const int64_t total = batch * Cn * Cn;
            hipLaunchKernelGGL((identity_kernel<T>), dim3(cdiv(total, 256)), dim3(256), 0, stream, W, Cn, total);
        }
        DNH_TRY(jacobi_run<T>(X, W, batch, R, Cn, Cn, counter, stream, "SVD"));
        hipLaunchKernelGGL((column_norm_kernel<T>), dim3((unsigned)Cn, (unsigned)batch), dim3(kPairThreads), 0, stream, X, norm, R, Cn, (int64_t)Cn * R);
        hipLaunchKernelGGL(rank_kernel, dim3(cdiv(Cn, 256), (unsigned)batch), dim3(256), 0, stream, norm, order, Cn, 1);
        hipLaunchKernelGGL((pick_values_kernel<T>), dim3(cdiv(K, 256), (unsigned)batch), dim3(256), 0, stream, Sv, norm, order, (const double*)nullptr, 0.0,
                           exps, Cn, K);
        DNH_LAUNCH_CHECK();
        {
            DnhTensor sd = dense_like(s, Sv);
            DNH_TRY(dnh_copy(s, &sd, stream));
        }
        if (!want_uv) return DNH_OK;
        // A column of X is normalised into a vector when its norm is above 4 eps sigma_max: the sweeps end on a test relative to the
        // norms, so even short columns are orthogonal to the others to sqrt(R) eps; below that a column is rounding residue.
        const double rel = 4.0 * (double)std::numeric_limits<T>::epsilon();
        hipLaunchKernelGGL(max_key_kernel, dim3((unsigned)batch), dim3(256), 0, stream, norm, kmax, Cn);
        hipLaunchKernelGGL(numeric_rank_kernel, dim3((unsigned)batch), dim3(256), 0, stream, norm, kmax, rel, Cn, rank);
        // short side: W's columns in the order of the singular values (always complete)
        hipLaunchKernelGGL((scatter_columns_kernel<T>), dim3(cdiv(Cn, 256), (unsigned)Cn, (unsigned)batch), dim3(256), 0, stream, Small, W, order,
                           (const double*)nullptr, (const double*)nullptr, 0.0, Cn, Cn, (int64_t)Cn * Cn);
        // tall side: normalised columns of X for the singular values above the threshold ...
        hipLaunchKernelGGL((scatter_columns_kernel<T>), dim3(cdiv(R, 256), (unsigned)Cn, (unsigned)batch), dim3(256), 0, stream, Big, X, order, norm, kmax,
                           rel, R, Cn, (int64_t)Cn * R);
        DNH_LAUNCH_CHECK();
        // ... and a basis of their complement for the rest.  Needed when the matrix is not square or numerically rank deficient.
        bool need_complement = R > Cn;
        if (!need_complement) {
            std::vector<int> hr((size_t)batch);
            DNH_HIP(hipMemcpyAsync(hr.data(), rank, sizeof(int) * (size_t)batch, hipMemcpyDeviceToHost, stream));
            DNH_HIP(hipStreamSynchronize(stream));
            for (int64_t b = 0; b < batch; b++) need_complement = need_complement || hr[(size_t)b] < R;
        }
        if (need_complement) {
            // Householder QR of the orthonormal columns found so far, then Q applied to the remaining unit vectors
            hipLaunchKernelGGL((gather_u1_kernel<T>), dim3(cdiv(R, 256), (unsigned)Cn, (unsigned)batch), dim3(256), 0, stream, Hh, Big, rank, R, Cn);
            for (int k = 0; k < Cn; k++) {
                hipLaunchKernelGGL((house_vector_kernel<T>), dim3((unsigned)batch), dim3(kPairThreads), 0, stream, Hh, tau, rank, R, Cn, k);
                if (k + 1 < Cn)
                    hipLaunchKernelGGL((house_apply_kernel<T>), dim3((unsigned)(Cn - k - 1), (unsigned)batch), dim3(kPairThreads), 0, stream, Hh, Hh, tau, rank,
                                       R, Cn, Cn, k, k + 1, 0);
            }
            DNH_LAUNCH_CHECK();
            hipLaunchKernelGGL((complement_seed_kernel<T>), dim3(cdiv(R, 256), (unsigned)R, (unsigned)batch), dim3(256), 0, stream, Z, rank, R);
            for (int k = Cn - 1; k >= 0; k--)
                hipLaunchKernelGGL((house_apply_kernel<T>), dim3((unsigned)R, (unsigned)batch), dim3(kPairThreads), 0, stream, Z, Hh, tau, rank, R, Cn, R, k, 0,
                                   1);
            hipLaunchKernelGGL((complement_store_kernel<T>), dim3(cdiv(R, 256), (unsigned)R, (unsigned)batch), dim3(256), 0, stream, Big, Z, rank, R);
            DNH_LAUNCH_CHECK();
        }
        {
            DnhTensor bd = dense_like(tall ? u : v, Big);
            DNH_TRY(dnh_copy(tall ? u : v, &bd, stream));
            DnhTensor sd2 = dense_like(tall ? v : u, Small);
            DNH_TRY(dnh_copy(tall ? v : u, &sd2, stream));
        }
        return DNH_OK;
    };
    const int32_t st = body();
    (void)dnh_free_async(block, stream);
    return st;
}

template <class T>
int32_t eig_impl(int32_t part, const DnhTensor* vals, const DnhTensor* vecs, const DnhTensor* src, hipStream_t stream) {
    if (src->shape[0] > 0x7FFFFFF) return fail(DNH_ERR_NOT_SUPPORTED, "dnh_symmetric_eig: matrix too large");
    const int n = (int)src->shape[0];
    if (n == 0) return DNH_OK;
    const size_t sz_m = align_up(sizeof(T) * (size_t)n * n);
    const size_t sz_norm = align_up(sizeof(double) * (size_t)n);
    const size_t sz_ord = align_up(sizeof(int) * (size_t)n);
    void* block = nullptr;
    DNH_TRY(dnh_alloc_async(4 * sz_m + sz_norm + sz_ord + 1024 + align_up(sizeof(T) * (size_t)n), stream, &block));
    char* base = (char*)block;
    T* A = (T*)base;               base += sz_m;   // dense copy of src
    T* X = (T*)base;               base += sz_m;   // mirrored triangle + mu I (symmetric: its rows are its columns)
    T* W = (T*)base;               base += sz_m;
    T* Out = (T*)base;             base += sz_m;
    double* norm = (double*)base;  base += sz_norm;
    int* order = (int*)base;       base += sz_ord;
    double* mu = (double*)base;    base += 256;
    int* counter = (int*)base;     base += 256;
    unsigned long long* maxbits = (unsigned long long*)base;   base += 256;
    int* exps = (int*)base;        base += 256;
    T* Vals = (T*)base;
    auto body = [&]() -> int32_t {
        DnhTensor ad = dense_like(src, A);
        DNH_TRY(dnh_copy(&ad, src, stream));
        hipLaunchKernelGGL((symmetrize_kernel<T>), dim3(cdiv(n, 256), (unsigned)n), dim3(256), 0, stream, X, A, n, part == 1 ? 1 : 0);
        prescale<T>(X, 1, (int64_t)n * n, maxbits, exps, stream);
        hipLaunchKernelGGL((column_norm_kernel<T>), dim3((unsigned)n, 1), dim3(kPairThreads), 0, stream, X, norm, n, n, (int64_t)n * n);
        hipLaunchKernelGGL(frobenius_kernel, dim3(1), dim3(256), 0, stream, norm, mu, n);
        hipLaunchKernelGGL((shift_diagonal_kernel<T>), dim3(cdiv(n, 256)), dim3(256), 0, stream, X, mu, n);
        hipLaunchKernelGGL((identity_kernel<T>), dim3(cdiv((int64_t)n * n, 256)), dim3(256), 0, stream, W, n, (int64_t)n * n);
        DNH_LAUNCH_CHECK();
        DNH_TRY(jacobi_run<T>(X, W, 1, n, n, n, counter, stream, "symmetric eigendecomposition"));
        // the column norms are lambda + mu >= 0; ascending eigenvalues, eigenvector k = column order[k] of W
        hipLaunchKernelGGL((column_norm_kernel<T>), dim3((unsigned)n, 1), dim3(kPairThreads), 0, stream, X, norm, n, n, (int64_t)n * n);
        hipLaunchKernelGGL(rank_kernel, dim3(cdiv(n, 256), 1), dim3(256), 0, stream, norm, order, n, 0);
        hipLaunchKernelGGL((pick_values_kernel<T>), dim3(cdiv(n, 256), 1), dim3(256), 0, stream, Vals, norm, order, (const double*)mu, -1.0, exps, n, n);
        hipLaunchKernelGGL((scatter_columns_kernel<T>), dim3(cdiv(n, 256), (unsigned)n, 1), dim3(256), 0, stream, Out, W, order, (const double*)nullptr,
                           (const double*)nullptr, 0.0, n, n, (int64_t)n * n);
        DNH_LAUNCH_CHECK();
        DnhTensor vd = dense_like(vals, Vals);
        DNH_TRY(dnh_copy(vals, &vd, stream));
        DnhTensor od = dense_like(vecs, Out);
        DNH_TRY(dnh_copy(vecs, &od, stream));
        return DNH_OK;
    };
    const int32_t st = body();
    (void)dnh_free_async(block, stream);
    return st;
}

}  // namespace

extern "C" int32_t dnh_batched_svd(const DnhTensor* s, const DnhTensor* u, const DnhTensor* v, const DnhTensor* src, void* stream) {
    DNH_TRY(ensure_init());
    DNH_TRY(check_tensor(s, "dnh_batched_svd"));
    DNH_TRY(check_tensor(src, "dnh_batched_svd"));
    if ((u == nullptr) != (v == nullptr)) return fail(DNH_ERR_INVALID_ARG, "dnh_batched_svd: u and v must be given together");
    if (u) {
        DNH_TRY(check_tensor(u, "dnh_batched_svd"));
        DNH_TRY(check_tensor(v, "dnh_batched_svd"));
    }
    if (!dtype_is_fp(src->dtype))
        return fail(DNH_ERR_NOT_SUPPORTED, "dnh_batched_svd: this operation is only supported for floating point numbers");
    if (s->dtype != src->dtype || (u && (u->dtype != src->dtype || v->dtype != src->dtype))) return fail(DNH_ERR_INVALID_ARG, "dnh_batched_svd: dtypes differ");
    const int nd = src->ndims;
    if (nd < 2) return fail(DNH_ERR_INVALID_ARG, "dnh_batched_svd: need at least a matrix");
    const int64_t M = src->shape[nd - 2], N = src->shape[nd - 1], K = M < N ? M : N;
    bool ok = s->ndims == nd - 1 && s->shape[nd - 2] == K;
    for (int d = 0; d < nd - 2 && ok; d++) ok = s->shape[d] == src->shape[d];
    if (!ok) return fail(DNH_ERR_INVALID_ARG, "dnh_batched_svd: the singular values need shape [batch...; min(M, N)]");
    if (u) {
        ok = u->ndims == nd && v->ndims == nd && u->shape[nd - 2] == M && u->shape[nd - 1] == M && v->shape[nd - 2] == N && v->shape[nd - 1] == N;
        for (int d = 0; d < nd - 2 && ok; d++) ok = u->shape[d] == src->shape[d] && v->shape[d] == src->shape[d];
        if (!ok) return fail(DNH_ERR_INVALID_ARG, "dnh_batched_svd: the unitary matrices need shapes [batch...; M; M] and [batch...; N; N]");
    }
    if (src->dtype == DNH_F32) return svd_impl<float>(s, u, v, src, (hipStream_t)stream);
    return svd_impl<double>(s, u, v, src, (hipStream_t)stream);
}

extern "C" int32_t dnh_symmetric_eig(int32_t part, const DnhTensor* eigvals, const DnhTensor* eigvecs, const DnhTensor* src, void* stream) {
    DNH_TRY(ensure_init());
    DNH_TRY(check_tensor(eigvals, "dnh_symmetric_eig"));
    DNH_TRY(check_tensor(eigvecs, "dnh_symmetric_eig"));
    DNH_TRY(check_tensor(src, "dnh_symmetric_eig"));
    if (part != 0 && part != 1) return fail(DNH_ERR_INVALID_ARG, "dnh_symmetric_eig: part must be 0 (upper) or 1 (lower)");
    if (!dtype_is_fp(src->dtype))
        return fail(DNH_ERR_NOT_SUPPORTED, "dnh_symmetric_eig: this operation is only supported for floating point numbers");
    if (eigvals->dtype != src->dtype || eigvecs->dtype != src->dtype) return fail(DNH_ERR_INVALID_ARG, "dnh_symmetric_eig: dtypes differ");
    if (src->ndims != 2 || src->shape[0] != src->shape[1]) return fail(DNH_ERR_INVALID_ARG, "dnh_symmetric_eig: need a square matrix");
    if (!same_shape(eigvecs, src)) return fail(DNH_ERR_INVALID_ARG, "dnh_symmetric_eig: eigenvectors and source must have the same shape");
    if (eigvals->ndims != 1 || eigvals->shape[0] != src->shape[0]) return fail(DNH_ERR_INVALID_ARG, "dnh_symmetric_eig: eigenvalues must be a vector of length n");
    if (src->dtype == DNH_F32) return eig_impl<float>(part, eigvals, eigvecs, src, (hipStream_t)stream);
    return eig_impl<double>(part, eigvals, eigvecs, src, (hipStream_t)stream);
}
