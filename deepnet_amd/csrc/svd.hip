// dnh_batched_svd, dnh_symmetric_eig: ITensorBackend BatchedSVD and SymmetricEigenDecomposition (Tensor/Tensor/TensorBackend.fs:143,
// 145).  The reference's host backend calls LAPACK gesdd / syevd (Tensor/Tensor/Host/HostBackend.fs:579-628); its CUDA backend
// does not implement either (Tensor/Tensor/Cuda/CudaBackend.fs:486-492).
//
// Both run on one-sided Jacobi (Hestenes) rotations, which need nothing but column pairs: for the columns x_p, x_q of a work
// matrix X (R rows, C <= R columns, every column contiguous) a plane rotation makes them orthogonal, and the same rotation is
// applied to the columns of W, which starts as the identity.  The C / 2 pairs of a round of the round-robin schedule are
// disjoint, so a round is one launch with one workgroup per pair and matrix; C - 1 rounds visit every pair once (a sweep).
// When a sweep rotates nothing, X = A W has orthogonal columns: their norms are the singular values, the normalised
// columns the left vectors, W the right vectors.  Relative accuracy is that of the rotations (no squaring of the condition
// number as with the eigenvalues of A^T A).
//
//   SVD of A (M x N):  the side with fewer vectors plays W (it comes out complete); the taller side's vectors are the
//     normalised columns of X for the singular values above max(M, N) * eps * sigma_max, and an orthonormal basis of their
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

// Sums of three values over a wavefront, left in lane 63, through DPP lane moves (see wave_argmax.h): row shifts by 1, 2, 4, 8
// add up each row of 16 lanes into its lane 15 (a lane without a source adds zero), two row broadcasts carry the row sums on.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp_fetch_or_zero(double v) {
    const long long b = __double_as_longlong(v);
    const int lo = __builtin_amdgcn_update_dpp(0, (int)(unsigned)(b & 0xFFFFFFFFLL), CTRL, ROW_MASK, 0xF, false);
    const int hi = __builtin_amdgcn_update_dpp(0, (int)(b >> 32), CTRL, ROW_MASK, 0xF, false);
    return __longlong_as_double(((long long)hi << 32) | (unsigned)lo);
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ void sum3_step(double& a, double& b, double& c) {
    a += dpp_fetch_or_zero<CTRL, ROW_MASK>(a);
    b += dpp_fetch_or_zero<CTRL, ROW_MASK>(b);
    c += dpp_fetch_or_zero<CTRL, ROW_MASK>(c);
}
__device__ __forceinline__ void wave_sum3_to_lane63(double& a, double& b, double& c) {
    sum3_step<0x111, 0xF>(a, b, c);   // row_shr:1
    sum3_step<0x112, 0xF>(a, b, c);   // row_shr:2: lane i now holds the sum of lanes i-3 .. i of its row
    sum3_step<0x114, 0xF>(a, b, c);   // row_shr:4
    sum3_step<0x118, 0xF>(a, b, c);   // row_shr:8: lane 15 of a row holds the row's sum
    sum3_step<0x142, 0xA>(a, b, c);   // row_bcast:15 into rows 1 and 3
    sum3_step<0x143, 0xC>(a, b, c);   // row_bcast:31 into rows 2 and 3: lane 63 holds the wavefront's sum
}

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

// One round: workgroup (k, matrix) orthogonalises columns p, q of X and applies the rotation to the same columns of W.
// X is [batch][c][r] (column j of a matrix = r contiguous values), W is [batch][c][cw_rows] or null.
template <class T>
__global__ __launch_bounds__(kPairThreads) void jacobi_round_kernel(T* __restrict__ x, T* __restrict__ w, int rows, int c, int ce, int round,
                                                                    int wrows, int64_t bsx, int64_t bsw, double tol, int* rotations) {
    __shared__ double red3[3][kPairThreads / 64];
    int a, b;
    pair_of(ce, round, blockIdx.x, &a, &b);
    if (a >= c || b >= c) return;
    const int p = a < b ? a : b, q = a < b ? b : a;
    T* xp = x + (int64_t)blockIdx.y * bsx + (int64_t)p * rows;
    T* xq = x + (int64_t)blockIdx.y * bsx + (int64_t)q * rows;
    double sa = 0, sb = 0, sg = 0;
    for (int i = threadIdx.x; i < rows; i += kPairThreads) {
        const double u = (double)xp[i], v = (double)xq[i];
        sa += u * u;
        sb += v * v;
        sg += u * v;
    }
    // the three sums share one pair of barriers
    wave_sum3_to_lane63(sa, sb, sg);
    if ((threadIdx.x & 63) == 63) {
        red3[0][threadIdx.x >> 6] = sa;
        red3[1][threadIdx.x >> 6] = sb;
        red3[2][threadIdx.x >> 6] = sg;
    }
    __syncthreads();
    double alpha = 0, beta = 0, gamma = 0;
#pragma unroll
    for (int i = 0; i < kPairThreads / 64; i++) {
        alpha += red3[0][i];
        beta += red3[1][i];
        gamma += red3[2][i];
    }
    if (gamma == 0.0 || fabs(gamma) <= tol * sqrt(alpha * beta)) return;   // uniform: every thread holds the same sums
    const double zeta = (beta - alpha) / (2.0 * gamma);
    const double t = (zeta >= 0.0 ? 1.0 : -1.0) / (fabs(zeta) + sqrt(1.0 + zeta * zeta));
    const double cs = 1.0 / sqrt(1.0 + t * t), sn = cs * t;
    for (int i = threadIdx.x; i < rows; i += kPairThreads) {
        const double u = (double)xp[i], v = (double)xq[i];
        xp[i] = (T)(cs * u - sn * v);
        xq[i] = (T)(sn * u + cs * v);
    }
    if (w) {
        T* wp = w + (int64_t)blockIdx.y * bsw + (int64_t)p * wrows;
        T* wq = w + (int64_t)blockIdx.y * bsw + (int64_t)q * wrows;
        for (int i = threadIdx.x; i < wrows; i += kPairThreads) {
            const double u = (double)wp[i], v = (double)wq[i];
            wp[i] = (T)(cs * u - sn * v);
            wq[i] = (T)(sn * u + cs * v);
        }
    }
    if (threadIdx.x == 0) *rotations = 1;   // a flag, not a count: every writer stores the same value, no atomic queue at one address
}

// The same round for columns of at most NPT * 256 elements: a thread keeps its elements of both column pairs (X and W) in
// registers, so every global load of the round is issued before the reduction and the rotation only computes and stores (the
// two-pass form above waits for a second round trip after the barrier; a round is latency-bound, not bandwidth-bound).
template <class T, int NPT>
__global__ __launch_bounds__(kPairThreads) void jacobi_round_reg_kernel(T* __restrict__ x, T* __restrict__ w, int rows, int c, int ce, int round,
                                                                        int wrows, int64_t bsx, int64_t bsw, double tol, int* rotations) {
    __shared__ double red3[3][kPairThreads / 64];
    int a, b;
    pair_of(ce, round, blockIdx.x, &a, &b);
    if (a >= c || b >= c) return;
    const int p = a < b ? a : b, q = a < b ? b : a;
    T* xp = x + (int64_t)blockIdx.y * bsx + (int64_t)p * rows;
    T* xq = x + (int64_t)blockIdx.y * bsx + (int64_t)q * rows;
    T* wp = w ? w + (int64_t)blockIdx.y * bsw + (int64_t)p * wrows : nullptr;
    T* wq = w ? w + (int64_t)blockIdx.y * bsw + (int64_t)q * wrows : nullptr;
    T u[NPT], v[NPT], wu[NPT], wv[NPT];
#pragma unroll
    for (int k = 0; k < NPT; k++) {
        const int i = threadIdx.x + k * kPairThreads;
        u[k] = i < rows ? xp[i] : T(0);
        v[k] = i < rows ? xq[i] : T(0);
    }
    if (w) {
#pragma unroll
        for (int k = 0; k < NPT; k++) {
            const int i = threadIdx.x + k * kPairThreads;
            wu[k] = i < wrows ? wp[i] : T(0);
            wv[k] = i < wrows ? wq[i] : T(0);
        }
    }
    double sa = 0, sb = 0, sg = 0;
#pragma unroll
    for (int k = 0; k < NPT; k++) {
        const double du = (double)u[k], dv = (double)v[k];
        sa += du * du;
        sb += dv * dv;
        sg += du * dv;
    }
    wave_sum3_to_lane63(sa, sb, sg);
    if ((threadIdx.x & 63) == 63) {
        red3[0][threadIdx.x >> 6] = sa;
        red3[1][threadIdx.x >> 6] = sb;
        red3[2][threadIdx.x >> 6] = sg;
    }
    __syncthreads();
    double alpha = 0, beta = 0, gamma = 0;
#pragma unroll
    for (int i = 0; i < kPairThreads / 64; i++) {
        alpha += red3[0][i];
        beta += red3[1][i];
        gamma += red3[2][i];
    }
    if (gamma == 0.0 || fabs(gamma) <= tol * sqrt(alpha * beta)) return;
    const double zeta = (beta - alpha) / (2.0 * gamma);
    const double t = (zeta >= 0.0 ? 1.0 : -1.0) / (fabs(zeta) + sqrt(1.0 + zeta * zeta));
    const double cs = 1.0 / sqrt(1.0 + t * t), sn = cs * t;
#pragma unroll
    for (int k = 0; k < NPT; k++) {
        const int i = threadIdx.x + k * kPairThreads;
        if (i < rows) {
            const double du = (double)u[k], dv = (double)v[k];
            xp[i] = (T)(cs * du - sn * dv);
            xq[i] = (T)(sn * du + cs * dv);
        }
    }
    if (w) {
#pragma unroll
        for (int k = 0; k < NPT; k++) {
            const int i = threadIdx.x + k * kPairThreads;
            if (i < wrows) {
                const double du = (double)wu[k], dv = (double)wv[k];
                wp[i] = (T)(cs * du - sn * dv);
                wq[i] = (T)(sn * du + cs * dv);
            }
        }
    }
    if (threadIdx.x == 0) *rotations = 1;   // a flag, not a count: every writer stores the same value, no atomic queue at one address
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

// out[b][k] = (T)(key[b][order[b][k]] + shift[b] * sign) for k < count
template <class T>
__global__ __launch_bounds__(256) void pick_values_kernel(T* __restrict__ out, const double* __restrict__ key, const int* __restrict__ order,
                                                          const double* __restrict__ shift, double sign, int c, int count) {
    const int k = blockIdx.x * 256 + threadIdx.x;
    if (k >= count) return;
    const int64_t b = blockIdx.y;
    const double v = key[b * c + order[b * c + k]] + (shift ? sign * shift[b] : 0.0);
    out[b * count + k] = (T)v;
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

// Sweeps until a sweep rotates nothing.  x: [batch][c][rows], w: [batch][c][wrows] or null.
template <class T>
int32_t jacobi_run(T* x, T* w, int64_t batch, int rows, int c, int wrows, int* counter, hipStream_t stream, const char* what) {
    if (c < 2 || batch == 0 || rows == 0) return DNH_OK;
    const int ce = c + (c & 1);
    const double tol = sqrt((double)rows) * (double)std::numeric_limits<T>::epsilon();   // as LAPACK's Jacobi SVD (xGESVJ)
    for (int sweep = 0; sweep < kMaxSweeps; sweep++) {
        hipLaunchKernelGGL(clear_int_kernel, dim3(1), dim3(1), 0, stream, counter);
        const int longest = rows > wrows ? rows : wrows;
        const dim3 grid((unsigned)(ce / 2), (unsigned)batch);
#define DNH_ROUND(KERNEL) hipLaunchKernelGGL((KERNEL), grid, dim3(kPairThreads), 0, stream, x, w, rows, c, ce, r, wrows, (int64_t)c * rows, (int64_t)c * wrows, tol, counter)
        for (int r = 0; r < ce - 1; r++) {
            if (longest <= 1 * kPairThreads) DNH_ROUND((jacobi_round_reg_kernel<T, 1>));
            else if (longest <= 4 * kPairThreads) DNH_ROUND((jacobi_round_reg_kernel<T, 4>));
            else if (longest <= 8 * kPairThreads) DNH_ROUND((jacobi_round_reg_kernel<T, 8>));
            else if (sizeof(T) == 8 && longest <= 16 * kPairThreads) DNH_ROUND((jacobi_round_reg_kernel<T, 16>));   // single precision: the two-pass form measured faster at 4000 rows
            else DNH_ROUND((jacobi_round_kernel<T>));
        }
#undef DNH_ROUND
        DNH_LAUNCH_CHECK();
        int rotated = 0;
        DNH_HIP(hipMemcpyAsync(&rotated, counter, sizeof(int), hipMemcpyDeviceToHost, stream));
        DNH_HIP(hipStreamSynchronize(stream));
        if (rotated == 0) return DNH_OK;
    }
    return fail(DNH_ERR_NO_CONVERGENCE, "%s did not converge in %d sweeps", what, kMaxSweeps);
}

size_t align_up(size_t b) { return (b + 255) / 256 * 256; }

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
    const size_t sz_misc = align_up(sizeof(double) * (size_t)batch) + align_up(sizeof(int) * (size_t)batch) + 256;
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
        if (want_uv) {
            const int64_t total = batch * Cn * Cn;
            hipLaunchKernelGGL((identity_kernel<T>), dim3(cdiv(total, 256)), dim3(256), 0, stream, W, Cn, total);
        }
        DNH_TRY(jacobi_run<T>(X, W, batch, R, Cn, Cn, counter, stream, "SVD"));
        hipLaunchKernelGGL((column_norm_kernel<T>), dim3((unsigned)Cn, (unsigned)batch), dim3(kPairThreads), 0, stream, X, norm, R, Cn, (int64_t)Cn * R);
        hipLaunchKernelGGL(rank_kernel, dim3(cdiv(Cn, 256), (unsigned)batch), dim3(256), 0, stream, norm, order, Cn, 1);
        hipLaunchKernelGGL((pick_values_kernel<T>), dim3(cdiv(K, 256), (unsigned)batch), dim3(256), 0, stream, Sv, norm, order, (const double*)nullptr, 0.0,
                           Cn, K);
        DNH_LAUNCH_CHECK();
        {
            DnhTensor sd = dense_like(s, Sv);
            DNH_TRY(dnh_copy(s, &sd, stream));
        }
        if (!want_uv) return DNH_OK;
        const double rel = (double)R * (double)std::numeric_limits<T>::epsilon();
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
    DNH_TRY(dnh_alloc_async(4 * sz_m + sz_norm + sz_ord + 512 + align_up(sizeof(T) * (size_t)n), stream, &block));
    char* base = (char*)block;
    T* A = (T*)base;               base += sz_m;   // dense copy of src
    T* X = (T*)base;               base += sz_m;   // mirrored triangle + mu I (symmetric: its rows are its columns)
    T* W = (T*)base;               base += sz_m;
    T* Out = (T*)base;             base += sz_m;
    double* norm = (double*)base;  base += sz_norm;
    int* order = (int*)base;       base += sz_ord;
    double* mu = (double*)base;    base += 256;
    int* counter = (int*)base;     base += 256;
    T* Vals = (T*)base;
    auto body = [&]() -> int32_t {
        DnhTensor ad = dense_like(src, A);
        DNH_TRY(dnh_copy(&ad, src, stream));
        hipLaunchKernelGGL((symmetrize_kernel<T>), dim3(cdiv(n, 256), (unsigned)n), dim3(256), 0, stream, X, A, n, part == 1 ? 1 : 0);
        hipLaunchKernelGGL((column_norm_kernel<T>), dim3((unsigned)n, 1), dim3(kPairThreads), 0, stream, X, norm, n, n, (int64_t)n * n);
        hipLaunchKernelGGL(frobenius_kernel, dim3(1), dim3(256), 0, stream, norm, mu, n);
        hipLaunchKernelGGL((shift_diagonal_kernel<T>), dim3(cdiv(n, 256)), dim3(256), 0, stream, X, mu, n);
        hipLaunchKernelGGL((identity_kernel<T>), dim3(cdiv((int64_t)n * n, 256)), dim3(256), 0, stream, W, n, (int64_t)n * n);
        DNH_LAUNCH_CHECK();
        DNH_TRY(jacobi_run<T>(X, W, 1, n, n, n, counter, stream, "symmetric eigendecomposition"));
        // the column norms are lambda + mu >= 0; ascending eigenvalues, eigenvector k = column order[k] of W
        hipLaunchKernelGGL((column_norm_kernel<T>), dim3((unsigned)n, 1), dim3(kPairThreads), 0, stream, X, norm, n, n, (int64_t)n * n);
        hipLaunchKernelGGL(rank_kernel, dim3(cdiv(n, 256), 1), dim3(256), 0, stream, norm, order, n, 0);
        hipLaunchKernelGGL((pick_values_kernel<T>), dim3(cdiv(n, 256), 1), dim3(256), 0, stream, Vals, norm, order, (const double*)mu, -1.0, n, n);
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
