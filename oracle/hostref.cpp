// hostref — CPU restatement of the reference HostTensor backend (TEST INFRASTRUCTURE, not product code).
//
// This file is the parity oracle and the timed CPU baseline for the HIP tensor backend.  Only tests, the
// smoke check and the benchmark's cpu_baseline leg may load it; the product library never does.
//
// It restates, operation by operation, what the reference computes on its Host device:
//   loop nests and threading shape ..... Tensor/Tensor/Host/ScalarOps.fs:15-361 (Apply*Op, ApplyAxisFold;
//                                        Parallel.For over dimension 0 only, and only when rank > 1)
//   element semantics .................. Tensor/Tensor/Host/ScalarOps.fs:363-707, Tensor/Tensor/ScalarPrimitives.fs:50-246,
//                                        Tensor/Tensor/Sgn.fs:11-15, Tensor/Tensor/Utils.fs:226-299 (zero/one/min/max values)
//   address math and index checks ...... Tensor/Tensor/Host/FastAccess.fs:41-61, 67-123
//   which ops run single-threaded ...... Tensor/Tensor/Host/VectorOps.fs:254-301 (SIMD list), Host/HostBackend.fs:187-389
//   dot ................................ Tensor/Tensor/Host/HostBackend.fs:463-546 (BLAS for fp32/fp64, multiply+sum otherwise)
//   batched inversion .................. Tensor/Tensor/Host/HostBackend.fs:548-576 (LAPACK getrf + getri per matrix),
//                                        matrix hand-over Tensor/Tensor/BlasSupport.fs:148-190
//   special values ..................... Tensor/Tensor/TensorRng.fs:24 (NotFound)
//
// Pinning (what each function is checked against, see tests/test_oracle_*.py):
//   element ops, compare, logic, ifThenElse, copy, convert: the reference's doc/docstring vectors in tests/golden/
//     plus NumPy, which is bit-identical for IEEE-exact ops; transcendentals: double libm rounded to T, special values by closed form;
//   sequential folds: np.add.accumulate / np.multiply.accumulate (sequential, in T); max/min/all/any/countTrue: NumPy reductions;
//   argMax/argMin: np.argmax/argmin (first occurrence) + planted ties + NotFound rows by hand; find: brute force;
//   gather/scatter/maskedGet/maskedSet/trueIndices: NumPy fancy indexing, np.add.at, boolean masks, np.argwhere + doc vectors;
//   dot: fp64 matmul as truth within the stated K-term bound, doc vector, structural identities.
//   batched inversion: the reference's own fixture (Tensor.Test/TestData/MatInv.h5, BaseTests.fs:214-233: inv(Kk).Kk = I to 1e-5),
//     its doc example and singular-matrix test, closed forms (Hilbert, diagonal, permutation, 2x2) and A.inv(A) = I.
//   PARITY UNPINNED at bit level (tolerance-level only): fp32 transcendental last bits (FSharp.Core + libm, not in the
//   reference tree); the summation order inside MKL sgemm/sdot and the blocking inside MKL getrf/getri (binary not in the
//   reference tree: the published unblocked LAPACK algorithms getf2 / trti2 / getri are restated).
//
// Build: g++ -O2 -fopenmp -ffp-contract=off (no fast-math) — every + and * rounds separately, as in the reference.

#include <cmath>
#include <cstdint>
#include <cstring>
#include <cstdlib>
#include <limits>
#include <type_traits>
#include <vector>
#include <omp.h>

#include "../include/tensor_hip.h"

namespace {

constexpr int64_t kNotFound = DNH_NOT_FOUND;
int g_threads = 0;  // 0 = all cores

inline int nthreads() { return g_threads > 0 ? g_threads : omp_get_num_procs(); }

struct Lay {
    int nd;
    int64_t shape[DNH_MAX_DIMS];
    int64_t stride[DNH_MAX_DIMS];
    int64_t offset;
};

inline Lay lay_of(const DnhTensor* t) {
    Lay l;
    l.nd = t->ndims;
    l.offset = t->offset;
    for (int d = 0; d < DNH_MAX_DIMS; d++) {
        l.shape[d] = d < t->ndims ? t->shape[d] : 1;
        l.stride[d] = d < t->ndims ? t->stride[d] : 0;
    }
    return l;
}

inline bool valid(const DnhTensor* t) { return t && t->ndims >= 0 && t->ndims <= DNH_MAX_DIMS; }

inline bool same_shape(const DnhTensor* a, const DnhTensor* b) {
    if (a->ndims != b->ndims) return false;
    for (int d = 0; d < a->ndims; d++)
        if (a->shape[d] != b->shape[d]) return false;
    return true;
}

inline int64_t nelems(const DnhTensor* t) {
    int64_t n = 1;
    for (int d = 0; d < t->ndims; d++) n *= t->shape[d];
    return n;
}

// Row iteration shared by every element-wise op and fold (ScalarOps.fs:15-230, 299-361): dimensions 0..nd-2 are walked in
// row-major order, `row(addr[K], pos)` handles the whole last dimension.  `nd`/`shape` describe the iteration space;
// operand k contributes stride[k][0..nd-2] and offset[k].  With threads the loop over dimension 0 is split (Parallel.For).
template <int K, class Row>
void for_rows(int nd, const int64_t* shape, const Lay* const (&ops)[K], bool threads, Row row) {
    for (int d = 0; d < nd; d++)
        if (shape[d] == 0) return;
    if (nd <= 1) {
        int64_t addr[K], pos[DNH_MAX_DIMS] = {0};
        for (int k = 0; k < K; k++) addr[k] = ops[k]->offset;
        row(addr, pos);
        return;
    }
    auto walk = [&](int64_t p0) {
        int64_t pos[DNH_MAX_DIMS] = {0};
        int64_t addr[K];
        pos[0] = p0;
        for (int k = 0; k < K; k++) addr[k] = ops[k]->offset + p0 * ops[k]->stride[0];
        // odometer over dims 1..nd-2
        for (;;) {
            row(addr, pos);
            int d = nd - 2;
            for (; d >= 1; d--) {
                if (pos[d] == shape[d] - 1) {
                    for (int k = 0; k < K; k++) addr[k] -= pos[d] * ops[k]->stride[d];
                    pos[d] = 0;
                } else {
                    for (int k = 0; k < K; k++) addr[k] += ops[k]->stride[d];
                    pos[d]++;
                    break;
                }
            }
            if (d < 1) break;
        }
    };
    if (threads && nthreads() > 1) {
#pragma omp parallel for schedule(static) num_threads(nthreads())
        for (int64_t p0 = 0; p0 < shape[0]; p0++) walk(p0);
    } else {
        for (int64_t p0 = 0; p0 < shape[0]; p0++) walk(p0);
    }
}

// HostBackend.ElemwiseLayouts (HostBackend.fs:139-153): move the largest dimension in which the target has stride 1 and
// every source stride 0 or 1 to the last position.  Results do not depend on it; the loop order (and so the timing) does.
template <int K>
void elemwise_layouts(Lay (&l)[K]) {
    int nd = l[0].nd, best = -1;
    int64_t bestSize = -1;
    for (int d = 0; d < nd; d++) {
        bool good = l[0].stride[d] == 1;
        for (int k = 1; k < K; k++) good = good && (l[k].stride[d] == 1 || l[k].stride[d] == 0);
        if (good && l[0].shape[d] > bestSize) { best = d; bestSize = l[0].shape[d]; }
    }
    if (best >= 0 && best != nd - 1)
        for (int k = 0; k < K; k++) {
            std::swap(l[k].shape[best], l[k].shape[nd - 1]);
            std::swap(l[k].stride[best], l[k].stride[nd - 1]);
        }
}

// VectorOps.CanUse (VectorOps.fs:287-301): SIMD (hence single-threaded) loops apply when the last target stride is 1 and
// every last source stride is 0 or 1.
template <int K>
bool vector_ops_can_use(const Lay (&l)[K]) {
    int nd = l[0].nd;
    if (nd == 0) return false;
    if (l[0].stride[nd - 1] != 1) return false;
    for (int k = 1; k < K; k++)
        if (l[k].stride[nd - 1] != 1 && l[k].stride[nd - 1] != 0) return false;
    return true;
}

// ---- scalar semantics -------------------------------------------------------------------------------------------------

template <class T> constexpr bool is_fp = std::is_floating_point<T>::value;

// fp32 transcendental = double libm result rounded to fp32 (F# Operators.<fn> on float32); fp64 = libm.
#define HREF_FP_FN(NAME, EXPR)                                       \
    template <class T> inline T NAME(T x) {                          \
        double v = (double)x;                                        \
        (void)v;                                                     \
        return (T)(EXPR);                                            \
    }
HREF_FP_FN(f_log, std::log(v))
HREF_FP_FN(f_log10, std::log10(v))
HREF_FP_FN(f_exp, std::exp(v))
HREF_FP_FN(f_sin, std::sin(v))
HREF_FP_FN(f_cos, std::cos(v))
HREF_FP_FN(f_tan, std::tan(v))
HREF_FP_FN(f_asin, std::asin(v))
HREF_FP_FN(f_acos, std::acos(v))
HREF_FP_FN(f_atan, std::atan(v))
HREF_FP_FN(f_sinh, std::sinh(v))
HREF_FP_FN(f_cosh, std::cosh(v))
HREF_FP_FN(f_tanh, std::tanh(v))
HREF_FP_FN(f_sqrt, std::sqrt(v))
HREF_FP_FN(f_ceil, std::ceil(v))
HREF_FP_FN(f_floor, std::floor(v))
HREF_FP_FN(f_round, std::nearbyint(v))  // Math.Round: ties to even
HREF_FP_FN(f_trunc, std::trunc(v))

template <class T> inline T sgn_of(T x) { return x < T(0) ? T(-1) : (x > T(0) ? T(1) : T(0)); }  // Sgn.fs:11-15

template <class T> inline T wrap_neg(T x) {
    if constexpr (is_fp<T>) return -x;
    else { using U = typename std::make_unsigned<T>::type; return (T)(U(0) - (U)x); }
}
template <class T> inline T wrap_abs(T x) {
    if constexpr (is_fp<T>) return std::fabs(x);
    else return x < 0 ? wrap_neg(x) : x;
}
template <class T> inline T wrap_add(T a, T b) {
    if constexpr (is_fp<T>) return a + b;
    else { using U = typename std::make_unsigned<T>::type; return (T)((U)a + (U)b); }
}
template <class T> inline T wrap_sub(T a, T b) {
    if constexpr (is_fp<T>) return a - b;
    else { using U = typename std::make_unsigned<T>::type; return (T)((U)a - (U)b); }
}
template <class T> inline T wrap_mul(T a, T b) {
    if constexpr (is_fp<T>) return a * b;
    else if constexpr (sizeof(T) < 4) return (T)((unsigned)a * (unsigned)b);
    else { using U = typename std::make_unsigned<T>::type; return (T)((U)a * (U)b); }
}
// Integer division/modulo truncate toward zero.  .NET raises on x/0 and MinValue/-1; the GPU cannot, so these inputs
// are "unspecified, must not fault" — the oracle returns 0 for them and tests keep them out.
template <class T> inline T safe_div(T a, T b) {
    if constexpr (is_fp<T>) return a / b;
    else {
        if (b == 0) return 0;
        if constexpr (std::is_signed<T>::value && sizeof(T) >= 4)   // narrower operands divide as int32 and wrap when stored (IL div, conv.i2)
            if (a == std::numeric_limits<T>::min() && b == T(-1)) return 0;
        return (T)(a / b);
    }
}
template <class T> inline T safe_mod(T a, T b) {
    if constexpr (is_fp<T>) return (T)std::fmod(a, b);
    else {
        if (b == 0) return 0;
        if constexpr (std::is_signed<T>::value && sizeof(T) >= 4)   // narrower operands divide as int32 and wrap when stored (IL div, conv.i2)
            if (a == std::numeric_limits<T>::min() && b == T(-1)) return 0;
        return (T)(a % b);
    }
}
template <class T> inline T f_pow(T a, T b) { return (T)std::pow((double)a, (double)b); }

template <class T> inline T min_value() { return std::numeric_limits<T>::lowest(); }  // Single.MinValue = -FLT_MAX
template <class T> inline T max_value() { return std::numeric_limits<T>::max(); }

// ---- dtype dispatch ---------------------------------------------------------------------------------------------------

#define HREF_NUMERIC_CASES(M) \
    case DNH_U8: M(uint8_t) break; case DNH_I8: M(int8_t) break; case DNH_I16: M(int16_t) break; case DNH_U16: M(uint16_t) break; \
    case DNH_I32: M(int32_t) break; case DNH_U32: M(uint32_t) break; \
    case DNH_I64: M(int64_t) break; case DNH_U64: M(uint64_t) break; case DNH_F32: M(float) break; case DNH_F64: M(double) break;
#define HREF_ALL_CASES(M) case DNH_BOOL: M(uint8_t) break; HREF_NUMERIC_CASES(M)

inline int dtype_size(int dt) {
    switch (dt) {
        case DNH_BOOL: case DNH_U8: case DNH_I8: return 1;
        case DNH_I16: case DNH_U16: return 2;
        case DNH_I32: case DNH_U32: case DNH_F32: return 4;
        case DNH_I64: case DNH_U64: case DNH_F64: return 8;
    }
    return 0;
}

// ---- element-wise drivers ---------------------------------------------------------------------------------------------

template <class TT, class TA, class F>
int run_unary(const DnhTensor* t, const DnhTensor* a, bool simdList, F f) {
    if (!same_shape(t, a)) return DNH_ERR_INVALID_ARG;
    Lay l[2] = {lay_of(t), lay_of(a)};
    elemwise_layouts(l);
    bool threads = !(simdList && vector_ops_can_use(l));
    int nd = l[0].nd;
    int64_t n = nd ? l[0].shape[nd - 1] : 1, ts = nd ? l[0].stride[nd - 1] : 0, as = nd ? l[1].stride[nd - 1] : 0;
    TT* tp = (TT*)t->base;
    const TA* ap = (const TA*)a->base;
    const Lay* ops[2] = {&l[0], &l[1]};
    for_rows<2>(nd, l[0].shape, ops, threads, [=](const int64_t* addr, const int64_t*) {
        TT* tr = tp + addr[0];
        const TA* ar = ap + addr[1];
        for (int64_t i = 0; i < n; i++) tr[i * ts] = f(ar[i * as]);
    });
    return DNH_OK;
}

template <class TT, class TA, class F>
int run_binary(const DnhTensor* t, const DnhTensor* a, const DnhTensor* b, bool simdList, F f) {
    if (!same_shape(t, a) || !same_shape(t, b)) return DNH_ERR_INVALID_ARG;
    Lay l[3] = {lay_of(t), lay_of(a), lay_of(b)};
    elemwise_layouts(l);
    bool threads = !(simdList && vector_ops_can_use(l));
    int nd = l[0].nd;
    int64_t n = nd ? l[0].shape[nd - 1] : 1;
    int64_t ts = nd ? l[0].stride[nd - 1] : 0, as = nd ? l[1].stride[nd - 1] : 0, bs = nd ? l[2].stride[nd - 1] : 0;
    TT* tp = (TT*)t->base;
    const TA* ap = (const TA*)a->base;
    const TA* bp = (const TA*)b->base;
    const Lay* ops[3] = {&l[0], &l[1], &l[2]};
    for_rows<3>(nd, l[0].shape, ops, threads, [=](const int64_t* addr, const int64_t*) {
        TT* tr = tp + addr[0];
        const TA* ar = ap + addr[1];
        const TA* br = bp + addr[2];
        for (int64_t i = 0; i < n; i++) tr[i * ts] = f(ar[i * as], br[i * bs]);
    });
    return DNH_OK;
}

// ---- folds ------------------------------------------------------------------------------------------------------------

// ApplyAxisFold (ScalarOps.fs:299-361): per target element a strictly sequential left fold over the last source axis.
template <class TT, class TS, class State, class Step, class Extract>
int run_fold(const DnhTensor* t, const DnhTensor* s, State init, Step step, Extract extract) {
    if (s->ndims != t->ndims + 1) return DNH_ERR_INVALID_ARG;
    for (int d = 0; d < t->ndims; d++)
        if (t->shape[d] != s->shape[d]) return DNH_ERR_INVALID_ARG;
    Lay lt = lay_of(t), ls = lay_of(s);
    int nd = s->ndims;
    int64_t n = s->shape[nd - 1], ss = s->stride[nd - 1];
    // iterate the target space extended by a dummy last dim of size 1 so for_rows walks all target elements
    Lay lt2 = lt;
    lt2.nd = nd;
    lt2.shape[nd - 1] = 1;
    lt2.stride[nd - 1] = 0;
    int64_t shape[DNH_MAX_DIMS];
    for (int d = 0; d < nd; d++) shape[d] = d < nd - 1 ? s->shape[d] : 1;
    TT* tp = (TT*)t->base;
    const TS* sp = (const TS*)s->base;
    const Lay* ops[2] = {&lt2, &ls};
    for_rows<2>(nd, shape, ops, true, [=](const int64_t* addr, const int64_t*) {
        State st = init;
        const TS* sr = sp + addr[1];
        for (int64_t i = 0; i < n; i++) st = step(st, sr[i * ss], i);
        tp[addr[0]] = extract(st);
    });
    return DNH_OK;
}

template <class T> struct ArgState { int64_t pos; T val; };

// ---- generic position iterator for the sequential ops (PosIter32, FastAccess.fs:67-123) --------------------------------

struct PosIter {
    int nd;
    int64_t pos[DNH_MAX_DIMS];
    int64_t addr;
    bool active;
    const Lay* l;
    explicit PosIter(const Lay* lay) : nd(lay->nd), addr(lay->offset), active(true), l(lay) {
        for (int d = 0; d < DNH_MAX_DIMS; d++) pos[d] = 0;
        for (int d = 0; d < nd; d++)
            if (l->shape[d] <= 0) active = false;
    }
    void next() {
        int d = nd - 1;
        for (; d >= 0; d--) {
            if (pos[d] == l->shape[d] - 1) {
                addr -= pos[d] * l->stride[d];
                pos[d] = 0;
            } else {
                addr += l->stride[d];
                pos[d]++;
                break;
            }
        }
        if (d < 0) active = false;
    }
};

// FastLayout32.Addr (FastAccess.fs:51-61): checked address; false when any coordinate is out of range.
inline bool checked_addr(const Lay& l, const int64_t* pos, int64_t* out) {
    int64_t a = l.offset;
    for (int d = 0; d < l.nd; d++) {
        if (pos[d] < 0 || pos[d] >= l.shape[d]) return false;
        a += pos[d] * l.stride[d];
    }
    *out = a;
    return true;
}

// Convert: the reference's unchecked Expression.Convert (ScalarPrimitives.fs:50-52).  For a float that does not fit an integer target
// the CLI standard leaves the result unspecified; the rule below is what the reference's runtime does on 64-bit x86 (cvtt* sentinel =
// the type's minimum for int32 / int64, narrower targets through int32, uint32 through int64, uint64 through the runtime's
// 2^63 split), written out instead of relying on the C cast, whose out-of-range result is undefined.  Parity unpinned: no file of the
// reference fixes these values; the tests check this function against vectors worked out from the rule by hand.
template <class F> inline int32_t fp_to_i32(F x) { return (x >= (F)-2147483648.0 && x < (F)2147483648.0) ? (int32_t)x : INT32_MIN; }
template <class F> inline int64_t fp_to_i64(F x) {
    return (x >= (F)-9223372036854775808.0 && x < (F)9223372036854775808.0) ? (int64_t)x : INT64_MIN;
}
template <class TT, class TA> inline TT convert_elem(TA x) {
    if constexpr (std::is_floating_point<TA>::value && !std::is_floating_point<TT>::value) {
        if constexpr (std::is_same<TT, int32_t>::value) return fp_to_i32(x);
        else if constexpr (std::is_same<TT, int64_t>::value) return fp_to_i64(x);
        else if constexpr (sizeof(TT) <= 2) return (TT)(uint32_t)fp_to_i32(x);
        else if constexpr (std::is_same<TT, uint32_t>::value) return (uint32_t)(uint64_t)fp_to_i64(x);
        else {
            if (x < (TA)9223372036854775808.0) return (uint64_t)fp_to_i64(x);
            return (uint64_t)fp_to_i64(x - (TA)9223372036854775808.0) + 0x8000000000000000ull;
        }
    } else {
        return (TT)x;
    }
}

template <class TT>
int convert_from(const DnhTensor* t, const DnhTensor* a) {
#define M(TA) return run_unary<TT, TA>(t, a, false, [](TA x) { return convert_elem<TT, TA>(x); });
    switch (a->dtype) { HREF_ALL_CASES(M) default: return DNH_ERR_NOT_SUPPORTED; }
#undef M
}
inline int convert_to_bool(const DnhTensor* t, const DnhTensor* a) {
#define M(TA) return run_unary<uint8_t, TA>(t, a, false, [](TA x) { return (uint8_t)(x != TA(0)); });
    switch (a->dtype) { HREF_ALL_CASES(M) default: return DNH_ERR_NOT_SUPPORTED; }
#undef M
}

}  // namespace

extern "C" {

int32_t href_set_threads(int32_t n) { g_threads = n; return DNH_OK; }
int32_t href_get_threads(void) { return nthreads(); }

// FillConst: ScalarOps.fs:363-365; single-threaded when VectorOps applies (HostBackend.fs:187-190).
int32_t href_fill_const(const DnhTensor* t, const void* value) {
    if (!valid(t)) return DNH_ERR_INVALID_ARG;
    Lay l[1] = {lay_of(t)};
    elemwise_layouts(l);
    bool threads = !vector_ops_can_use(l);
    int nd = l[0].nd;
    int64_t n = nd ? l[0].shape[nd - 1] : 1, ts = nd ? l[0].stride[nd - 1] : 0;
    const Lay* ops[1] = {&l[0]};
#define M(T) { T v; std::memcpy(&v, value, sizeof(T)); T* tp = (T*)t->base; \
        for_rows<1>(nd, l[0].shape, ops, threads, [=](const int64_t* addr, const int64_t*) { \
            T* tr = tp + addr[0]; for (int64_t i = 0; i < n; i++) tr[i * ts] = v; }); }
    switch (t->dtype) { HREF_ALL_CASES(M) default: return DNH_ERR_NOT_SUPPORTED; }
#undef M
    return DNH_OK;
}

// FillIncrementing: ScalarOps.fs:367-370 — start + incr * T(pos[0]).
int32_t href_fill_incrementing(const DnhTensor* t, const void* start, const void* incr) {
    if (!valid(t) || t->ndims < 1) return DNH_ERR_INVALID_ARG;
    Lay l = lay_of(t);
    int nd = l.nd;
    int64_t n = l.shape[nd - 1], ts = l.stride[nd - 1];
    const Lay* ops[1] = {&l};
#define M(T) { T s0, inc; std::memcpy(&s0, start, sizeof(T)); std::memcpy(&inc, incr, sizeof(T)); T* tp = (T*)t->base; \
        for_rows<1>(nd, l.shape, ops, true, [=](const int64_t* addr, const int64_t* pos) { \
            T* tr = tp + addr[0]; \
            for (int64_t i = 0; i < n; i++) { int64_t p0 = nd == 1 ? i : pos[0]; tr[i * ts] = wrap_add<T>(s0, wrap_mul<T>(inc, (T)p0)); } }); }
    switch (t->dtype) { HREF_NUMERIC_CASES(M) default: return DNH_ERR_NOT_SUPPORTED; }
#undef M
    return DNH_OK;
}

// Copy: HostBackend.fs:196-208 (block copy / VectorOps / ScalarOps — identical results).
int32_t href_copy(const DnhTensor* t, const DnhTensor* a) {
    if (!valid(t) || !valid(a) || t->dtype != a->dtype) return DNH_ERR_INVALID_ARG;
#define M(T) return run_unary<T, T>(t, a, true, [](T x) { return x; });
    switch (t->dtype) { HREF_ALL_CASES(M) default: return DNH_ERR_NOT_SUPPORTED; }
#undef M
}

// Convert: ScalarOps.fs:376-379, ScalarPrimitives.fs:50-52 (Expression.Convert, unchecked).  bool<->number follows the
// C++ static_cast rule of the reference's device kernel (Cuda/Kernels/Elemwise.cuh:50-63): nonzero -> true, true -> 1.
int32_t href_convert(const DnhTensor* t, const DnhTensor* a) {
    if (!valid(t) || !valid(a)) return DNH_ERR_INVALID_ARG;
#define M(TT) return convert_from<TT>(t, a);
    switch (t->dtype) {
        case DNH_BOOL: return convert_to_bool(t, a);
        HREF_NUMERIC_CASES(M)
        default: return DNH_ERR_NOT_SUPPORTED;
    }
#undef M
}

// Unary ops: ScalarOps.fs:381-493.
int32_t href_unary(int32_t op, const DnhTensor* t, const DnhTensor* a) {
    if (!valid(t) || !valid(a) || t->dtype != a->dtype) return DNH_ERR_INVALID_ARG;
    int dt = t->dtype;
    bool fp = dt == DNH_F32 || dt == DNH_F64;
    bool sgnd = fp || dt == DNH_I8 || dt == DNH_I16 || dt == DNH_I32 || dt == DNH_I64;
    if (op == DNH_NEGATE) {
        if (dt != DNH_BOOL) return DNH_ERR_NOT_SUPPORTED;
        return run_unary<uint8_t, uint8_t>(t, a, false, [](uint8_t x) { return (uint8_t)(x ? 0 : 1); });
    }
    if (dt == DNH_BOOL) return DNH_ERR_NOT_SUPPORTED;
    switch (op) {
        case DNH_UNARY_PLUS:
#define M(T) return run_unary<T, T>(t, a, false, [](T x) { return x; });
            switch (dt) { HREF_NUMERIC_CASES(M) } return DNH_ERR_NOT_SUPPORTED;
#undef M
        case DNH_UNARY_MINUS:
            if (!sgnd) return DNH_ERR_NOT_SUPPORTED;
#define M(T) return run_unary<T, T>(t, a, true, [](T x) { return wrap_neg<T>(x); });
            switch (dt) { case DNH_I8: M(int8_t) case DNH_I16: M(int16_t) case DNH_I32: M(int32_t) case DNH_I64: M(int64_t) case DNH_F32: M(float) case DNH_F64: M(double) }
            return DNH_ERR_NOT_SUPPORTED;
#undef M
        case DNH_ABS:
            if (!sgnd) return DNH_ERR_NOT_SUPPORTED;
#define M(T) return run_unary<T, T>(t, a, true, [](T x) { return wrap_abs<T>(x); });
            switch (dt) { case DNH_I8: M(int8_t) case DNH_I16: M(int16_t) case DNH_I32: M(int32_t) case DNH_I64: M(int64_t) case DNH_F32: M(float) case DNH_F64: M(double) }
            return DNH_ERR_NOT_SUPPORTED;
#undef M
        case DNH_SGN:  // Sgn.fs implements int16/int32/int64/single/double only
#define M(T) return run_unary<T, T>(t, a, false, [](T x) { return sgn_of<T>(x); });
            switch (dt) { case DNH_I16: M(int16_t) case DNH_I32: M(int32_t) case DNH_I64: M(int64_t) case DNH_F32: M(float) case DNH_F64: M(double) }
            return DNH_ERR_NOT_SUPPORTED;
#undef M
        default: break;
    }
    if (!fp) return DNH_ERR_NOT_SUPPORTED;
#define FPCASE(OP, FN, SIMD) case OP: \
        if (dt == DNH_F32) return run_unary<float, float>(t, a, SIMD, [](float x) { return FN<float>(x); }); \
        return run_unary<double, double>(t, a, SIMD, [](double x) { return FN<double>(x); });
    switch (op) {
        FPCASE(DNH_LOG, f_log, false) FPCASE(DNH_LOG10, f_log10, false) FPCASE(DNH_EXP, f_exp, false)
        FPCASE(DNH_SIN, f_sin, false) FPCASE(DNH_COS, f_cos, false) FPCASE(DNH_TAN, f_tan, false)
        FPCASE(DNH_ASIN, f_asin, false) FPCASE(DNH_ACOS, f_acos, false) FPCASE(DNH_ATAN, f_atan, false)
        FPCASE(DNH_SINH, f_sinh, false) FPCASE(DNH_COSH, f_cosh, false) FPCASE(DNH_TANH, f_tanh, false)
        FPCASE(DNH_SQRT, f_sqrt, true) FPCASE(DNH_CEILING, f_ceil, false) FPCASE(DNH_FLOOR, f_floor, false)
        FPCASE(DNH_ROUND, f_round, false) FPCASE(DNH_TRUNCATE, f_trunc, false)
    }
#undef FPCASE
    return DNH_ERR_NOT_SUPPORTED;
}

// IsFinite: ScalarPrimitives.fs:181-188.
int32_t href_is_finite(const DnhTensor* t, const DnhTensor* a) {
    if (!valid(t) || !valid(a) || t->dtype != DNH_BOOL) return DNH_ERR_INVALID_ARG;
    switch (a->dtype) {
        case DNH_F32: return run_unary<uint8_t, float>(t, a, false, [](float x) { return (uint8_t)(std::isfinite(x) ? 1 : 0); });
        case DNH_F64: return run_unary<uint8_t, double>(t, a, false, [](double x) { return (uint8_t)(std::isfinite(x) ? 1 : 0); });
#define M(T) return run_unary<uint8_t, T>(t, a, false, [](T) { return (uint8_t)1; });
        case DNH_U8: M(uint8_t) case DNH_I8: M(int8_t) case DNH_I16: M(int16_t) case DNH_U16: M(uint16_t) case DNH_I32: M(int32_t) case DNH_U32: M(uint32_t)
        case DNH_I64: M(int64_t) case DNH_U64: M(uint64_t)
#undef M
    }
    return DNH_ERR_NOT_SUPPORTED;
}

// Binary ops: ScalarOps.fs:495-533, 565-575.
int32_t href_binary(int32_t op, const DnhTensor* t, const DnhTensor* a, const DnhTensor* b) {
    if (!valid(t) || !valid(a) || !valid(b) || t->dtype != a->dtype || t->dtype != b->dtype) return DNH_ERR_INVALID_ARG;
    int dt = t->dtype;
    if (op == DNH_AND || op == DNH_OR || op == DNH_XOR) {
        if (dt != DNH_BOOL) return DNH_ERR_NOT_SUPPORTED;
        if (op == DNH_AND) return run_binary<uint8_t, uint8_t>(t, a, b, false, [](uint8_t x, uint8_t y) { return (uint8_t)((x && y) ? 1 : 0); });
        if (op == DNH_OR) return run_binary<uint8_t, uint8_t>(t, a, b, false, [](uint8_t x, uint8_t y) { return (uint8_t)((x || y) ? 1 : 0); });
        return run_binary<uint8_t, uint8_t>(t, a, b, false, [](uint8_t x, uint8_t y) { return (uint8_t)(((x != 0) != (y != 0)) ? 1 : 0); });
    }
    if (dt == DNH_BOOL) return DNH_ERR_NOT_SUPPORTED;
    if (op == DNH_POWER) {
        if (dt == DNH_F32) return run_binary<float, float>(t, a, b, false, [](float x, float y) { return f_pow<float>(x, y); });
        if (dt == DNH_F64) return run_binary<double, double>(t, a, b, false, [](double x, double y) { return f_pow<double>(x, y); });
        return DNH_ERR_NOT_SUPPORTED;
    }
#define M(T) switch (op) { \
        case DNH_ADD: return run_binary<T, T>(t, a, b, true, [](T x, T y) { return wrap_add<T>(x, y); }); \
        case DNH_SUBTRACT: return run_binary<T, T>(t, a, b, true, [](T x, T y) { return wrap_sub<T>(x, y); }); \
        case DNH_MULTIPLY: return run_binary<T, T>(t, a, b, true, [](T x, T y) { return wrap_mul<T>(x, y); }); \
        case DNH_DIVIDE: return run_binary<T, T>(t, a, b, true, [](T x, T y) { return safe_div<T>(x, y); }); \
        case DNH_MODULO: return run_binary<T, T>(t, a, b, false, [](T x, T y) { return safe_mod<T>(x, y); }); \
        case DNH_MAX_ELEMWISE: return run_binary<T, T>(t, a, b, true, [](T x, T y) { return x > y ? x : y; }); \
        case DNH_MIN_ELEMWISE: return run_binary<T, T>(t, a, b, true, [](T x, T y) { return x < y ? x : y; }); \
        default: return DNH_ERR_NOT_SUPPORTED; }
    switch (dt) { HREF_NUMERIC_CASES(M) }
#undef M
    return DNH_ERR_NOT_SUPPORTED;
}

// Comparisons: ScalarOps.fs:535-563.
int32_t href_compare(int32_t op, const DnhTensor* t, const DnhTensor* a, const DnhTensor* b) {
    if (!valid(t) || !valid(a) || !valid(b) || t->dtype != DNH_BOOL || a->dtype != b->dtype) return DNH_ERR_INVALID_ARG;
#define M(T) switch (op) { \
        case DNH_EQUAL: return run_binary<uint8_t, T>(t, a, b, false, [](T x, T y) { return (uint8_t)(x == y); }); \
        case DNH_NOT_EQUAL: return run_binary<uint8_t, T>(t, a, b, false, [](T x, T y) { return (uint8_t)(x != y); }); \
        case DNH_LESS: return run_binary<uint8_t, T>(t, a, b, false, [](T x, T y) { return (uint8_t)(x < y); }); \
        case DNH_LESS_OR_EQUAL: return run_binary<uint8_t, T>(t, a, b, false, [](T x, T y) { return (uint8_t)(x <= y); }); \
        case DNH_GREATER: return run_binary<uint8_t, T>(t, a, b, false, [](T x, T y) { return (uint8_t)(x > y); }); \
        case DNH_GREATER_OR_EQUAL: return run_binary<uint8_t, T>(t, a, b, false, [](T x, T y) { return (uint8_t)(x >= y); }); \
        default: return DNH_ERR_NOT_SUPPORTED; }
    switch (a->dtype) { HREF_ALL_CASES(M) }
#undef M
    return DNH_ERR_NOT_SUPPORTED;
}

// IfThenElse: ScalarOps.fs:577-581 (ApplyTernaryOp :178-230).
int32_t href_if_then_else(const DnhTensor* t, const DnhTensor* c, const DnhTensor* a, const DnhTensor* b) {
    if (!valid(t) || !valid(c) || !valid(a) || !valid(b) || c->dtype != DNH_BOOL || t->dtype != a->dtype || t->dtype != b->dtype)
        return DNH_ERR_INVALID_ARG;
    if (!same_shape(t, c) || !same_shape(t, a) || !same_shape(t, b)) return DNH_ERR_INVALID_ARG;
    Lay l[4] = {lay_of(t), lay_of(c), lay_of(a), lay_of(b)};
    elemwise_layouts(l);
    int nd = l[0].nd;
    int64_t n = nd ? l[0].shape[nd - 1] : 1;
    int64_t ts = nd ? l[0].stride[nd - 1] : 0, cs = nd ? l[1].stride[nd - 1] : 0, as = nd ? l[2].stride[nd - 1] : 0, bs = nd ? l[3].stride[nd - 1] : 0;
    const uint8_t* cp = (const uint8_t*)c->base;
    const Lay* ops[4] = {&l[0], &l[1], &l[2], &l[3]};
#define M(T) { T* tp = (T*)t->base; const T* ap = (const T*)a->base; const T* bp = (const T*)b->base; \
        for_rows<4>(nd, l[0].shape, ops, true, [=](const int64_t* addr, const int64_t*) { \
            for (int64_t i = 0; i < n; i++) tp[addr[0] + i * ts] = cp[addr[1] + i * cs] ? ap[addr[2] + i * as] : bp[addr[3] + i * bs]; }); }
    switch (t->dtype) { HREF_ALL_CASES(M) default: return DNH_ERR_NOT_SUPPORTED; }
#undef M
    return DNH_OK;
}

// SumLastAxis .. CountTrueLastAxis: ScalarOps.fs:606-636.
int32_t href_reduce_last_axis(int32_t op, const DnhTensor* t, const DnhTensor* s) {
    if (!valid(t) || !valid(s) || s->ndims < 1) return DNH_ERR_INVALID_ARG;
    if (op == DNH_ALL || op == DNH_ANY) {
        if (s->dtype != DNH_BOOL || t->dtype != DNH_BOOL) return DNH_ERR_INVALID_ARG;
        if (op == DNH_ALL)
            return run_fold<uint8_t, uint8_t, bool>(t, s, true, [](bool r, uint8_t v, int64_t) { return r && v != 0; }, [](bool r) { return (uint8_t)r; });
        return run_fold<uint8_t, uint8_t, bool>(t, s, false, [](bool r, uint8_t v, int64_t) { return r || v != 0; }, [](bool r) { return (uint8_t)r; });
    }
    if (op == DNH_COUNT_TRUE) {
        if (s->dtype != DNH_BOOL || t->dtype != DNH_I64) return DNH_ERR_INVALID_ARG;
        return run_fold<int64_t, uint8_t, int64_t>(t, s, 0, [](int64_t r, uint8_t v, int64_t) { return v ? r + 1 : r; }, [](int64_t r) { return r; });
    }
    if (t->dtype != s->dtype) return DNH_ERR_INVALID_ARG;
#define M(T) switch (op) { \
        case DNH_SUM: return run_fold<T, T, T>(t, s, T(0), [](T r, T v, int64_t) { return wrap_add<T>(r, v); }, [](T r) { return r; }); \
        case DNH_PRODUCT: return run_fold<T, T, T>(t, s, T(1), [](T r, T v, int64_t) { return wrap_mul<T>(r, v); }, [](T r) { return r; }); \
        case DNH_MAX: return run_fold<T, T, T>(t, s, min_value<T>(), [](T r, T v, int64_t) { return r > v ? r : v; }, [](T r) { return r; }); \
        case DNH_MIN: return run_fold<T, T, T>(t, s, max_value<T>(), [](T r, T v, int64_t) { return r < v ? r : v; }, [](T r) { return r; }); \
        default: return DNH_ERR_NOT_SUPPORTED; }
    switch (s->dtype) { HREF_NUMERIC_CASES(M) }
#undef M
    return DNH_ERR_NOT_SUPPORTED;
}

// ArgMaxLastAxis / ArgMinLastAxis: ScalarOps.fs:638-654.  State (NotFound, minValue|maxValue); strict comparison.
int32_t href_arg_reduce_last_axis(int32_t op, const DnhTensor* t, const DnhTensor* s) {
    if (!valid(t) || !valid(s) || s->ndims < 1 || t->dtype != DNH_I64) return DNH_ERR_INVALID_ARG;
#define M(T) { using S = ArgState<T>; \
        if (op == DNH_ARG_MAX) return run_fold<int64_t, T, S>(t, s, S{kNotFound, min_value<T>()}, \
            [](S st, T v, int64_t i) { return v > st.val ? S{i, v} : st; }, [](S st) { return st.pos; }); \
        if (op == DNH_ARG_MIN) return run_fold<int64_t, T, S>(t, s, S{kNotFound, max_value<T>()}, \
            [](S st, T v, int64_t i) { return v < st.val ? S{i, v} : st; }, [](S st) { return st.pos; }); \
        return DNH_ERR_NOT_SUPPORTED; }
    switch (s->dtype) { HREF_NUMERIC_CASES(M) }
#undef M
    return DNH_ERR_NOT_SUPPORTED;
}

// FindLastAxis: ScalarOps.fs:656-665.
int32_t href_find_last_axis(const void* value, const DnhTensor* t, const DnhTensor* s) {
    if (!valid(t) || !valid(s) || s->ndims < 1 || t->dtype != DNH_I64) return DNH_ERR_INVALID_ARG;
#define M(T) { T val; std::memcpy(&val, value, sizeof(T)); \
        return run_fold<int64_t, T, int64_t>(t, s, kNotFound, \
            [=](int64_t pos, T v, int64_t i) { return pos != kNotFound ? pos : (v == val ? i : kNotFound); }, [](int64_t p) { return p; }); }
    switch (s->dtype) { HREF_ALL_CASES(M) }
#undef M
    return DNH_ERR_NOT_SUPPORTED;
}

// Gather: ScalarOps.fs:583-591.  idx[d] == NULL means identity on source dimension d.
int32_t href_gather(const DnhTensor* t, const DnhTensor* const* idx, int32_t n_idx, const DnhTensor* s) {
    if (!valid(t) || !valid(s) || t->dtype != s->dtype || n_idx != s->ndims) return DNH_ERR_INVALID_ARG;
    Lay lt = lay_of(t), ls = lay_of(s);
    Lay li[DNH_MAX_DIMS];
    for (int d = 0; d < n_idx; d++) {
        if (idx[d]) {
            if (idx[d]->dtype != DNH_I64 || !same_shape(idx[d], t)) return DNH_ERR_INVALID_ARG;
            li[d] = lay_of(idx[d]);
        } else if (d >= t->ndims) return DNH_ERR_INVALID_ARG;
    }
    int es = dtype_size(t->dtype);
    int status = DNH_OK;
    for (PosIter it(&lt); it.active; it.next()) {
        int64_t sp[DNH_MAX_DIMS];
        for (int d = 0; d < n_idx; d++) {
            if (idx[d]) {
                int64_t ia = 0;
                checked_addr(li[d], it.pos, &ia);
                sp[d] = ((const int64_t*)idx[d]->base)[ia];
            } else sp[d] = it.pos[d];
        }
        int64_t sa;
        if (!checked_addr(ls, sp, &sa)) { status = DNH_ERR_INDEX_OUT_OF_RANGE; continue; }
        std::memcpy((char*)t->base + it.addr * es, (const char*)s->base + sa * es, es);
    }
    return status;
}

// Scatter: ScalarOps.fs:593-604 — sequential `trgt[idx] += src`, row-major source order.  The caller zero-fills trgt.
int32_t href_scatter(const DnhTensor* t, const DnhTensor* const* idx, int32_t n_idx, const DnhTensor* s) {
    if (!valid(t) || !valid(s) || t->dtype != s->dtype || n_idx != t->ndims) return DNH_ERR_INVALID_ARG;
    Lay lt = lay_of(t), ls = lay_of(s);
    Lay li[DNH_MAX_DIMS];
    for (int d = 0; d < n_idx; d++) {
        if (idx[d]) {
            if (idx[d]->dtype != DNH_I64 || !same_shape(idx[d], s)) return DNH_ERR_INVALID_ARG;
            li[d] = lay_of(idx[d]);
        } else if (d >= s->ndims) return DNH_ERR_INVALID_ARG;
    }
    int status = DNH_OK;
#define M(T) { T* tp = (T*)t->base; const T* sp = (const T*)s->base; \
        for (PosIter it(&ls); it.active; it.next()) { \
            int64_t tpos[DNH_MAX_DIMS]; \
            for (int d = 0; d < n_idx; d++) { \
                if (idx[d]) { int64_t ia = 0; checked_addr(li[d], it.pos, &ia); tpos[d] = ((const int64_t*)idx[d]->base)[ia]; } \
                else tpos[d] = it.pos[d]; } \
            int64_t ta; \
            if (!checked_addr(lt, tpos, &ta)) { status = DNH_ERR_INDEX_OUT_OF_RANGE; continue; } \
            tp[ta] = wrap_add<T>(tp[ta], sp[it.addr]); } }
    switch (t->dtype) { HREF_NUMERIC_CASES(M) default: return DNH_ERR_NOT_SUPPORTED; }
#undef M
    return status;
}

static bool mask_value(const DnhTensor* const* masks, int n, const int64_t* pos) {
    bool m = true;
    for (int d = 0; d < n; d++)
        if (masks[d]) m = m && ((const uint8_t*)masks[d]->base)[masks[d]->offset + pos[d] * masks[d]->stride[0]] != 0;
    return m;
}

static int check_masks(const DnhTensor* const* masks, int n, const DnhTensor* full) {
    if (n != full->ndims) return DNH_ERR_INVALID_ARG;
    for (int d = 0; d < n; d++)
        if (masks[d] && (masks[d]->dtype != DNH_BOOL || masks[d]->ndims != 1 || masks[d]->shape[0] != full->shape[d])) return DNH_ERR_INVALID_ARG;
    return DNH_OK;
}

// MaskedGet: ScalarOps.fs:667-681 — single-threaded order-preserving compaction.
int32_t href_masked_get(const DnhTensor* t, const DnhTensor* s, const DnhTensor* const* masks, int32_t n_masks) {
    if (!valid(t) || !valid(s) || t->dtype != s->dtype) return DNH_ERR_INVALID_ARG;
    if (int e = check_masks(masks, n_masks, s)) return e;
    Lay lt = lay_of(t), ls = lay_of(s);
    int es = dtype_size(t->dtype);
    PosIter ti(&lt), si(&ls);
    while (ti.active && si.active) {
        if (mask_value(masks, n_masks, si.pos)) {
            std::memcpy((char*)t->base + ti.addr * es, (const char*)s->base + si.addr * es, es);
            ti.next();
        }
        si.next();
    }
    return DNH_OK;
}

// MaskedSet: ScalarOps.fs:683-697.
int32_t href_masked_set(const DnhTensor* t, const DnhTensor* const* masks, int32_t n_masks, const DnhTensor* s) {
    if (!valid(t) || !valid(s) || t->dtype != s->dtype) return DNH_ERR_INVALID_ARG;
    if (int e = check_masks(masks, n_masks, t)) return e;
    Lay lt = lay_of(t), ls = lay_of(s);
    int es = dtype_size(t->dtype);
    PosIter ti(&lt), si(&ls);
    while (ti.active) {
        if (mask_value(masks, n_masks, ti.pos)) {
            if (!si.active) break;
            std::memcpy((char*)t->base + ti.addr * es, (const char*)s->base + si.addr * es, es);
            si.next();
        }
        ti.next();
    }
    return DNH_OK;
}

// TrueIndices: ScalarOps.fs:699-707 — rows of positions of true elements, row-major order.
int32_t href_true_indices(const DnhTensor* t, const DnhTensor* s) {
    if (!valid(t) || !valid(s) || t->dtype != DNH_I64 || s->dtype != DNH_BOOL || t->ndims != 2 || t->shape[1] != s->ndims) return DNH_ERR_INVALID_ARG;
    Lay lt = lay_of(t), ls = lay_of(s);
    PosIter ti(&lt), si(&ls);
    while (ti.active && si.active) {
        if (((const uint8_t*)s->base)[si.addr]) {
            for (int d = 0; d < s->ndims; d++) {
                ((int64_t*)t->base)[ti.addr] = si.pos[d];
                ti.next();
            }
        }
        si.next();
    }
    return DNH_OK;
}

// Dot: HostBackend.fs:463-546.  The reference hands fp32/fp64 to MKL (sdot/sgemv/sgemm/sgemm_batch), whose summation
// order is not recoverable; this restatement accumulates k = 0..K-1 sequentially in T, which is also what the
// reference's non-BLAS path does (multiply then FillSumAxis, HostBackend.fs:544-546).  Threads split the output rows.
int32_t href_dot(const DnhTensor* t, const DnhTensor* a, const DnhTensor* b) {
    if (!valid(t) || !valid(a) || !valid(b) || t->dtype != a->dtype || t->dtype != b->dtype) return DNH_ERR_INVALID_ARG;
    int nt = t->ndims, na = a->ndims, nb = b->ndims;
    // normalise everything to batched [batch..., M, K] x [batch..., K, N] -> [batch..., M, N]
    Lay lt = lay_of(t), la = lay_of(a), lb = lay_of(b);
    int64_t M, N, K;
    int64_t tsm, tsn, asm_, ask, bsk, bsn;
    int nbatch = 0;
    if (nt == 0 && na == 1 && nb == 1) {
        if (a->shape[0] != b->shape[0]) return DNH_ERR_INVALID_ARG;
        M = 1; N = 1; K = a->shape[0]; tsm = tsn = 0; asm_ = 0; ask = a->stride[0]; bsk = b->stride[0]; bsn = 0;
    } else if (nt == 1 && na == 2 && nb == 1) {
        if (t->shape[0] != a->shape[0] || a->shape[1] != b->shape[0]) return DNH_ERR_INVALID_ARG;
        M = a->shape[0]; N = 1; K = a->shape[1]; tsm = t->stride[0]; tsn = 0; asm_ = a->stride[0]; ask = a->stride[1]; bsk = b->stride[0]; bsn = 0;
    } else if (nt >= 2 && na == nt && nb == nt) {
        nbatch = nt - 2;
        M = a->shape[na - 2]; K = a->shape[na - 1]; N = b->shape[nb - 1];
        if (b->shape[nb - 2] != K || t->shape[nt - 2] != M || t->shape[nt - 1] != N) return DNH_ERR_INVALID_ARG;
        for (int d = 0; d < nbatch; d++)
            if (a->shape[d] != t->shape[d] || b->shape[d] != t->shape[d]) return DNH_ERR_INVALID_ARG;
        tsm = t->stride[nt - 2]; tsn = t->stride[nt - 1]; asm_ = a->stride[na - 2]; ask = a->stride[na - 1]; bsk = b->stride[nb - 2]; bsn = b->stride[nb - 1];
    } else return DNH_ERR_INVALID_ARG;
    int64_t batch = 1;
    for (int d = 0; d < nbatch; d++) batch *= t->shape[d];
    if (batch == 0 || M == 0 || N == 0) return DNH_OK;
#define MDOT(T) { T* tp = (T*)t->base; const T* ap = (const T*)a->base; const T* bp = (const T*)b->base; \
    _Pragma("omp parallel for schedule(static) num_threads(nthreads())") \
    for (int64_t bm = 0; bm < batch * M; bm++) { \
        int64_t bi = bm / M, m = bm % M; \
        int64_t to = lt.offset, ao = la.offset, bo = lb.offset, r = bi; \
        for (int d = nbatch - 1; d >= 0; d--) { int64_t p = r % t->shape[d]; r /= t->shape[d]; to += p * lt.stride[d]; ao += p * la.stride[d]; bo += p * lb.stride[d]; } \
        std::vector<T> acc((size_t)N, T(0)); \
        for (int64_t k = 0; k < K; k++) { \
            T av = ap[ao + m * asm_ + k * ask]; const T* brow = bp + bo + k * bsk; \
            for (int64_t n = 0; n < N; n++) acc[(size_t)n] = wrap_add<T>(acc[(size_t)n], wrap_mul<T>(av, brow[n * bsn])); } \
        for (int64_t n = 0; n < N; n++) tp[to + m * tsm + n * tsn] = acc[(size_t)n]; } }
    switch (t->dtype) { HREF_NUMERIC_CASES(MDOT) default: return DNH_ERR_NOT_SUPPORTED; }
#undef MDOT
    return DNH_OK;
}

}  // extern "C"

namespace {
// BatchedInvert: HostBackend.fs:548-576.  The reference copies src into trgt, hands each matrix to LAPACKE_?getrf and
// LAPACKE_?getri in column-major order and raises SingularMatrixException when either reports info > 0.  BLAS.GetMatrix
// (BlasSupport.fs:148-190, canTranspose=true) passes a row-major matrix as the column-major matrix with the same memory, i.e.
// LAPACK factors the transpose; a column-major matrix is passed as it is; any other layout goes through a column-major copy.
// MKL's binary is not in the reference tree, so LAPACK's published unblocked algorithms are restated in T:
//   getf2: for each column j, the first entry of largest magnitude at or below the diagonal becomes the pivot, rows are
//          exchanged, the column is scaled by 1/pivot (reciprocal when |pivot| >= sfmin) and the trailing block updated;
//   getri: inv(U) by trti2 (column by column), then inv(A).L = inv(U) solved from the last column backwards, then the
//          row exchanges undone as column exchanges in reverse order.
template <class T>
int32_t invert_colmajor(T* a, int64_t n, std::vector<int64_t>& ipiv, std::vector<T>& work) {
    auto A = [&](int64_t i, int64_t j) -> T& { return a[i + j * n]; };
    const T sfmin = std::numeric_limits<T>::min();
    int64_t info = 0;
    for (int64_t j = 0; j < n; j++) {
        int64_t jp = j;
        T best = std::fabs(A(j, j));
        for (int64_t i = j + 1; i < n; i++) {
            const T v = std::fabs(A(i, j));
            if (v > best) { best = v; jp = i; }
        }
        ipiv[(size_t)j] = jp;
        if (A(jp, j) != T(0)) {
            if (jp != j)
                for (int64_t c = 0; c < n; c++) std::swap(A(j, c), A(jp, c));
            if (std::fabs(A(j, j)) >= sfmin) {
                const T r = T(1) / A(j, j);
                for (int64_t i = j + 1; i < n; i++) A(i, j) = A(i, j) * r;
            } else {
                for (int64_t i = j + 1; i < n; i++) A(i, j) = A(i, j) / A(j, j);
            }
        } else if (info == 0) {
            info = j + 1;
        }
        for (int64_t c = j + 1; c < n; c++) {
            const T u = A(j, c);
            for (int64_t i = j + 1; i < n; i++) A(i, c) = A(i, c) - A(i, j) * u;
        }
    }
    if (info > 0) return DNH_ERR_SINGULAR_MATRIX;
    // trti2, upper, non-unit
    for (int64_t j = 0; j < n; j++) {
        if (A(j, j) == T(0)) return DNH_ERR_SINGULAR_MATRIX;
        A(j, j) = T(1) / A(j, j);
        const T ajj = -A(j, j);
        // x := inv(U)[0:j, 0:j] * x for x = A[0:j, j] (trmv, upper, no transpose, non-unit): columns left to right
        for (int64_t c = 0; c < j; c++) {
            const T temp = A(c, j);
            if (temp != T(0)) {
                for (int64_t i = 0; i < c; i++) A(i, j) = A(i, j) + temp * A(i, c);
                A(c, j) = A(c, j) * A(c, c);
            }
        }
        for (int64_t i = 0; i < j; i++) A(i, j) = ajj * A(i, j);
    }
    // inv(A) * L = inv(U), last column first
    for (int64_t j = n - 1; j >= 0; j--) {
        for (int64_t i = j + 1; i < n; i++) { work[(size_t)i] = A(i, j); A(i, j) = T(0); }
        for (int64_t c = j + 1; c < n; c++) {
            const T wv = work[(size_t)c];
            if (wv != T(0))
                for (int64_t i = 0; i < n; i++) A(i, j) = A(i, j) - wv * A(i, c);
        }
    }
    for (int64_t j = n - 2; j >= 0; j--) {
        const int64_t jp = ipiv[(size_t)j];
        if (jp != j)
            for (int64_t i = 0; i < n; i++) std::swap(A(i, j), A(i, jp));
    }
    return DNH_OK;
}

template <class T>
int32_t batched_invert_t(const DnhTensor* t, const DnhTensor* s) {
    const int nd = t->ndims;
    const int64_t n = t->shape[nd - 1];
    int64_t batch = 1;
    for (int d = 0; d < nd - 2; d++) batch *= t->shape[d];
    if (batch == 0 || n == 0) return DNH_OK;
    const int64_t sr = t->stride[nd - 2], sc = t->stride[nd - 1];
    // row-major (passed transposed) or column-major / copied (passed as it is)
    const bool as_transpose = (sc == 1 && sr >= std::max<int64_t>(1, n));
    std::vector<T> a((size_t)(n * n)), work((size_t)n);
    std::vector<int64_t> ipiv((size_t)n);
    T* tp = (T*)t->base;
    const T* sp = (const T*)s->base;
    for (int64_t b = 0; b < batch; b++) {
        int64_t to = t->offset, so = s->offset, r = b;
        for (int d = nd - 3; d >= 0; d--) { const int64_t p = r % t->shape[d]; r /= t->shape[d]; to += p * t->stride[d]; so += p * s->stride[d]; }
        for (int64_t i = 0; i < n; i++)
            for (int64_t j = 0; j < n; j++) {
                const T v = sp[so + i * s->stride[nd - 2] + j * s->stride[nd - 1]];
                if (as_transpose) a[(size_t)(j + i * n)] = v; else a[(size_t)(i + j * n)] = v;
            }
        const int32_t st = invert_colmajor<T>(a.data(), n, ipiv, work);
        if (st != DNH_OK) return st;
        for (int64_t i = 0; i < n; i++)
            for (int64_t j = 0; j < n; j++)
                tp[to + i * sr + j * sc] = as_transpose ? a[(size_t)(j + i * n)] : a[(size_t)(i + j * n)];
    }
    return DNH_OK;
}

}  // namespace

extern "C" {

int32_t href_batched_invert(const DnhTensor* t, const DnhTensor* s) {
    if (!valid(t) || !valid(s) || t->dtype != s->dtype || t->ndims != s->ndims || t->ndims < 2) return DNH_ERR_INVALID_ARG;
    for (int d = 0; d < t->ndims; d++)
        if (t->shape[d] != s->shape[d]) return DNH_ERR_INVALID_ARG;
    if (t->shape[t->ndims - 1] != t->shape[t->ndims - 2]) return DNH_ERR_INVALID_ARG;
    if (t->dtype == DNH_F32) return batched_invert_t<float>(t, s);
    if (t->dtype == DNH_F64) return batched_invert_t<double>(t, s);
    return DNH_ERR_NOT_SUPPORTED;  // "this operation is only supported for floating point numbers" (HostBackend.fs:549-550)
}

}  // extern "C"
