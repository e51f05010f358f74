// hip_tensor.hpp — C++ host side of the HIP tensor backend, header-only, above the C ABI of include/tensor_hip.h.
//
// It mirrors the reference's plugin surface and frontend for this path with the reference's own names:
//   TensorLayout + module functions ....... Tensor/Tensor/TensorLayout.fs
//   TensorHipStorage<T>, TensorHipBackend<T>, TensorHipDevice ... the slot of Tensor/Tensor/Cuda/CudaBackend.fs behind
//                                            ITensorStorage / ITensorBackend / ITensorDevice (Tensor/Tensor/TensorBackend.fs:13-146)
//   Tensor<T> ............................. the prepare-target / broadcast-sources / one-backend-call frontend of
//                                            Tensor/Tensor/Tensor.fs (helpers :4520-4597)
// .NET exceptions map to: InvalidOperation/Argument -> std::invalid_argument, NotSupported -> NotSupportedException,
// IndexOutOfRange -> std::out_of_range, OutOfMemory -> std::bad_alloc, SingularMatrixException under its own name,
// other HIP failures -> HipException.
// No arithmetic on tensor data happens here; every operation is one call into libtensor_hip.so.
#pragma once

#include <cstdint>
#include <algorithm>
#include <cstring>
#include <memory>
#include <new>
#include <optional>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

#include "tensor_hip.h"

namespace Tensor {

using Shape = std::vector<int64_t>;

struct NotSupportedException : std::runtime_error { using std::runtime_error::runtime_error; };
struct HipException : std::runtime_error { using std::runtime_error::runtime_error; };
struct SingularMatrixException : std::runtime_error { using std::runtime_error::runtime_error; };   // Tensor.fs:2831-2834
enum class MatrixPart { Upper, Lower };   // which triangle a symmetric operation reads (TensorBackend.fs)

constexpr int64_t NotFound = DNH_NOT_FOUND;                         // SpecialIdx.NotFound, TensorRng.fs:24
constexpr int64_t Remainder = (-9223372036854775807LL - 1LL) + 3;   // SpecialIdx.Remainder, TensorRng.fs:21

// ---- TensorLayout (TensorLayout.fs:12-24 and the module below it) ---------------------------------------------------------
struct TensorLayout {
    Shape Shape_;
    int64_t Offset = 0;
    Shape Stride;
    int NDims() const { return (int)Shape_.size(); }
    int64_t NElems() const { int64_t n = 1; for (auto s : Shape_) n *= s; return n; }
};

namespace Layout {
inline Shape cStride(const Shape& shp) {
    Shape st(shp.size());
    int64_t cum = 1;
    for (int d = (int)shp.size() - 1; d >= 0; d--) { st[d] = cum; cum *= shp[d]; }
    return st;
}
inline TensorLayout newC(const Shape& shp) { return TensorLayout{shp, 0, cStride(shp)}; }
inline bool isC(const TensorLayout& a) {
    Shape c = cStride(a.Shape_);
    for (size_t d = 0; d < c.size(); d++) if (a.Shape_[d] > 1 && a.Stride[d] != c[d]) return false;
    return true;
}
inline TensorLayout padLeft(TensorLayout a) { a.Shape_.insert(a.Shape_.begin(), 1); a.Stride.insert(a.Stride.begin(), 0); return a; }
inline TensorLayout padRight(TensorLayout a) { a.Shape_.push_back(1); a.Stride.push_back(0); return a; }
inline TensorLayout insertAxis(int ax, TensorLayout a) {
    if (ax < 0 || ax > a.NDims()) throw std::out_of_range("insertAxis: axis out of range");
    a.Shape_.insert(a.Shape_.begin() + ax, 1); a.Stride.insert(a.Stride.begin() + ax, 0); return a;
}
inline TensorLayout broadcastToShape(const Shape& bs, TensorLayout a) {                    // TensorLayout.fs:257-271
    if ((int)bs.size() < a.NDims()) throw std::invalid_argument("Cannot broadcast to a shape of lower rank.");
    while (a.NDims() < (int)bs.size()) a = padLeft(a);
    for (size_t d = 0; d < bs.size(); d++) {
        if (a.Shape_[d] == bs[d]) continue;
        if (a.Shape_[d] == 1) { a.Shape_[d] = bs[d]; a.Stride[d] = 0; }
        else throw std::invalid_argument("Cannot broadcast shape to the requested shape.");
    }
    return a;
}
inline void broadcastToSame(TensorLayout& a, TensorLayout& b) {                            // TensorLayout.fs:246-254
    while (a.NDims() < b.NDims()) a = padLeft(a);
    while (b.NDims() < a.NDims()) b = padLeft(b);
    for (int d = 0; d < a.NDims(); d++) {
        if (a.Shape_[d] == b.Shape_[d]) continue;
        if (a.Shape_[d] == 1) { a.Shape_[d] = b.Shape_[d]; a.Stride[d] = 0; }
        else if (b.Shape_[d] == 1) { b.Shape_[d] = a.Shape_[d]; b.Stride[d] = 0; }
        else throw std::invalid_argument("Cannot broadcast shapes to same size.");
    }
}
inline TensorLayout swapDim(int ax1, int ax2, TensorLayout a) {
    if (ax1 < 0 || ax2 < 0 || ax1 >= a.NDims() || ax2 >= a.NDims()) throw std::invalid_argument("Cannot swap dimensions.");
    std::swap(a.Shape_[ax1], a.Shape_[ax2]); std::swap(a.Stride[ax1], a.Stride[ax2]); return a;
}
inline TensorLayout transpose(const TensorLayout& a) {
    if (a.NDims() < 2) throw std::invalid_argument("cannot transpose non-matrix");
    return swapDim(a.NDims() - 2, a.NDims() - 1, a);
}
// permut[i] is the DESTINATION of axis i (F# List.permute, TensorLayout.fs:358-365)
inline TensorLayout permuteAxes(const std::vector<int>& permut, const TensorLayout& a) {
    if ((int)permut.size() != a.NDims()) throw std::invalid_argument("Permutation must have same rank as shape.");
    TensorLayout r{Shape(a.NDims()), a.Offset, Shape(a.NDims())};
    std::vector<bool> seen(a.NDims(), false);
    for (int i = 0; i < a.NDims(); i++) {
        int p = permut[i];
        if (p < 0 || p >= a.NDims() || seen[p]) throw std::invalid_argument("not a permutation");
        seen[p] = true; r.Shape_[p] = a.Shape_[i]; r.Stride[p] = a.Stride[i];
    }
    return r;
}
inline TensorLayout reverseAxis(int ax, TensorLayout a) {
    if (ax < 0 || ax >= a.NDims()) throw std::out_of_range("axis out of range");
    a.Offset += (a.Shape_[ax] - 1) * a.Stride[ax]; a.Stride[ax] = -a.Stride[ax]; return a;
}
// slice dimension `ax` to [first, last] inclusive, as Rng.Rng (TensorLayout.fs:374-422)
inline TensorLayout sliceDim(int ax, int64_t first, int64_t last, TensorLayout a) {
    if (ax < 0 || ax >= a.NDims()) throw std::out_of_range("axis out of range");
    if (last >= first) {
        if (first < 0 || first >= a.Shape_[ax] || last >= a.Shape_[ax]) throw std::out_of_range("slice out of range");
        a.Offset += first * a.Stride[ax]; a.Shape_[ax] = last + 1 - first;
    } else a.Shape_[ax] = 0;
    return a;
}
// the view without copying when the layout allows (row-major, or singleton insertions/removals), TensorLayout.fs:282-325
inline std::optional<TensorLayout> tryReshape(Shape shp, const TensorLayout& a) {
    int nrem = 0; int64_t sofar = 1;
    for (auto s : shp) { if (s == Remainder) nrem++; else sofar *= s; }
    if (nrem > 1) throw std::invalid_argument("only the size of one dimension can be determined automatically");
    if (nrem == 1) {
        if (sofar == 0 || a.NElems() % sofar != 0) throw std::invalid_argument("cannot reshape: not an integer");
        for (auto& s : shp) if (s == Remainder) s = a.NElems() / sofar;
    }
    int64_t n = 1; for (auto s : shp) n *= s;
    if (n != a.NElems()) throw std::invalid_argument("cannot reshape: number of elements differs");
    if (isC(a)) return TensorLayout{shp, a.Offset, cStride(shp)};
    Shape ns; size_t i = 0, j = 0;
    for (;;) {
        if (i < shp.size() && j < a.Shape_.size() && shp[i] == a.Shape_[j]) { ns.push_back(a.Stride[j]); i++; j++; }
        else if (i < shp.size() && shp[i] == 1) { ns.push_back(0); i++; }
        else if (j < a.Shape_.size() && a.Shape_[j] == 1) j++;
        else if (i == shp.size() && j == a.Shape_.size()) return TensorLayout{shp, a.Offset, ns};
        else return std::nullopt;
    }
}
inline int64_t addr(const std::vector<int64_t>& idx, const TensorLayout& a) {              // checked, TensorLayout.fs:32-42
    if ((int)idx.size() != a.NDims()) throw std::out_of_range("index has other dimensionality than tensor");
    int64_t o = a.Offset;
    for (int d = 0; d < a.NDims(); d++) {
        if (idx[d] < 0 || idx[d] >= a.Shape_[d]) throw std::out_of_range("index out of range");
        o += idx[d] * a.Stride[d];
    }
    return o;
}
}  // namespace Layout

// ---- native plumbing ---------------------------------------------------------------------------------------------------------
template <class T> struct DTypeOf;
template <> struct DTypeOf<bool> { static constexpr int value = DNH_BOOL; };
template <> struct DTypeOf<uint8_t> { static constexpr int value = DNH_U8; };
template <> struct DTypeOf<int8_t> { static constexpr int value = DNH_I8; };
template <> struct DTypeOf<int16_t> { static constexpr int value = DNH_I16; };
template <> struct DTypeOf<uint16_t> { static constexpr int value = DNH_U16; };
template <> struct DTypeOf<int32_t> { static constexpr int value = DNH_I32; };
template <> struct DTypeOf<uint32_t> { static constexpr int value = DNH_U32; };
template <> struct DTypeOf<int64_t> { static constexpr int value = DNH_I64; };
template <> struct DTypeOf<uint64_t> { static constexpr int value = DNH_U64; };
template <> struct DTypeOf<float> { static constexpr int value = DNH_F32; };
template <> struct DTypeOf<double> { static constexpr int value = DNH_F64; };

inline void check(int32_t status) {
    if (status == DNH_OK) return;
    char buf[1024];
    dnh_last_error(buf, sizeof(buf));
    switch (status) {
        case DNH_ERR_INVALID_ARG: throw std::invalid_argument(buf);
        case DNH_ERR_NOT_SUPPORTED: throw NotSupportedException(buf);
        case DNH_ERR_OUT_OF_MEMORY: throw std::bad_alloc();
        case DNH_ERR_INDEX_OUT_OF_RANGE: throw std::out_of_range(buf);
        case DNH_ERR_SINGULAR_MATRIX: throw SingularMatrixException(buf);
        case DNH_ERR_NO_CONVERGENCE: throw std::runtime_error(buf);                  // "SVD did not converge" (HostBackend.fs:598)
        default: throw HipException(buf);
    }
}

// Thread-local options (Tensor/Tensor/Cuda/CudaCfg.fs:14-60): the stream ops are issued on; Stacktrace = read the device
// index-error flag after every Gather/Scatter so an out-of-range index raises at the faulting call, as on the host.
struct Cfg {
    static void*& Stream() { thread_local void* s = nullptr; return s; }
    static bool& Stacktrace() { thread_local bool v = true; return v; }
};

// Device memory owned by one tensor storage (Cuda/CudaBackend.fs:54-93).  The block comes from the library's stream-ordered
// cache under the stream current at creation; while every use is issued on that stream it is released without waiting for
// the device, otherwise with the synchronising dnh_free.
template <class T>
class TensorHipStorage {
  public:
    explicit TensorHipStorage(int64_t nElems) : nElems_(nElems), stream_(Cfg::Stream()) {
        check(dnh_alloc_async((size_t)(nElems > 0 ? nElems : 1) * sizeof(T), stream_, &ptr_));
    }
    ~TensorHipStorage() {
        if (!ptr_) return;
        if (singleStream_) dnh_free_async(ptr_, stream_); else dnh_free(ptr_);
    }
    TensorHipStorage(const TensorHipStorage&) = delete;
    TensorHipStorage& operator=(const TensorHipStorage&) = delete;
    void* Ptr() const {
        if (Cfg::Stream() != stream_) singleStream_ = false;
        return ptr_;
    }
    int64_t NElems() const { return nElems_; }
  private:
    void* ptr_ = nullptr;
    int64_t nElems_;
    void* stream_;
    mutable bool singleStream_ = true;
};

struct TensorHipDevice {                                      // Cuda/CudaBackend.fs:497-507
    static constexpr const char* Id = "Hip";
    static constexpr bool Zeroed = false;
    template <class T> static std::shared_ptr<TensorHipStorage<T>> Create(int64_t nElems) { return std::make_shared<TensorHipStorage<T>>(nElems); }
};

template <class T> class Tensor;

template <class T>
inline DnhTensor desc(const Tensor<T>& t);

// ---- ITensorBackend<'T> (TensorBackend.fs:64-146) ----------------------------------------------------------------------------------
template <class T>
struct TensorHipBackend {
    template <class A> static void unary(int op, const Tensor<T>& trgt, const Tensor<A>& a) { auto t = desc(trgt); auto x = desc(a); check(dnh_unary(op, &t, &x, Cfg::Stream())); }
    static void binary(int op, const Tensor<T>& trgt, const Tensor<T>& a, const Tensor<T>& b) { auto t = desc(trgt); auto x = desc(a); auto y = desc(b); check(dnh_binary(op, &t, &x, &y, Cfg::Stream())); }
    template <class A> static void compare(int op, const Tensor<bool>& trgt, const Tensor<A>& a, const Tensor<A>& b) { auto t = desc(trgt); auto x = desc(a); auto y = desc(b); check(dnh_compare(op, &t, &x, &y, Cfg::Stream())); }
    template <class R> static void reduce(int op, const Tensor<R>& trgt, const Tensor<T>& src) { auto t = desc(trgt); auto s = desc(src); check(dnh_reduce_last_axis(op, &t, &s, Cfg::Stream())); }

    static void Copy(const Tensor<T>& trgt, const Tensor<T>& src) { auto t = desc(trgt); auto s = desc(src); check(dnh_copy(&t, &s, Cfg::Stream())); }
    template <class S> static void Convert(const Tensor<T>& trgt, const Tensor<S>& src) { auto t = desc(trgt); auto s = desc(src); check(dnh_convert(&t, &s, Cfg::Stream())); }
    static void FillConst(T value, const Tensor<T>& trgt) { auto t = desc(trgt); check(dnh_fill_const(&t, &value, Cfg::Stream())); }
    static void FillIncrementing(T start, T incr, const Tensor<T>& trgt) { auto t = desc(trgt); check(dnh_fill_incrementing(&t, &start, &incr, Cfg::Stream())); }

    static void UnaryPlus(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_UNARY_PLUS, t, a); }
    static void UnaryMinus(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_UNARY_MINUS, t, a); }
    static void Abs(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_ABS, t, a); }
    static void Sgn(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_SGN, t, a); }
    static void Log(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_LOG, t, a); }
    static void Log10(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_LOG10, t, a); }
    static void Exp(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_EXP, t, a); }
    static void Sin(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_SIN, t, a); }
    static void Cos(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_COS, t, a); }
    static void Tan(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_TAN, t, a); }
    static void Asin(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_ASIN, t, a); }
    static void Acos(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_ACOS, t, a); }
    static void Atan(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_ATAN, t, a); }
    static void Sinh(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_SINH, t, a); }
    static void Cosh(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_COSH, t, a); }
    static void Tanh(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_TANH, t, a); }
    static void Sqrt(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_SQRT, t, a); }
    static void Ceiling(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_CEILING, t, a); }
    static void Floor(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_FLOOR, t, a); }
    static void Round(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_ROUND, t, a); }
    static void Truncate(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_TRUNCATE, t, a); }
    static void Negate(const Tensor<T>& t, const Tensor<T>& a) { unary(DNH_NEGATE, t, a); }
    static void IsFinite(const Tensor<bool>& trgt, const Tensor<T>& a) { auto t = desc(trgt); auto x = desc(a); check(dnh_is_finite(&t, &x, Cfg::Stream())); }

    static void Add(const Tensor<T>& t, const Tensor<T>& a, const Tensor<T>& b) { binary(DNH_ADD, t, a, b); }
    static void Subtract(const Tensor<T>& t, const Tensor<T>& a, const Tensor<T>& b) { binary(DNH_SUBTRACT, t, a, b); }
    static void Multiply(const Tensor<T>& t, const Tensor<T>& a, const Tensor<T>& b) { binary(DNH_MULTIPLY, t, a, b); }
    static void Divide(const Tensor<T>& t, const Tensor<T>& a, const Tensor<T>& b) { binary(DNH_DIVIDE, t, a, b); }
    static void Modulo(const Tensor<T>& t, const Tensor<T>& a, const Tensor<T>& b) { binary(DNH_MODULO, t, a, b); }
    static void Power(const Tensor<T>& t, const Tensor<T>& a, const Tensor<T>& b) { binary(DNH_POWER, t, a, b); }
    static void MaxElemwise(const Tensor<T>& t, const Tensor<T>& a, const Tensor<T>& b) { binary(DNH_MAX_ELEMWISE, t, a, b); }
    static void MinElemwise(const Tensor<T>& t, const Tensor<T>& a, const Tensor<T>& b) { binary(DNH_MIN_ELEMWISE, t, a, b); }
    static void And(const Tensor<T>& t, const Tensor<T>& a, const Tensor<T>& b) { binary(DNH_AND, t, a, b); }
    static void Or(const Tensor<T>& t, const Tensor<T>& a, const Tensor<T>& b) { binary(DNH_OR, t, a, b); }
    static void Xor(const Tensor<T>& t, const Tensor<T>& a, const Tensor<T>& b) { binary(DNH_XOR, t, a, b); }

    static void Equal(const Tensor<bool>& t, const Tensor<T>& a, const Tensor<T>& b) { compare(DNH_EQUAL, t, a, b); }
    static void NotEqual(const Tensor<bool>& t, const Tensor<T>& a, const Tensor<T>& b) { compare(DNH_NOT_EQUAL, t, a, b); }
    static void Less(const Tensor<bool>& t, const Tensor<T>& a, const Tensor<T>& b) { compare(DNH_LESS, t, a, b); }
    static void LessOrEqual(const Tensor<bool>& t, const Tensor<T>& a, const Tensor<T>& b) { compare(DNH_LESS_OR_EQUAL, t, a, b); }
    static void Greater(const Tensor<bool>& t, const Tensor<T>& a, const Tensor<T>& b) { compare(DNH_GREATER, t, a, b); }
    static void GreaterOrEqual(const Tensor<bool>& t, const Tensor<T>& a, const Tensor<T>& b) { compare(DNH_GREATER_OR_EQUAL, t, a, b); }

    static void IfThenElse(const Tensor<T>& trgt, const Tensor<bool>& cond, const Tensor<T>& ifTrue, const Tensor<T>& ifFalse) {
        auto t = desc(trgt); auto c = desc(cond); auto a = desc(ifTrue); auto b = desc(ifFalse);
        check(dnh_if_then_else(&t, &c, &a, &b, Cfg::Stream()));
    }
    static void checkIndexError() {
        if (!Cfg::Stacktrace()) return;
        int32_t code = 0;
        check(dnh_async_error(Cfg::Stream(), &code));
        check(code);
    }
    // index tensors / masks: nullptr = None / NoMask
    template <class X> static std::vector<DnhTensor> descs(const std::vector<const Tensor<X>*>& ts, std::vector<const DnhTensor*>& ptrs) {
        std::vector<DnhTensor> ds(ts.size());
        ptrs.assign(ts.size(), nullptr);
        for (size_t i = 0; i < ts.size(); i++) if (ts[i]) { ds[i] = desc(*ts[i]); }
        for (size_t i = 0; i < ts.size(); i++) if (ts[i]) ptrs[i] = &ds[i];
        return ds;
    }
    static void Gather(const Tensor<T>& trgt, const std::vector<const Tensor<int64_t>*>& srcIdxs, const Tensor<T>& src) {
        std::vector<const DnhTensor*> p; auto ds = descs(srcIdxs, p); auto t = desc(trgt); auto s = desc(src);
        check(dnh_gather(&t, p.data(), (int32_t)p.size(), &s, Cfg::Stream())); checkIndexError();
    }
    static void Scatter(const Tensor<T>& trgt, const std::vector<const Tensor<int64_t>*>& trgtIdxs, const Tensor<T>& src) {
        std::vector<const DnhTensor*> p; auto ds = descs(trgtIdxs, p); auto t = desc(trgt); auto s = desc(src);
        check(dnh_scatter(&t, p.data(), (int32_t)p.size(), &s, Cfg::Stream())); checkIndexError();
    }
    static void MaskedGet(const Tensor<T>& trgt, const Tensor<T>& src, const std::vector<const Tensor<bool>*>& masks) {
        std::vector<const DnhTensor*> p; auto ds = descs(masks, p); auto t = desc(trgt); auto s = desc(src);
        check(dnh_masked_get(&t, &s, p.data(), (int32_t)p.size(), Cfg::Stream()));
    }
    static void MaskedSet(const Tensor<T>& trgt, const std::vector<const Tensor<bool>*>& masks, const Tensor<T>& src) {
        std::vector<const DnhTensor*> p; auto ds = descs(masks, p); auto t = desc(trgt); auto s = desc(src);
        check(dnh_masked_set(&t, p.data(), (int32_t)p.size(), &s, Cfg::Stream()));
    }
    static void TrueIndices(const Tensor<int64_t>& trgt, const Tensor<bool>& src) { auto t = desc(trgt); auto s = desc(src); check(dnh_true_indices(&t, &s, Cfg::Stream())); }

    static void SumLastAxis(const Tensor<T>& t, const Tensor<T>& s) { reduce(DNH_SUM, t, s); }
    static void ProductLastAxis(const Tensor<T>& t, const Tensor<T>& s) { reduce(DNH_PRODUCT, t, s); }
    static void MinLastAxis(const Tensor<T>& t, const Tensor<T>& s) { reduce(DNH_MIN, t, s); }
    static void MaxLastAxis(const Tensor<T>& t, const Tensor<T>& s) { reduce(DNH_MAX, t, s); }
    static void AllLastAxis(const Tensor<bool>& t, const Tensor<bool>& s) { TensorHipBackend<bool>::reduce(DNH_ALL, t, s); }
    static void AnyLastAxis(const Tensor<bool>& t, const Tensor<bool>& s) { TensorHipBackend<bool>::reduce(DNH_ANY, t, s); }
    static void CountTrueLastAxis(const Tensor<int64_t>& t, const Tensor<bool>& s) { TensorHipBackend<bool>::reduce(DNH_COUNT_TRUE, t, s); }
    static void ArgMinLastAxis(const Tensor<int64_t>& trgt, const Tensor<T>& src) { auto t = desc(trgt); auto s = desc(src); check(dnh_arg_reduce_last_axis(DNH_ARG_MIN, &t, &s, Cfg::Stream())); }
    static void ArgMaxLastAxis(const Tensor<int64_t>& trgt, const Tensor<T>& src) { auto t = desc(trgt); auto s = desc(src); check(dnh_arg_reduce_last_axis(DNH_ARG_MAX, &t, &s, Cfg::Stream())); }
    static void FindLastAxis(T value, const Tensor<int64_t>& trgt, const Tensor<T>& src) { auto t = desc(trgt); auto s = desc(src); check(dnh_find_last_axis(&value, &t, &s, Cfg::Stream())); }

    static void dot(const Tensor<T>& trgt, const Tensor<T>& a, const Tensor<T>& b) { auto t = desc(trgt); auto x = desc(a); auto y = desc(b); check(dnh_dot(&t, &x, &y, Cfg::Stream())); }
    static void VecVecDot(const Tensor<T>& t, const Tensor<T>& a, const Tensor<T>& b) { dot(t, a, b); }
    static void MatVecDot(const Tensor<T>& t, const Tensor<T>& a, const Tensor<T>& b) { dot(t, a, b); }
    static void MatMatDot(const Tensor<T>& t, const Tensor<T>& a, const Tensor<T>& b) { dot(t, a, b); }
    static void BatchedMatMatDot(const Tensor<T>& t, const Tensor<T>& a, const Tensor<T>& b) { dot(t, a, b); }
    static void BatchedInvert(const Tensor<T>& trgt, const Tensor<T>& src) { auto t = desc(trgt); auto s = desc(src); check(dnh_batched_invert(&t, &s, Cfg::Stream())); }
    // trgtU / trgtV both null: singular values only (the reference's `trgtUV: (U, V) option`)
    static void BatchedSVD(const Tensor<T>& trgtS, const Tensor<T>* trgtU, const Tensor<T>* trgtV, const Tensor<T>& src) {
        auto s = desc(trgtS); auto a = desc(src);
        if (trgtU && trgtV) { auto u = desc(*trgtU); auto v = desc(*trgtV); check(dnh_batched_svd(&s, &u, &v, &a, Cfg::Stream())); }
        else check(dnh_batched_svd(&s, nullptr, nullptr, &a, Cfg::Stream()));
    }
    static void SymmetricEigenDecomposition(MatrixPart part, const Tensor<T>& eigVals, const Tensor<T>& eigVecs, const Tensor<T>& src) {
        auto w = desc(eigVals); auto v = desc(eigVecs); auto a = desc(src);
        check(dnh_symmetric_eig(part == MatrixPart::Upper ? 0 : 1, &w, &v, &a, Cfg::Stream()));
    }
};

// ---- Tensor<'T> frontend (Tensor.fs), the part that drives the backend path -----------------------------------------------------------
template <class T>
class Tensor {
  public:
    using Backend = TensorHipBackend<T>;
    Tensor(TensorLayout layout, std::shared_ptr<TensorHipStorage<T>> storage) : layout_(std::move(layout)), storage_(std::move(storage)) {}
    explicit Tensor(const Shape& shape) : layout_(Layout::newC(shape)), storage_(TensorHipDevice::Create<T>(layout_.NElems())) {}   // Tensor.fs:317-325

    const TensorLayout& Layout_() const { return layout_; }
    const Shape& Shape_() const { return layout_.Shape_; }
    int NDims() const { return layout_.NDims(); }
    int64_t NElems() const { return layout_.NElems(); }
    const std::shared_ptr<TensorHipStorage<T>>& Storage() const { return storage_; }
    Tensor Relayout(TensorLayout l) const { return Tensor(std::move(l), storage_); }

    // host <-> device, the HipTensor.transfer / HostTensor.transfer analogue (Cuda/CudaBackend.fs:206-270)
    static Tensor ofHost(const T* data, const Shape& shape) {
        Tensor t(shape);
        if (t.NElems()) check(dnh_memcpy_h2d(t.storage_->Ptr(), data, (size_t)t.NElems() * sizeof(T), Cfg::Stream(), 1));
        return t;
    }
    static Tensor ofHost(const std::vector<T>& data, const Shape& shape) { return ofHost(data.data(), shape); }
    void toHost(T* out) const {
        Tensor c = Layout::isC(layout_) ? *this : Copy();
        if (c.NElems()) check(dnh_memcpy_d2h(out, (const char*)c.storage_->Ptr() + c.layout_.Offset * (int64_t)sizeof(T), (size_t)c.NElems() * sizeof(T), Cfg::Stream(), 1));
    }
    T Value() const {                                                               // Tensor.fs:3761-3777
        if (NDims() != 0) throw std::invalid_argument("Value requires a scalar tensor");
        T v; check(dnh_memcpy_d2h(&v, (const char*)storage_->Ptr() + layout_.Offset * (int64_t)sizeof(T), sizeof(T), Cfg::Stream(), 1)); return v;
    }
    static Tensor filled(const Shape& shape, T value) { Tensor t(shape); Backend::FillConst(value, t); return t; }
    static Tensor zeros(const Shape& shape) { return filled(shape, T(0)); }
    static Tensor scalar(T value) { return filled({}, value); }
    static Tensor counting(int64_t n) { Tensor t(Shape{n}); Backend::FillIncrementing(T(0), T(1), t); return t; }

    // views
    Tensor broadcastTo(const Shape& s) const { return Relayout(Layout::broadcastToShape(s, layout_)); }
    Tensor permuteAxes(const std::vector<int>& p) const { return Relayout(Layout::permuteAxes(p, layout_)); }
    Tensor swapDim(int a, int b) const { return Relayout(Layout::swapDim(a, b, layout_)); }
    Tensor T_() const { return Relayout(Layout::transpose(layout_)); }
    Tensor reverseAxis(int ax) const { return Relayout(Layout::reverseAxis(ax, layout_)); }
    Tensor insertAxis(int ax) const { return Relayout(Layout::insertAxis(ax, layout_)); }
    Tensor padRight() const { return Relayout(Layout::padRight(layout_)); }
    Tensor slice(int ax, int64_t first, int64_t last) const { return Relayout(Layout::sliceDim(ax, first, last, layout_)); }
    Tensor reshape(const Shape& s) const {                                                // ITensor.fs:292-316
        if (auto l = Layout::tryReshape(s, layout_)) return Relayout(*l);
        Tensor c = Copy();
        return c.Relayout(*Layout::tryReshape(s, c.layout_));
    }
    Tensor flatten() const { return reshape({Remainder}); }
    Tensor Copy() const { Tensor t(Shape_()); Backend::Copy(t, *this); return t; }
    void CopyFrom(const Tensor& src) const { Backend::Copy(*this, src.broadcastTo(Shape_())); }
    template <class R> Tensor<R> convert() const { Tensor<R> t(Shape_()); TensorHipBackend<R>::Convert(t, *this); return t; }

    // element-wise (PrepareElemwise, Tensor.fs:4577-4597)
    template <class F> Tensor un(F f) const { Tensor t(Shape_()); f(t, *this); return t; }
    template <class R, class F> static Tensor<R> bin(const Tensor& a0, const Tensor& b0, F f) {
        TensorLayout la = a0.layout_, lb = b0.layout_;
        Layout::broadcastToSame(la, lb);
        Tensor a = a0.Relayout(la), b = b0.Relayout(lb);
        Tensor<R> t(a.Shape_());
        f(t, a, b);
        return t;
    }
    Tensor operator+(const Tensor& o) const { return bin<T>(*this, o, Backend::Add); }
    Tensor operator-(const Tensor& o) const { return bin<T>(*this, o, Backend::Subtract); }
    Tensor operator*(const Tensor& o) const { return bin<T>(*this, o, Backend::Multiply); }
    Tensor operator/(const Tensor& o) const { return bin<T>(*this, o, Backend::Divide); }
    Tensor operator%(const Tensor& o) const { return bin<T>(*this, o, Backend::Modulo); }
    Tensor operator+(T v) const { return *this + scalar(v); }
    Tensor operator*(T v) const { return *this * scalar(v); }
    Tensor operator-() const { return un(Backend::UnaryMinus); }
    Tensor pow(const Tensor& o) const { return bin<T>(*this, o, Backend::Power); }
    Tensor<bool> operator==(const Tensor& o) const { return bin<bool>(*this, o, Backend::Equal); }
    Tensor<bool> operator!=(const Tensor& o) const { return bin<bool>(*this, o, Backend::NotEqual); }
    Tensor<bool> operator<(const Tensor& o) const { return bin<bool>(*this, o, Backend::Less); }
    Tensor<bool> operator<=(const Tensor& o) const { return bin<bool>(*this, o, Backend::LessOrEqual); }
    Tensor<bool> operator>(const Tensor& o) const { return bin<bool>(*this, o, Backend::Greater); }
    Tensor<bool> operator>=(const Tensor& o) const { return bin<bool>(*this, o, Backend::GreaterOrEqual); }
    Tensor<bool> operator>(T v) const { return *this > scalar(v); }
    Tensor operator&(const Tensor& o) const { return bin<T>(*this, o, Backend::And); }
    Tensor operator|(const Tensor& o) const { return bin<T>(*this, o, Backend::Or); }
    Tensor operator^(const Tensor& o) const { return bin<T>(*this, o, Backend::Xor); }
    Tensor operator~() const { return un(Backend::Negate); }
    Tensor abs() const { return un(Backend::Abs); }
    Tensor sgn() const { return un(Backend::Sgn); }
    Tensor tanh() const { return un(Backend::Tanh); }
    Tensor exp() const { return un(Backend::Exp); }
    Tensor log() const { return un(Backend::Log); }
    Tensor sin() const { return un(Backend::Sin); }
    Tensor sqrt() const { return un(Backend::Sqrt); }
    Tensor round() const { return un(Backend::Round); }
    Tensor<bool> isFinite() const { Tensor<bool> t(Shape_()); Backend::IsFinite(t, *this); return t; }
    static Tensor maxElemwise(const Tensor& a, const Tensor& b) { return bin<T>(a, b, Backend::MaxElemwise); }
    static Tensor minElemwise(const Tensor& a, const Tensor& b) { return bin<T>(a, b, Backend::MinElemwise); }
    static Tensor ifThenElse(const Tensor<bool>& cond, const Tensor& ifTrue, const Tensor& ifFalse) {   // Tensor.fs:2055-2083
        TensorLayout lt = ifTrue.layout_, lf = ifFalse.layout_, lc = cond.Layout_();
        Layout::broadcastToSame(lt, lf); Layout::broadcastToSame(lc, lt); Layout::broadcastToSame(lc, lf);
        Tensor t(lt.Shape_);
        Backend::IfThenElse(t, cond.Relayout(lc), ifTrue.Relayout(lt), ifFalse.Relayout(lf));
        return t;
    }
    void FillMultiply(const Tensor& a, const Tensor& b) const { Backend::Multiply(*this, a.broadcastTo(Shape_()), b.broadcastTo(Shape_())); }

    // reductions: the reduced axis is permuted to the last position as a view (Tensor.fs:4544-4567)
    Tensor axisToLast(int ax) const {
        if (ax < 0 || ax >= NDims()) throw std::out_of_range("axis out of range");
        std::vector<int> p;
        for (int d = 0; d < ax; d++) p.push_back(d);
        p.push_back(NDims() - 1);
        for (int d = ax + 1; d < NDims(); d++) p.push_back(d - 1);
        return permuteAxes(p);
    }
    Shape reducedShape(int ax) const { Shape s = Shape_(); if (ax < 0 || ax >= NDims()) throw std::out_of_range("axis out of range"); s.erase(s.begin() + ax); return s; }
    Tensor sumAxis(int ax) const { Tensor t(reducedShape(ax)); Backend::SumLastAxis(t, axisToLast(ax)); return t; }
    Tensor productAxis(int ax) const { Tensor t(reducedShape(ax)); Backend::ProductLastAxis(t, axisToLast(ax)); return t; }
    Tensor maxAxis(int ax) const { Tensor t(reducedShape(ax)); Backend::MaxLastAxis(t, axisToLast(ax)); return t; }
    Tensor minAxis(int ax) const { Tensor t(reducedShape(ax)); Backend::MinLastAxis(t, axisToLast(ax)); return t; }
    Tensor<int64_t> argMaxAxis(int ax) const { Tensor<int64_t> t(reducedShape(ax)); Backend::ArgMaxLastAxis(t, axisToLast(ax)); return t; }
    Tensor<int64_t> argMinAxis(int ax) const { Tensor<int64_t> t(reducedShape(ax)); Backend::ArgMinLastAxis(t, axisToLast(ax)); return t; }
    Tensor<int64_t> findAxis(T value, int ax) const { Tensor<int64_t> t(reducedShape(ax)); Backend::FindLastAxis(value, t, axisToLast(ax)); return t; }
    Tensor<int64_t> countTrueAxis(int ax) const { Tensor<int64_t> t(reducedShape(ax)); Backend::CountTrueLastAxis(t, axisToLast(ax)); return t; }
    Tensor allAxis(int ax) const { Tensor t(reducedShape(ax)); Backend::AllLastAxis(t, axisToLast(ax)); return t; }
    Tensor anyAxis(int ax) const { Tensor t(reducedShape(ax)); Backend::AnyLastAxis(t, axisToLast(ax)); return t; }
    T sum() const { return flatten().sumAxis(0).Value(); }                               // Tensor.fs:2293-2307
    T max() const { return flatten().maxAxis(0).Value(); }
    T min() const { return flatten().minAxis(0).Value(); }
    int64_t countTrue() const { return flatten().countTrueAxis(0).Value(); }
    bool all() const { return flatten().allAxis(0).Value(); }
    bool any() const { return flatten().anyAxis(0).Value(); }
    Tensor<int64_t> trueIdx() const {                                                      // Tensor.fs:2259-2263
        Tensor<int64_t> t(Shape{countTrue(), (int64_t)NDims()});
        Backend::TrueIndices(t, *this);
        return t;
    }

    // gather / scatter (Tensor.fs:2090-2198): nullptr = None; index tensors are broadcast to the iteration shape
    static Tensor gather(const std::vector<const Tensor<int64_t>*>& indices, const Tensor& src) {
        const Tensor<int64_t>* first = nullptr;
        for (auto i : indices) if (i) { first = i; break; }
        if (!first) throw std::invalid_argument("At least one index tensor must not be None.");
        if ((int)indices.size() != src.NDims()) throw std::invalid_argument("For each dimension of src an index tensor must be specified.");
        TensorLayout common = first->Layout_();
        for (auto i : indices) if (i) { TensorLayout l = i->Layout_(); Layout::broadcastToSame(common, l); }
        Tensor trgt(common.Shape_);
        std::vector<Tensor<int64_t>> bc;
        bc.reserve(indices.size());
        std::vector<const Tensor<int64_t>*> p(indices.size(), nullptr);
        for (size_t d = 0; d < indices.size(); d++) if (indices[d]) { bc.push_back(indices[d]->broadcastTo(common.Shape_)); p[d] = &bc.back(); }
        Backend::Gather(trgt, p, src);
        return trgt;
    }
    static Tensor scatter(const std::vector<const Tensor<int64_t>*>& indices, const Shape& trgtShp, const Tensor& src) {
        if (indices.size() != trgtShp.size()) throw std::invalid_argument("For each dimension of the target an index tensor must be specified.");
        Tensor trgt(trgtShp);
        std::vector<Tensor<int64_t>> bc;
        bc.reserve(indices.size());
        std::vector<const Tensor<int64_t>*> p(indices.size(), nullptr);
        for (size_t d = 0; d < indices.size(); d++) if (indices[d]) { bc.push_back(indices[d]->broadcastTo(src.Shape_())); p[d] = &bc.back(); }
        Backend::FillConst(T(0), trgt);                                                    // Tensor.fs:2159
        Backend::Scatter(trgt, p, src);
        return trgt;
    }
    // a.M(mask) for a mask of the tensor's full shape (Tensor.fs:3044-3052)
    Tensor M(const Tensor<bool>& mask) const {
        if (mask.Shape_() != Shape_()) throw std::invalid_argument("Shape of mask does not match the tensor shape.");
        Tensor trgt(Shape{mask.countTrue()});
        Tensor src = reshape({NElems()});
        Tensor<bool> fm = mask.flatten();
        Backend::MaskedGet(trgt, src, {&fm});
        return trgt;
    }
    void setM(const Tensor<bool>& mask, const Tensor& value) const {
        if (mask.Shape_() != Shape_()) throw std::invalid_argument("Shape of mask does not match the tensor shape.");
        auto view = Layout::tryReshape({NElems()}, layout_);
        if (!view) throw NotSupportedException("setM on a non-reshapeable view");
        Tensor<bool> fm = mask.flatten();
        Backend::MaskedSet(Relayout(*view), {&fm}, value.broadcastTo(Shape{mask.countTrue()}));
    }

    // (batched) matrix inverse (Tensor.fs:2807-2839)
    void FillInvert(const Tensor& a) const {
        if (a.NDims() < 2) throw std::invalid_argument("Need at least a matrix to invert.");
        Backend::BatchedInvert(*this, a.broadcastTo(Shape_()));
    }
    static Tensor invert(const Tensor& a) { Tensor t(a.Shape_()); t.FillInvert(a); return t; }

    // SVD and symmetric eigendecomposition (Tensor.fs:2841-2977); U is column-major, V row-major as in the reference
    struct SVDResult { Tensor U, S, V; };
    static SVDResult SVD(const Tensor& a) {
        if (a.NDims() < 2) throw std::invalid_argument("Need at least a matrix to SVD.");
        Shape batch(a.Shape_().begin(), a.Shape_().end() - 2);
        const int64_t M = a.Shape_()[a.NDims() - 2], N = a.Shape_()[a.NDims() - 1];
        Shape su = batch, ss = batch, sv = batch;
        su.push_back(M); su.push_back(M); ss.push_back(M < N ? M : N); sv.push_back(N); sv.push_back(N);
        SVDResult r{Tensor(su), Tensor(ss), Tensor(sv)};
        Backend::BatchedSVD(r.S, &r.U, &r.V, a);
        return r;
    }
    static Tensor SVDWithoutUV(const Tensor& a) {
        if (a.NDims() < 2) throw std::invalid_argument("Need at least a matrix to SVD.");
        Shape ss(a.Shape_().begin(), a.Shape_().end() - 2);
        ss.push_back(std::min(a.Shape_()[a.NDims() - 2], a.Shape_()[a.NDims() - 1]));
        Tensor s(ss);
        Backend::BatchedSVD(s, nullptr, nullptr, a);
        return s;
    }
    struct EigResult { Tensor vals, vecs; };
    static EigResult symmetricEigenDecomposition(MatrixPart part, const Tensor& a) {
        if (a.NDims() != 2 || a.Shape_()[0] != a.Shape_()[1]) throw std::invalid_argument("Require a square matrix for symmetric eigen-decomposition.");
        EigResult r{Tensor(Shape{a.Shape_()[0]}), Tensor(a.Shape_())};
        Backend::SymmetricEigenDecomposition(part, r.vals, r.vecs, a);
        return r;
    }

    // dot, dispatched by rank as Tensor.(.*) / FillDot (Tensor.fs:2714-2797)
    Tensor dot(const Tensor& b) const {
        const Tensor& a = *this;
        const int na = a.NDims(), nb = b.NDims();
        if (na == 1 && nb == 1 && a.Shape_() == b.Shape_()) { Tensor t(Shape{}); Backend::VecVecDot(t, a, b); return t; }
        if (na == 2 && nb == 1 && a.Shape_()[1] == b.Shape_()[0]) { Tensor t(Shape{a.Shape_()[0]}); Backend::MatVecDot(t, a, b); return t; }
        if (na == 2 && nb == 2 && a.Shape_()[1] == b.Shape_()[0]) { Tensor t(Shape{a.Shape_()[0], b.Shape_()[1]}); Backend::MatMatDot(t, a, b); return t; }
        if (na > 2 && na == nb && a.Shape_()[na - 1] == b.Shape_()[na - 2]) {
            Shape batch(na - 2);
            for (int d = 0; d < na - 2; d++) {
                const int64_t x = a.Shape_()[d], y = b.Shape_()[d];
                if (x != y && x != 1 && y != 1) throw std::invalid_argument("Cannot broadcast batch dimensions.");
                batch[d] = x == 1 ? y : x;
            }
            Shape sa = batch, sb = batch, st = batch;
            sa.push_back(a.Shape_()[na - 2]); sa.push_back(a.Shape_()[na - 1]);
            sb.push_back(b.Shape_()[na - 2]); sb.push_back(b.Shape_()[na - 1]);
            st.push_back(a.Shape_()[na - 2]); st.push_back(b.Shape_()[na - 1]);
            Tensor t(st);
            Backend::BatchedMatMatDot(t, a.broadcastTo(sa), b.broadcastTo(sb));
            return t;
        }
        throw std::invalid_argument("Cannot compute dot product between tensors of these shapes.");
    }

  private:
    TensorLayout layout_;
    std::shared_ptr<TensorHipStorage<T>> storage_;
};

template <class T>
inline DnhTensor desc(const Tensor<T>& t) {
    const TensorLayout& l = t.Layout_();
    if (l.NDims() > DNH_MAX_DIMS) throw NotSupportedException("the HIP backend supports at most 8 dimensions");
    DnhTensor d;
    std::memset(&d, 0, sizeof(d));
    d.base = t.Storage()->Ptr();
    d.offset = l.Offset;
    d.ndims = l.NDims();
    d.dtype = DTypeOf<T>::value;
    for (int i = 0; i < l.NDims(); i++) { d.shape[i] = l.Shape_[i]; d.stride[i] = l.Stride[i]; }
    return d;
}

}  // namespace Tensor
