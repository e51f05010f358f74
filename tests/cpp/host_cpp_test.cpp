// Test driver for the C++ host layer (deepnet_amd/cpp/hip_tensor.hpp).
//   host_cpp_test layout   — layout algebra only, needs no GPU
//   host_cpp_test gpu      — every frontend operation on the GPU, compared with the CPU oracle (liboracle's href_*) on the
//                            same seeded inputs, plus the examples of the reference's doc comments (Tensor/Tensor/Tensor.fs)
// Integer, bool and index results must match bit for bit; fp32 element-wise within 1e-6 relative; reordered fp32 sums
// within n * eps * sum|x|.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <random>
#include <string>

#include "hip_tensor.hpp"

extern "C" {
int32_t href_fill_incrementing(const DnhTensor* t, const void* start, const void* incr);
int32_t href_copy(const DnhTensor* t, const DnhTensor* a);
int32_t href_convert(const DnhTensor* t, const DnhTensor* a);
int32_t href_unary(int32_t op, const DnhTensor* t, const DnhTensor* a);
int32_t href_binary(int32_t op, const DnhTensor* t, const DnhTensor* a, const DnhTensor* b);
int32_t href_compare(int32_t op, const DnhTensor* t, const DnhTensor* a, const DnhTensor* b);
int32_t href_if_then_else(const DnhTensor* t, const DnhTensor* c, const DnhTensor* a, const DnhTensor* b);
int32_t href_reduce_last_axis(int32_t op, const DnhTensor* t, const DnhTensor* s);
int32_t href_arg_reduce_last_axis(int32_t op, const DnhTensor* t, const DnhTensor* s);
int32_t href_find_last_axis(const void* value, const DnhTensor* t, const DnhTensor* s);
int32_t href_gather(const DnhTensor* t, const DnhTensor* const* idx, int32_t n_idx, const DnhTensor* s);
int32_t href_scatter(const DnhTensor* t, const DnhTensor* const* idx, int32_t n_idx, const DnhTensor* s);
int32_t href_masked_get(const DnhTensor* t, const DnhTensor* s, const DnhTensor* const* masks, int32_t n_masks);
int32_t href_true_indices(const DnhTensor* t, const DnhTensor* s);
int32_t href_dot(const DnhTensor* t, const DnhTensor* a, const DnhTensor* b);
int32_t href_batched_invert(const DnhTensor* t, const DnhTensor* s);
}

namespace tn = Tensor;
using tn::Shape;

static int g_failed = 0, g_passed = 0;
static void report(const std::string& name, bool ok, const std::string& why = "") {
    std::printf("%s %s%s%s\n", ok ? "PASS" : "FAIL", name.c_str(), why.empty() ? "" : ": ", why.c_str());
    std::fflush(stdout);
    (ok ? g_passed : g_failed)++;
}
#define EXPECT(name, cond) report(name, (cond))
template <class E, class F>
static void expect_throws(const std::string& name, F f) {
    try { f(); report(name, false, "no exception"); }
    catch (const E&) { report(name, true); }
    catch (const std::exception& e) { report(name, false, std::string("other exception: ") + e.what()); }
}

// vector<bool> is bit-packed; host bools are kept as uint8_t 0/1, the layout the ABI uses for DNH_BOOL
template <class T> struct HostElem { using type = T; };
template <> struct HostElem<bool> { using type = uint8_t; };

// A host tensor in row-major order with a view layout, described to the oracle with the same DnhTensor struct.
template <class T>
struct HostT {
    using E = typename HostElem<T>::type;
    std::shared_ptr<std::vector<E>> data;
    tn::TensorLayout layout;
    explicit HostT(const Shape& s) : data(std::make_shared<std::vector<E>>((size_t)std::max<int64_t>(1, tn::Layout::newC(s).NElems()))), layout(tn::Layout::newC(s)) {}
    HostT(std::shared_ptr<std::vector<E>> d, tn::TensorLayout l) : data(std::move(d)), layout(std::move(l)) {}
    HostT relayout(tn::TensorLayout l) const { return HostT(data, std::move(l)); }
    DnhTensor desc() const {
        DnhTensor d;
        std::memset(&d, 0, sizeof(d));
        d.base = data->data(); d.offset = layout.Offset; d.ndims = layout.NDims(); d.dtype = tn::DTypeOf<T>::value;
        for (int i = 0; i < layout.NDims(); i++) { d.shape[i] = layout.Shape_[i]; d.stride[i] = layout.Stride[i]; }
        return d;
    }
    tn::Tensor<T> toDevice() const {                    // same storage contents and same view layout on the device
        auto st = tn::TensorHipDevice::Create<T>((int64_t)data->size());
        tn::check(dnh_memcpy_h2d(st->Ptr(), data->data(), data->size() * sizeof(E), nullptr, 1));
        return tn::Tensor<T>(layout, st);
    }
};
template <class T>
static std::vector<typename HostElem<T>::type> download(const tn::Tensor<T>& t) {
    std::vector<typename HostElem<T>::type> out((size_t)std::max<int64_t>(1, t.NElems()));
    t.toHost(reinterpret_cast<T*>(out.data()));
    out.resize((size_t)t.NElems());
    return out;
}
template <class T>
static std::vector<typename HostElem<T>::type> flat(const HostT<T>& h) {      // row-major contents of a (possibly strided) host view
    HostT<T> c(h.layout.Shape_);
    auto dc = c.desc(); auto ds = h.desc();
    href_copy(&dc, &ds);
    c.data->resize((size_t)h.layout.NElems());
    return *c.data;
}
template <class V>
static bool same(const V& a, const V& b, std::string& why) {
    if (a.size() != b.size()) { why = "size " + std::to_string(a.size()) + " vs " + std::to_string(b.size()); return false; }
    for (size_t i = 0; i < a.size(); i++)
        if (std::memcmp(&a[i], &b[i], sizeof(a[i])) != 0 && !(a[i] == b[i])) { why = "first difference at " + std::to_string(i); return false; }
    return true;
}
static bool close_rel(const std::vector<float>& a, const std::vector<float>& b, double rel, double abs_tol, std::string& why) {
    if (a.size() != b.size()) { why = "size"; return false; }
    for (size_t i = 0; i < a.size(); i++) {
        if (std::isnan(a[i]) && std::isnan(b[i])) continue;
        double d = std::fabs((double)a[i] - (double)b[i]);
        if (d > abs_tol + rel * std::fabs((double)b[i])) { why = "at " + std::to_string(i) + ": " + std::to_string(a[i]) + " vs " + std::to_string(b[i]); return false; }
    }
    return true;
}
template <class T> static void check_exact(const std::string& name, const tn::Tensor<T>& got, const HostT<T>& want) {
    std::string why; bool ok = got.Shape_() == want.layout.Shape_ && same(download(got), flat(want), why);
    report(name, ok, why);
}
static void check_close(const std::string& name, const tn::Tensor<float>& got, const HostT<float>& want, double rel, double abs_tol = 0) {
    std::string why; bool ok = got.Shape_() == want.layout.Shape_ && close_rel(download(got), flat(want), rel, abs_tol, why);
    report(name, ok, why);
}

static std::mt19937_64 g_rng(20240607);
static HostT<float> randf(const Shape& s, float lo = -2.f, float hi = 2.f) {
    HostT<float> h(s); std::uniform_real_distribution<float> d(lo, hi);
    for (auto& v : *h.data) v = d(g_rng);
    return h;
}
template <class T> static HostT<T> randi(const Shape& s, int64_t lo, int64_t hi) {
    HostT<T> h(s); std::uniform_int_distribution<int64_t> d(lo, hi);
    for (auto& v : *h.data) v = (typename HostElem<T>::type)d(g_rng);
    return h;
}

// oracle-side mirrors of the frontend steps (allocate target, broadcast, call)
template <class T> static HostT<T> o_binary(int op, HostT<T> a, HostT<T> b) {
    tn::Layout::broadcastToSame(a.layout, b.layout);
    HostT<T> t(a.layout.Shape_); auto dt = t.desc(), da = a.desc(), db = b.desc();
    if (href_binary(op, &dt, &da, &db)) std::abort();
    return t;
}
template <class T> static HostT<bool> o_compare(int op, HostT<T> a, HostT<T> b) {
    tn::Layout::broadcastToSame(a.layout, b.layout);
    HostT<bool> t(a.layout.Shape_); auto dt = t.desc(), da = a.desc(), db = b.desc();
    if (href_compare(op, &dt, &da, &db)) std::abort();
    return t;
}
template <class T> static HostT<T> o_unary(int op, const HostT<T>& a) {
    HostT<T> t(a.layout.Shape_); auto dt = t.desc(), da = a.desc();
    if (href_unary(op, &dt, &da)) std::abort();
    return t;
}
template <class T> static HostT<T> o_axis_last(const HostT<T>& a, int ax) {
    std::vector<int> p;
    for (int d = 0; d < ax; d++) p.push_back(d);
    p.push_back(a.layout.NDims() - 1);
    for (int d = ax + 1; d < a.layout.NDims(); d++) p.push_back(d - 1);
    return a.relayout(tn::Layout::permuteAxes(p, a.layout));
}
template <class R, class T> static HostT<R> o_reduce(int op, const HostT<T>& a, int ax, int kind = 0) {
    Shape s = a.layout.Shape_; s.erase(s.begin() + ax);
    HostT<R> t(s); HostT<T> v = o_axis_last(a, ax); auto dt = t.desc(), ds = v.desc();
    int32_t st = kind == 0 ? href_reduce_last_axis(op, &dt, &ds) : href_arg_reduce_last_axis(op, &dt, &ds);
    if (st) std::abort();
    return t;
}
template <class T> static HostT<T> o_dot(const HostT<T>& a, const HostT<T>& b, const Shape& ts) {
    HostT<T> t(ts); auto dt = t.desc(), da = a.desc(), db = b.desc();
    if (href_dot(&dt, &da, &db)) std::abort();
    return t;
}

// ---- layout algebra (no GPU) -----------------------------------------------------------------------------------------------
static void layout_tests() {
    using namespace tn::Layout;
    tn::TensorLayout a = newC({2, 3, 4});
    EXPECT("layout.cStride", (a.Stride == Shape{12, 4, 1}) && a.NElems() == 24);
    // permuteAxes: entry i is the destination of axis i — [2;0;1] on 2x3x4 gives 3x4x2 (Tensor.fs permuteAxes doc example uses [1;0])
    tn::TensorLayout p = permuteAxes({2, 0, 1}, a);
    EXPECT("layout.permuteAxes.destination", (p.Shape_ == Shape{3, 4, 2}) && (p.Stride == Shape{4, 1, 12}));
    EXPECT("layout.transpose", (transpose(a).Shape_ == Shape{2, 4, 3}) && (transpose(a).Stride == Shape{12, 1, 4}));
    tn::TensorLayout b = broadcastToShape({5, 2, 3, 4}, a);
    EXPECT("layout.broadcastToShape", (b.Shape_ == Shape{5, 2, 3, 4}) && (b.Stride == Shape{0, 12, 4, 1}));
    tn::TensorLayout x = newC({3, 1}), y = newC({4});
    broadcastToSame(x, y);
    EXPECT("layout.broadcastToSame", (x.Shape_ == Shape{3, 4}) && (y.Shape_ == Shape{3, 4}) && (x.Stride == Shape{1, 0}) && (y.Stride == Shape{0, 1}));
    expect_throws<std::invalid_argument>("layout.broadcast.mismatch", [] { tn::TensorLayout u = newC({3}), v = newC({4}); broadcastToSame(u, v); });
    tn::TensorLayout r = reverseAxis(1, a);
    EXPECT("layout.reverseAxis", r.Offset == 8 && (r.Stride == Shape{12, -4, 1}));
    tn::TensorLayout s = sliceDim(2, 1, 2, a);
    EXPECT("layout.slice", s.Offset == 1 && (s.Shape_ == Shape{2, 3, 2}));
    auto rs = tryReshape({6, tn::Remainder}, a);
    EXPECT("layout.reshape.remainder", rs && (rs->Shape_ == Shape{6, 4}) && (rs->Stride == Shape{4, 1}));
    EXPECT("layout.reshape.transposed.needsCopy", !tryReshape({24}, transpose(a)));
    auto ins = tryReshape({2, 1, 4, 3}, transpose(a));
    EXPECT("layout.reshape.singleton.view", ins && (ins->Stride == Shape{12, 0, 1, 4}));
    EXPECT("layout.addr", addr({1, 2, 3}, a) == 23);
    expect_throws<std::out_of_range>("layout.addr.range", [&] { addr({1, 3, 0}, a); });
    expect_throws<std::invalid_argument>("layout.permute.invalid", [&] { permuteAxes({0, 0, 1}, a); });
}

// ---- GPU: doc examples -----------------------------------------------------------------------------------------------------------
static void doc_examples() {
    using TF = tn::Tensor<float>; using TI = tn::Tensor<int64_t>; using TB = tn::Tensor<bool>;
    std::string why;
    // Tensor.fs sumAxis example: [[1;2;3;4];[5;6;7;8]] sumAxis 1 = [10; 26]
    TF a = TF::ofHost({1, 2, 3, 4, 5, 6, 7, 8}, {2, 4});
    EXPECT("doc.sumAxis", download(a.sumAxis(1)) == (std::vector<float>{10, 26}));
    EXPECT("doc.sum", a.sum() == 36.0f);
    EXPECT("doc.productAxis", download(a.productAxis(1)) == (std::vector<float>{24, 1680}));
    EXPECT("doc.maxAxis", download(a.maxAxis(1)) == (std::vector<float>{4, 8}));
    EXPECT("doc.minAxis", download(a.minAxis(1)) == (std::vector<float>{1, 5}));
    EXPECT("doc.argMaxAxis", download(a.argMaxAxis(1)) == (std::vector<int64_t>{3, 3}));
    EXPECT("doc.argMinAxis", download(a.argMinAxis(1)) == (std::vector<int64_t>{0, 0}));
    // findAxis example: [[1;2;3;4];[5;6;7;3]] findAxis 3 1 = [2; 3]
    TF f = TF::ofHost({1, 2, 3, 4, 5, 6, 7, 3}, {2, 4});
    EXPECT("doc.findAxis", download(f.findAxis(3.0f, 1)) == (std::vector<int64_t>{2, 3}));
    EXPECT("doc.findAxis.notFound", download(f.findAxis(9.0f, 1)) == (std::vector<int64_t>{tn::NotFound, tn::NotFound}));
    // arithmetic examples: [5;6;7] + [2;3;4], / , % , pow
    TF u = TF::ofHost({5, 6, 7}, {3}), v = TF::ofHost({2, 3, 4}, {3});
    EXPECT("doc.add", download(u + v) == (std::vector<float>{7, 9, 11}));
    EXPECT("doc.sub", download(u - v) == (std::vector<float>{3, 3, 3}));
    EXPECT("doc.mul", download(u * v) == (std::vector<float>{10, 18, 28}));
    EXPECT("doc.mod", download(u % v) == (std::vector<float>{1, 0, 3}));
    EXPECT("doc.pow", download(u.pow(v)) == (std::vector<float>{25, 216, 2401}));
    EXPECT("doc.greater", download(TF::ofHost({2, 3, 4}, {3}) > TF::ofHost({1, 3, 5}, {3})) == (std::vector<uint8_t>{1, 0, 0}));
    EXPECT("doc.maxElemwise", download(TF::maxElemwise(TF::ofHost({2, 3, 4}, {3}), TF::ofHost({1, 5, 3}, {3}))) == (std::vector<float>{2, 5, 4}));
    // round: ties to even
    EXPECT("doc.round.tiesToEven", download(TF::ofHost({0.5f, 1.5f, 2.5f, -0.5f, -2.7f}, {5}).round()) == (std::vector<float>{0, 2, 2, -0.0f, -3}));
    EXPECT("doc.sgn", download(TF::ofHost({-2, -0.0f, 0, 3}, {4}).sgn()) == (std::vector<float>{-1, 0, 0, 1}));
    // integer division truncates; division by zero is the backend's defined 0
    tn::Tensor<int32_t> i = tn::Tensor<int32_t>::ofHost({7, -7, 7, -7}, {4}), j = tn::Tensor<int32_t>::ofHost({2, 2, -2, -2}, {4});
    EXPECT("doc.int.divide", download(i / j) == (std::vector<int32_t>{3, -3, -3, 3}));
    EXPECT("doc.int.modulo", download(i % j) == (std::vector<int32_t>{1, -1, 1, -1}));
    // ifThenElse example: cond [true;false;false], [2;3;4], [5;6;7] = [2;6;7]
    bool cb[3] = {true, false, false};
    TB cond = TB::ofHost(cb, {3});
    EXPECT("doc.ifThenElse", download(TF::ifThenElse(cond, v, u)) == (std::vector<float>{2, 6, 7}));
    // logic
    bool pb[4] = {true, true, false, false}, qb[4] = {true, false, true, false};
    TB p = TB::ofHost(pb, {4}), q = TB::ofHost(qb, {4});
    EXPECT("doc.and", download(p & q) == (std::vector<uint8_t>{1, 0, 0, 0}));
    EXPECT("doc.or", download(p | q) == (std::vector<uint8_t>{1, 1, 1, 0}));
    EXPECT("doc.xor", download(p ^ q) == (std::vector<uint8_t>{0, 1, 1, 0}));
    EXPECT("doc.negate", download(~p) == (std::vector<uint8_t>{0, 0, 1, 1}));
    EXPECT("doc.countTrue", p.countTrue() == 2 && q.any() && !q.all());
    // trueIdx example: [[true;false;true;false];[false;false;true;true]] -> [[0;0];[0;2];[1;2];[1;3]]
    bool tb[8] = {true, false, true, false, false, false, true, true};
    EXPECT("doc.trueIdx", download(TB::ofHost(tb, {2, 4}).trueIdx()) == (std::vector<int64_t>{0, 0, 0, 2, 1, 2, 1, 3}));
    // gather example: src [[1;2;3];[4;5;6]], i0=[1;1;0;0], i1=[0;1;1;2] -> [4;5;2;3]
    TF g = TF::ofHost({1, 2, 3, 4, 5, 6}, {2, 3});
    TI i0 = TI::ofHost({1, 1, 0, 0}, {4}), i1 = TI::ofHost({0, 1, 1, 2}, {4});
    EXPECT("doc.gather", download(TF::gather({&i0, &i1}, g)) == (std::vector<float>{4, 5, 2, 3}));
    // gather with None: identity index in that dimension
    TI j1 = TI::ofHost({2, 0}, {2, 1});
    EXPECT("doc.gather.none", download(TF::gather({nullptr, &j1}, g)) == (std::vector<float>{3, 4}));
    // scatter example: src [[1;2;3];[4;5;6]], i0=[[0;0;0];[1;1;1]]... sums duplicates: all rows to row 0
    TI s0 = TI::ofHost({0, 0, 0, 0, 0, 0}, {2, 3}), s1 = TI::ofHost({0, 1, 2, 0, 1, 2}, {2, 3});
    EXPECT("doc.scatter.sum", download(TF::scatter({&s0, &s1}, {2, 3}, g)) == (std::vector<float>{5, 7, 9, 0, 0, 0}));
    expect_throws<std::out_of_range>("doc.gather.outOfRange", [&] { TI bad = TI::ofHost({0, 1, 2, 0}, {4}); TF::gather({&bad, &i1}, g); });
    // masked get/set: a.M(a > 3)
    EXPECT("doc.maskedGet", download(g.M(g > 3.0f)) == (std::vector<float>{4, 5, 6}));
    TF gs = g.Copy();
    gs.setM(g > 3.0f, TF::scalar(0.f));
    EXPECT("doc.maskedSet", download(gs) == (std::vector<float>{1, 2, 3, 0, 0, 0}));
    // dot example: [[1;2];[3;4]] .* [[5;6];[7;8]] = [[19;22];[43;50]]; matrix-vector; vector-vector
    TF m1 = TF::ofHost({1, 2, 3, 4}, {2, 2}), m2 = TF::ofHost({5, 6, 7, 8}, {2, 2});
    EXPECT("doc.dot.matmat", download(m1.dot(m2)) == (std::vector<float>{19, 22, 43, 50}));
    EXPECT("doc.dot.matvec", download(m1.dot(TF::ofHost({5, 6}, {2}))) == (std::vector<float>{17, 39}));
    EXPECT("doc.dot.vecvec", TF::ofHost({1, 2, 3}, {3}).dot(TF::ofHost({4, 5, 6}, {3})).Value() == 32.0f);
    EXPECT("doc.dot.transposed", download(m1.T_().dot(m2)) == (std::vector<float>{26, 30, 38, 44}));
    expect_throws<std::invalid_argument>("doc.dot.shapeMismatch", [&] { m1.dot(TF::ofHost({1, 2, 3}, {3})); });
    expect_throws<std::invalid_argument>("doc.broadcast.mismatch", [&] { u + TF::ofHost({1, 2}, {2}); });
    expect_throws<tn::NotSupportedException>("doc.int.log.notSupported", [&] { i.un(tn::TensorHipBackend<int32_t>::Log); });
    // invert example (Tensor.fs:2820-2825) and the singular matrix of BaseTests.fs:204-211
    {
        std::string why;
        auto inv = download(tn::Tensor<double>::invert(tn::Tensor<double>::ofHost({1, 2, 3, 4}, {2, 2})));
        std::vector<double> want{-2, 1, 1.5, -0.5};
        bool ok = true;
        for (int k = 0; k < 4; k++) ok = ok && std::fabs(inv[k] - want[k]) <= 2e-15;
        report("doc.invert", ok);
        expect_throws<tn::SingularMatrixException>("doc.invert.singular", [] { tn::Tensor<double>::invert(tn::Tensor<double>::ofHost({1, 0, 0, 1, 2, 0, 1, 0, 0}, {3, 3})); });
        expect_throws<tn::NotSupportedException>("doc.invert.int", [] { tn::Tensor<int32_t>::invert(tn::Tensor<int32_t>::ofHost({1, 0, 0, 1}, {2, 2})); });
    }
    // SVD and symmetric eigendecomposition through the C++ frontend: defining properties on small matrices
    {
        using TD = tn::Tensor<double>;
        const std::vector<double> a{4, 0, 3, -5, 1, 2};                      // 3 x 2
        auto r = TD::SVD(TD::ofHost(a, {3, 2}));
        auto U = download(r.U), S = download(r.S), V = download(r.V);
        bool ok = S.size() == 2 && S[0] >= S[1] && S[1] >= 0 && U.size() == 9 && V.size() == 4;
        for (int i = 0; i < 3 && ok; i++)
            for (int j = 0; j < 2; j++) {
                double rec = 0;
                for (int k = 0; k < 2; k++) rec += U[i * 3 + k] * S[k] * V[j * 2 + k];
                ok = ok && std::fabs(rec - a[i * 2 + j]) <= 1e-12;
            }
        for (int p = 0; p < 3 && ok; p++)
            for (int q = 0; q < 3; q++) {
                double d = 0;
                for (int i = 0; i < 3; i++) d += U[i * 3 + p] * U[i * 3 + q];
                ok = ok && std::fabs(d - (p == q ? 1.0 : 0.0)) <= 1e-12;
            }
        report("parity.svd.3x2", ok);
        auto s2 = download(TD::SVDWithoutUV(TD::ofHost(a, {3, 2})));
        report("parity.svd.valuesOnly", s2.size() == 2 && std::fabs(s2[0] - S[0]) <= 1e-12 && std::fabs(s2[1] - S[1]) <= 1e-12);
        auto e = TD::symmetricEigenDecomposition(tn::MatrixPart::Lower, TD::ofHost({2, 99, 99, -1, 2, 99, 0, -1, 2}, {3, 3}));
        auto w = download(e.vals);
        const double r2 = std::sqrt(2.0);
        report("parity.eig.tridiagonal", w.size() == 3 && std::fabs(w[0] - (2 - r2)) <= 1e-12 && std::fabs(w[1] - 2) <= 1e-12 && std::fabs(w[2] - (2 + r2)) <= 1e-12);
        expect_throws<tn::NotSupportedException>("doc.svd.int", [] { tn::Tensor<int32_t>::SVD(tn::Tensor<int32_t>::ofHost({1, 0, 0, 1}, {2, 2})); });
    }
    // counting / convert / reshape of a transposed view copies
    EXPECT("doc.counting", download(TI::counting(5)) == (std::vector<int64_t>{0, 1, 2, 3, 4}));
    EXPECT("doc.convert", download(TF::ofHost({1.7f, -1.7f, 3.0f}, {3}).convert<int32_t>()) == (std::vector<int32_t>{1, -1, 3}));
    EXPECT("doc.transpose.flatten", download(g.T_().flatten()) == (std::vector<float>{1, 4, 2, 5, 3, 6}));
    EXPECT("doc.reverseAxis", download(g.reverseAxis(1)) == (std::vector<float>{3, 2, 1, 6, 5, 4}));
    EXPECT("doc.permuteAxes", download(g.permuteAxes({1, 0})) == (std::vector<float>{1, 4, 2, 5, 3, 6}));
}

// ---- GPU vs oracle on seeded inputs ------------------------------------------------------------------------------------------------
static void oracle_parity() {
    // element-wise chain with broadcasting and a transposed operand: tanh(a * b + c) > 0
    {
        HostT<float> a = randf({257, 130}), b0 = randf({130, 257}), c = randf({130});
        HostT<float> b = b0.relayout(tn::Layout::transpose(b0.layout));
        auto ga = a.toDevice(); auto gb = b.toDevice(); auto gc = c.toDevice();
        HostT<float> oab = o_binary(DNH_MULTIPLY, a, b), osum = o_binary(DNH_ADD, oab, c), oth = o_unary(DNH_TANH, osum);
        auto gsum = ga * gb + gc;
        check_exact("parity.f32.mul_add.broadcast.transposed", gsum, osum);
        check_close("parity.f32.tanh", gsum.tanh(), oth, 1e-6, 1e-7);
        HostT<float> zero({}); (*zero.data)[0] = 0.f;
        check_exact("parity.f32.greater", gsum.tanh() > 0.f, o_compare(DNH_GREATER, o_unary(DNH_TANH, osum), zero));
        // reductions over either axis: reordered fp32 sums, bound n*eps*sum|x|
        for (int ax = 0; ax < 2; ax++) {
            auto want = o_reduce<float>(DNH_SUM, osum, ax);
            auto absum = o_reduce<float>(DNH_SUM, o_unary(DNH_ABS, osum), ax);
            auto got = download(gsum.sumAxis(ax)); auto w = flat(want); auto ab = flat(absum);
            const double n = (double)osum.layout.Shape_[ax];
            bool ok = got.size() == w.size(); std::string why;
            for (size_t k = 0; ok && k < w.size(); k++)
                if (std::fabs((double)got[k] - (double)w[k]) > n * 1.1920929e-7 * (double)ab[k]) { ok = false; why = "at " + std::to_string(k); }
            report("parity.f32.sumAxis" + std::to_string(ax), ok, why);
            check_exact("parity.f32.maxAxis" + std::to_string(ax), gsum.maxAxis(ax), o_reduce<float>(DNH_MAX, osum, ax));
            check_exact("parity.f32.argMinAxis" + std::to_string(ax), gsum.argMinAxis(ax), o_reduce<int64_t>(DNH_ARG_MIN, osum, ax, 1));
        }
    }
    // integer work is bit-exact, including wrap-around sums, ties in argMax and a reversed view
    {
        HostT<int32_t> a = randi<int32_t>({63, 5, 33}, -2000000000, 2000000000), b = randi<int32_t>({5, 1}, -7, 7);
        HostT<int32_t> ar = a.relayout(tn::Layout::reverseAxis(2, a.layout));
        auto ga = ar.toDevice(); auto gb = b.toDevice();
        check_exact("parity.i32.add.wrap", ga + gb, o_binary(DNH_ADD, ar, b));
        check_exact("parity.i32.divide", ga / gb, o_binary(DNH_DIVIDE, ar, b));
        check_exact("parity.i32.modulo", ga % gb, o_binary(DNH_MODULO, ar, b));
        for (int ax = 0; ax < 3; ax++) check_exact("parity.i32.sumAxis" + std::to_string(ax), ga.sumAxis(ax), o_reduce<int32_t>(DNH_SUM, ar, ax));
        HostT<int8_t> t = randi<int8_t>({40, 300}, -3, 3);
        auto gt = t.toDevice();
        check_exact("parity.i8.argMaxAxis.ties", gt.argMaxAxis(1), o_reduce<int64_t>(DNH_ARG_MAX, t, 1, 1));
        check_exact("parity.i8.argMaxAxis0.ties", gt.argMaxAxis(0), o_reduce<int64_t>(DNH_ARG_MAX, t, 0, 1));
        HostT<int64_t> w = randi<int64_t>({1000}, -5, 5);
        auto gw = w.toDevice();
        HostT<int64_t> fw({}); int64_t val = 3; auto dfw = fw.desc(), dw = w.desc(); href_find_last_axis(&val, &dfw, &dw);
        check_exact("parity.i64.find", gw.findAxis(3, 0), fw);
    }
    // bool reductions, compaction and index lists
    {
        HostT<bool> m = randi<bool>({64, 1000}, 0, 1);
        auto gm = m.toDevice();
        check_exact("parity.bool.countTrueAxis1", gm.countTrueAxis(1), o_reduce<int64_t>(DNH_COUNT_TRUE, m, 1));
        check_exact("parity.bool.allAxis0", gm.allAxis(0), o_reduce<bool>(DNH_ALL, m, 0));
        check_exact("parity.bool.anyAxis0", gm.anyAxis(0), o_reduce<bool>(DNH_ANY, m, 0));
        HostT<int64_t> cnt = o_reduce<int64_t>(DNH_COUNT_TRUE, m.relayout(*tn::Layout::tryReshape({64000}, m.layout)), 0);
        const int64_t n = (*cnt.data)[0];
        HostT<int64_t> ti({n, 2}); auto dti = ti.desc(), dm = m.desc(); href_true_indices(&dti, &dm);
        check_exact("parity.bool.trueIdx", gm.trueIdx(), ti);
        HostT<float> x = randf({64, 1000});
        HostT<float> xf = x.relayout(*tn::Layout::tryReshape({64000}, x.layout)); HostT<bool> mf = m.relayout(*tn::Layout::tryReshape({64000}, m.layout));
        HostT<float> sel({n}); auto dsel = sel.desc(), dxf = xf.desc(), dmf = mf.desc(); const DnhTensor* masks[1] = {&dmf};
        href_masked_get(&dsel, &dxf, masks, 1);
        check_exact("parity.f32.maskedGet", x.toDevice().M(gm), sel);
    }
    // gather (bit-exact) and scatter with duplicate targets on integers (order-independent, so bit-exact as well)
    {
        HostT<int32_t> src = randi<int32_t>({300, 70}, -1000, 1000);
        HostT<int64_t> i0 = randi<int64_t>({500, 1}, 0, 299), i1 = randi<int64_t>({1, 40}, 0, 69);
        HostT<int64_t> b0 = i0.relayout(tn::Layout::broadcastToShape({500, 40}, i0.layout)), b1 = i1.relayout(tn::Layout::broadcastToShape({500, 40}, i1.layout));
        HostT<int32_t> want({500, 40}); auto dw = want.desc(), ds = src.desc(), d0 = b0.desc(), d1 = b1.desc(); const DnhTensor* idx[2] = {&d0, &d1};
        href_gather(&dw, idx, 2, &ds);
        auto g0 = i0.toDevice(); auto g1 = i1.toDevice(); auto gsrc = src.toDevice();
        auto got = tn::Tensor<int32_t>::gather({&g0, &g1}, gsrc);
        check_exact("parity.i32.gather.broadcastIdx", got, want);
        HostT<int32_t> sw({300, 70}); auto dsw = sw.desc(); auto dwant = want.desc();
        href_scatter(&dsw, idx, 2, &dwant);
        check_exact("parity.i32.scatter.duplicates", tn::Tensor<int32_t>::scatter({&g0, &g1}, {300, 70}, got), sw);
    }
    // dot: matrix-matrix with a transposed operand, batched with a broadcast batch dimension, matrix-vector; fp32 accumulation
    // order differs from the sequential oracle: |err| <= K * eps * sum|a||b| <= K * eps * K * 4 for inputs in [-2, 2]
    {
        const int64_t M = 150, K = 200, N = 90;
        HostT<float> a0 = randf({K, M}), b = randf({K, N});
        HostT<float> a = a0.relayout(tn::Layout::transpose(a0.layout));
        check_close("parity.f32.dot.matmat.transposedA", a.toDevice().dot(b.toDevice()), o_dot(a, b, {M, N}), 0, K * 1.2e-7 * K * 4);
        HostT<float> ba = randf({3, 1, 33, 65}), bb = randf({1, 2, 65, 17});
        HostT<float> bab = ba.relayout(tn::Layout::broadcastToShape({3, 2, 33, 65}, ba.layout)), bbb = bb.relayout(tn::Layout::broadcastToShape({3, 2, 65, 17}, bb.layout));
        check_close("parity.f32.dot.batched.broadcast", ba.toDevice().dot(bb.toDevice()), o_dot(bab, bbb, {3, 2, 33, 17}), 0, 65 * 1.2e-7 * 65 * 4);
        HostT<float> v = randf({K});
        check_close("parity.f32.dot.matvec", a.toDevice().dot(v.toDevice()), o_dot(a, v, {M}), 0, K * 1.2e-7 * K * 4);
        // integer dot wraps like the host backend's multiply + sumAxis (HostBackend.fs:544-546): bit-exact
        HostT<int32_t> ia = randi<int32_t>({37, 41}, -2000000000, 2000000000), ib = randi<int32_t>({41, 29}, -2000000000, 2000000000);
        check_exact("parity.i32.dot", ia.toDevice().dot(ib.toDevice()), o_dot(ia, ib, {37, 29}));
        HostT<double> da = HostT<double>({64, 48}), db = HostT<double>({48, 80});
        for (auto& x : *da.data) x = std::uniform_real_distribution<double>(-2, 2)(g_rng);
        for (auto& x : *db.data) x = std::uniform_real_distribution<double>(-2, 2)(g_rng);
        {
            auto got = download(da.toDevice().dot(db.toDevice())); auto want = flat(o_dot(da, db, {64, 80}));
            bool ok = got.size() == want.size(); std::string why;
            for (size_t k = 0; ok && k < want.size(); k++) if (std::fabs(got[k] - want[k]) > 48 * 2.3e-16 * 48 * 4) { ok = false; why = "at " + std::to_string(k); }
            report("parity.f64.dot.matmat", ok, why);
        }
    }
    // batched inverse against the oracle's LU inverse: diagonally dominant matrices (cond < 3), |diff| <= 64 n eps max|inv|
    {
        HostT<float> a = randf({4, 70, 70}, -1.f, 1.f);
        for (int b = 0; b < 4; b++) for (int i = 0; i < 70; i++) (*a.data)[(size_t)(b * 4900 + i * 71)] += 70.f;
        HostT<float> want({4, 70, 70}); auto dw = want.desc(), da = a.desc();
        if (href_batched_invert(&dw, &da)) std::abort();
        check_close("parity.f32.invert.batched", tn::Tensor<float>::invert(a.toDevice()), want, 0, 64 * 70 * 1.2e-7 * 0.02);
    }
    // a second stream through Cfg::Stream
    {
        void* s = nullptr; tn::check(dnh_stream_create(&s));
        tn::Cfg::Stream() = s;
        HostT<float> a = randf({1000, 37}), b = randf({37});
        check_exact("parity.stream.sub", a.toDevice() - b.toDevice(), o_binary(DNH_SUBTRACT, a, b));
        tn::Cfg::Stream() = nullptr;
        tn::check(dnh_stream_destroy(s));
    }
}

int main(int argc, char** argv) {
    const std::string mode = argc > 1 ? argv[1] : "gpu";
    try {
        layout_tests();
        if (mode == "gpu") {
            tn::check(dnh_init(0));
            doc_examples();
            oracle_parity();
            tn::check(dnh_device_sync());
        }
    } catch (const std::exception& e) {
        std::printf("FAIL uncaught exception: %s\n", e.what());
        g_failed++;
    }
    std::printf("%d passed, %d failed\n", g_passed, g_failed);
    return g_failed ? 1 : 0;
}
