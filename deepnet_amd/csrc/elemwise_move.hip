// dnh_fill_const, dnh_fill_incrementing, dnh_copy, dnh_convert:
// ITensorBackend FillConst / FillIncrementing / Copy / Convert (Tensor/Tensor/TensorBackend.fs:67-72).
#include "map_kernels.h"
#include "ops.h"

using namespace dnh;

namespace {

struct IncArgs {
    int nd;
    uint32_t shape[DNH_MAX_DIMS];
    int64_t stride[DNH_MAX_DIMS];
};

// t[pos] = start + incr * X(pos[0])  (Host/ScalarOps.fs:367-370); row-major decomposition of the linear thread index.
template <class X>
__global__ __launch_bounds__(kBlock) void fill_inc_kernel(X* t, X start, X incr, IncArgs p, uint32_t n) {
    const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    uint32_t rem = i, idx = 0;
    int64_t off = 0;
    for (int d = p.nd - 1; d >= 0; d--) {
        const uint32_t q = (d == 0) ? 0u : rem / p.shape[d];
        idx = rem - q * p.shape[d];
        rem = q;
        off += (int64_t)idx * p.stride[d];
    }
    t[off] = OpAdd<X>{}(start, OpMul<X>{}(incr, (X)idx));
}

template <class TT>
int32_t convert_to(int sdt, const MapPlan& p, hipStream_t s) {
    switch (sdt) {
        case DNH_BOOL: case DNH_U8: return launch_map(OpConvert<TT, uint8_t>{}, p, s);
        case DNH_I8: return launch_map(OpConvert<TT, int8_t>{}, p, s);
        case DNH_I16: return launch_map(OpConvert<TT, int16_t>{}, p, s);
        case DNH_U16: return launch_map(OpConvert<TT, uint16_t>{}, p, s);
        case DNH_I32: return launch_map(OpConvert<TT, int32_t>{}, p, s);
        case DNH_U32: return launch_map(OpConvert<TT, uint32_t>{}, p, s);
        case DNH_I64: return launch_map(OpConvert<TT, int64_t>{}, p, s);
        case DNH_U64: return launch_map(OpConvert<TT, uint64_t>{}, p, s);
        case DNH_F32: return launch_map(OpConvert<TT, float>{}, p, s);
        case DNH_F64: return launch_map(OpConvert<TT, double>{}, p, s);
    }
    return fail(DNH_ERR_NOT_SUPPORTED, "convert from unknown dtype");
}

int32_t convert_to_bool(int sdt, const MapPlan& p, hipStream_t s) {
    switch (sdt) {
        case DNH_BOOL: case DNH_U8: case DNH_I8: return launch_map(OpToBool<uint8_t>{}, p, s);
        case DNH_I16: case DNH_U16: return launch_map(OpToBool<uint16_t>{}, p, s);
        case DNH_I32: case DNH_U32: return launch_map(OpToBool<uint32_t>{}, p, s);
        case DNH_I64: case DNH_U64: return launch_map(OpToBool<uint64_t>{}, p, s);
        case DNH_F32: return launch_map(OpToBool<float>{}, p, s);
        case DNH_F64: return launch_map(OpToBool<double>{}, p, s);
    }
    return fail(DNH_ERR_NOT_SUPPORTED, "convert from unknown dtype");
}

}  // namespace

extern "C" int32_t dnh_fill_const(const DnhTensor* t, const void* value, void* stream) {
    DNH_TRY(ensure_init());
    if (!value) return fail(DNH_ERR_INVALID_ARG, "dnh_fill_const: null value");
    const DnhTensor* ops[1] = {t};
    MapPlan p;
    DNH_TRY(make_map_plan(&p, 1, ops, "dnh_fill_const"));
    hipStream_t s = (hipStream_t)stream;
    switch (dtype_size(t->dtype)) {
        case 1: { uint8_t v; memcpy(&v, value, 1); if (t->dtype == DNH_BOOL) v = v ? 1 : 0; return launch_map(OpFill<uint8_t>{v}, p, s); }
        case 2: { uint16_t v; memcpy(&v, value, 2); return launch_map(OpFill<uint16_t>{v}, p, s); }
        case 4: { uint32_t v; memcpy(&v, value, 4); return launch_map(OpFill<uint32_t>{v}, p, s); }
        case 8: { uint64_t v; memcpy(&v, value, 8); return launch_map(OpFill<uint64_t>{v}, p, s); }
    }
    return fail(DNH_ERR_NOT_SUPPORTED, "dnh_fill_const: unsupported element width");
}

extern "C" int32_t dnh_fill_incrementing(const DnhTensor* t, const void* start, const void* incr, void* stream) {
    DNH_TRY(ensure_init());
    DNH_TRY(check_tensor(t, "dnh_fill_incrementing"));
    if (!start || !incr) return fail(DNH_ERR_INVALID_ARG, "dnh_fill_incrementing: null value");
    if (t->ndims < 1) return fail(DNH_ERR_INVALID_ARG, "dnh_fill_incrementing: target must have at least one dimension");
    const int64_t n = nelems(t);
    if (n == 0) return DNH_OK;
    if (n > (int64_t)kMaxItems) return fail(DNH_ERR_NOT_SUPPORTED, "dnh_fill_incrementing: more than 2^32 elements");
    IncArgs p;
    p.nd = t->ndims;
    for (int d = 0; d < DNH_MAX_DIMS; d++) {
        p.shape[d] = d < t->ndims ? (uint32_t)t->shape[d] : 1;
        p.stride[d] = d < t->ndims ? t->stride[d] : 0;
    }
    hipStream_t s = (hipStream_t)stream;
    const unsigned blocks = cdiv(n, kBlock);
#define CASE(DT, X) case DT: { X s0, inc; memcpy(&s0, start, sizeof(X)); memcpy(&inc, incr, sizeof(X)); \
        hipLaunchKernelGGL(fill_inc_kernel<X>, dim3(blocks), dim3(kBlock), 0, s, (X*)elem_ptr(t), s0, inc, p, (uint32_t)n); break; }
    switch (t->dtype) {
        CASE(DNH_U8, uint8_t) CASE(DNH_I8, int8_t) CASE(DNH_I16, int16_t) CASE(DNH_U16, uint16_t) CASE(DNH_I32, int32_t) CASE(DNH_U32, uint32_t)
        CASE(DNH_I64, int64_t) CASE(DNH_U64, uint64_t) CASE(DNH_F32, float) CASE(DNH_F64, double)
        default: return fail(DNH_ERR_NOT_SUPPORTED, "dnh_fill_incrementing on %s", dtype_name(t->dtype));
    }
#undef CASE
    DNH_LAUNCH_CHECK();
    return DNH_OK;
}

extern "C" int32_t dnh_copy(const DnhTensor* t, const DnhTensor* src, void* stream) {
    DNH_TRY(ensure_init());
    const DnhTensor* ops[2] = {t, src};
    MapPlan p;
    DNH_TRY(make_map_plan(&p, 2, ops, "dnh_copy"));
    if (t->dtype != src->dtype) return fail(DNH_ERR_INVALID_ARG, "dnh_copy: dtypes differ (%s, %s)", dtype_name(t->dtype), dtype_name(src->dtype));
    hipStream_t s = (hipStream_t)stream;
    switch (dtype_size(t->dtype)) {
        case 1: return launch_map(OpIdentity<uint8_t>{}, p, s);
        case 2: return launch_map(OpIdentity<uint16_t>{}, p, s);
        case 4: return launch_map(OpIdentity<uint32_t>{}, p, s);
        case 8: return launch_map(OpIdentity<uint64_t>{}, p, s);
    }
    return fail(DNH_ERR_NOT_SUPPORTED, "dnh_copy: unsupported element width");
}

// Convert follows Expression.Convert (ScalarPrimitives.fs:50-52) = C-style numeric conversion; to/from bool follows the
// reference device kernel's static_cast (Cuda/Kernels/Elemwise.cuh:50-63): nonzero -> true, true -> 1.
extern "C" int32_t dnh_convert(const DnhTensor* t, const DnhTensor* src, void* stream) {
    DNH_TRY(ensure_init());
    const DnhTensor* ops[2] = {t, src};
    MapPlan p;
    DNH_TRY(make_map_plan(&p, 2, ops, "dnh_convert"));
    hipStream_t s = (hipStream_t)stream;
    switch (t->dtype) {
        case DNH_BOOL: return convert_to_bool(src->dtype, p, s);
        case DNH_U8: return convert_to<uint8_t>(src->dtype, p, s);
        case DNH_I8: return convert_to<int8_t>(src->dtype, p, s);
        case DNH_I16: return convert_to<int16_t>(src->dtype, p, s);
        case DNH_U16: return convert_to<uint16_t>(src->dtype, p, s);
        case DNH_I32: return convert_to<int32_t>(src->dtype, p, s);
        case DNH_U32: return convert_to<uint32_t>(src->dtype, p, s);
        case DNH_I64: return convert_to<int64_t>(src->dtype, p, s);
        case DNH_U64: return convert_to<uint64_t>(src->dtype, p, s);
        case DNH_F32: return convert_to<float>(src->dtype, p, s);
        case DNH_F64: return convert_to<double>(src->dtype, p, s);
    }
    return fail(DNH_ERR_NOT_SUPPORTED, "convert to unknown dtype");
}
