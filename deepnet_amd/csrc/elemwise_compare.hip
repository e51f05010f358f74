// dnh_compare, dnh_if_then_else: ITensorBackend Equal..GreaterOrEqual, IfThenElse (Tensor/Tensor/TensorBackend.fs:106-111, 118).
#include "map_kernels.h"
#include "ops.h"

using namespace dnh;

namespace {

template <template <class> class OpT>
int32_t run_cmp(int dt, const MapPlan& p, hipStream_t s) {
    switch (dt) {
        case DNH_BOOL: case DNH_U8: return launch_map(OpT<uint8_t>{}, p, s);
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
    return fail(DNH_ERR_NOT_SUPPORTED, "comparison on unknown dtype");
}

}  // namespace

extern "C" int32_t dnh_compare(int32_t op, const DnhTensor* t, const DnhTensor* a, const DnhTensor* b, void* stream) {
    DNH_TRY(ensure_init());
    const DnhTensor* ops[3] = {t, a, b};
    MapPlan p;
    DNH_TRY(make_map_plan(&p, 3, ops, "dnh_compare"));
    if (t->dtype != DNH_BOOL) return fail(DNH_ERR_INVALID_ARG, "dnh_compare: target must be bool");
    if (a->dtype != b->dtype) return fail(DNH_ERR_INVALID_ARG, "dnh_compare: source dtypes differ (%s, %s)", dtype_name(a->dtype), dtype_name(b->dtype));
    hipStream_t s = (hipStream_t)stream;
    switch (op) {
        case DNH_EQUAL: return run_cmp<OpEq>(a->dtype, p, s);
        case DNH_NOT_EQUAL: return run_cmp<OpNe>(a->dtype, p, s);
        case DNH_LESS: return run_cmp<OpLt>(a->dtype, p, s);
        case DNH_LESS_OR_EQUAL: case DNH_GREATER: case DNH_GREATER_OR_EQUAL: return compare_second_unit(op, a->dtype, p, s);
    }
    return fail(DNH_ERR_INVALID_ARG, "dnh_compare: unknown op %d", op);
}

extern "C" int32_t dnh_if_then_else(const DnhTensor* t, const DnhTensor* c, const DnhTensor* a, const DnhTensor* b, void* stream) {
    DNH_TRY(ensure_init());
    const DnhTensor* ops[4] = {t, c, a, b};
    MapPlan p;
    DNH_TRY(make_map_plan(&p, 4, ops, "dnh_if_then_else"));
    if (c->dtype != DNH_BOOL) return fail(DNH_ERR_INVALID_ARG, "dnh_if_then_else: condition must be bool");
    if (t->dtype != a->dtype || t->dtype != b->dtype) return fail(DNH_ERR_INVALID_ARG, "dnh_if_then_else: value dtypes differ");
    hipStream_t s = (hipStream_t)stream;
    switch (dtype_size(t->dtype)) {
        case 1: return launch_map(OpSelect<uint8_t>{}, p, s);
        case 2: return launch_map(OpSelect<uint16_t>{}, p, s);
        case 4: return launch_map(OpSelect<uint32_t>{}, p, s);
        case 8: return launch_map(OpSelect<uint64_t>{}, p, s);
    }
    return fail(DNH_ERR_NOT_SUPPORTED, "dnh_if_then_else: unsupported element width");
}
