// dnh_binary: ITensorBackend Add..MinElemwise, And/Or/Xor (Tensor/Tensor/TensorBackend.fs:97-104, 114-116).
#include "map_kernels.h"
#include "ops.h"

using namespace dnh;

extern "C" int32_t dnh_binary(int32_t op, const DnhTensor* t, const DnhTensor* a, const DnhTensor* b, void* stream) {
    DNH_TRY(ensure_init());
    const DnhTensor* ops[3] = {t, a, b};
    MapPlan p;
    DNH_TRY(make_map_plan(&p, 3, ops, "dnh_binary"));
    if (t->dtype != a->dtype || t->dtype != b->dtype)
        return fail(DNH_ERR_INVALID_ARG, "dnh_binary: operand dtypes differ (%s, %s, %s)", dtype_name(t->dtype), dtype_name(a->dtype), dtype_name(b->dtype));
    hipStream_t s = (hipStream_t)stream;
    const int dt = t->dtype;
    if (op == DNH_AND || op == DNH_OR || op == DNH_XOR) {
        if (dt != DNH_BOOL) return fail(DNH_ERR_NOT_SUPPORTED, "logic op on %s", dtype_name(dt));
        if (op == DNH_AND) return launch_map(OpAnd{}, p, s);
        if (op == DNH_OR) return launch_map(OpOr{}, p, s);
        return launch_map(OpXor{}, p, s);
    }
    switch (op) {
        case DNH_ADD: return map_numeric<OpAdd>(dt, p, s);
        case DNH_SUBTRACT: return map_numeric<OpSub>(dt, p, s);
        case DNH_MULTIPLY: case DNH_POWER: return binary_fourth_unit(op, dt, p, s);
        case DNH_DIVIDE: case DNH_MODULO: return binary_second_unit(op, dt, p, s);
        case DNH_MAX_ELEMWISE: case DNH_MIN_ELEMWISE: return binary_third_unit(op, dt, p, s);
    }
    return fail(DNH_ERR_INVALID_ARG, "dnh_binary: unknown op %d", op);
}
