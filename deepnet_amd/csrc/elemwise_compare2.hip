// The second half of dnh_compare's ops: ITensorBackend LessOrEqual, Greater, GreaterOrEqual (Tensor/Tensor/TensorBackend.fs:109-111).
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

int32_t dnh::compare_second_unit(int32_t op, int dt, const MapPlan& p, hipStream_t s) {
    switch (op) {
        case DNH_LESS_OR_EQUAL: return run_cmp<OpLe>(dt, p, s);
        case DNH_GREATER: return run_cmp<OpGt>(dt, p, s);
        case DNH_GREATER_OR_EQUAL: return run_cmp<OpGe>(dt, p, s);
    }
    return fail(DNH_ERR_INVALID_ARG, "dnh_compare: unknown op %d", op);
}
