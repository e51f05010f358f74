// More of dnh_binary's ops: ITensorBackend MaxElemwise, MinElemwise (Tensor/Tensor/TensorBackend.fs:103-104).
#include "map_kernels.h"
#include "ops.h"

using namespace dnh;

namespace {

template <template <class> class OpT>
int32_t run_numeric(int dt, const MapPlan& p, hipStream_t s) {
    switch (dt) {
        case DNH_U8: return launch_map(OpT<uint8_t>{}, p, s);
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
    return fail(DNH_ERR_NOT_SUPPORTED, "binary arithmetic op is not defined for %s", dtype_name(dt));
}

}  // namespace

int32_t dnh::binary_third_unit(int32_t op, int dt, const MapPlan& p, hipStream_t s) {
    switch (op) {
        case DNH_MAX_ELEMWISE: return run_numeric<OpMax>(dt, p, s);
        case DNH_MIN_ELEMWISE: return run_numeric<OpMin>(dt, p, s);
    }
    return fail(DNH_ERR_INVALID_ARG, "dnh_binary: unknown op %d", op);
}
