// More of dnh_binary's ops: ITensorBackend MaxElemwise, MinElemwise (Tensor/Tensor/TensorBackend.fs:103-104).
#include "map_kernels.h"
#include "ops.h"

using namespace dnh;

int32_t dnh::binary_third_unit(int32_t op, int dt, const MapPlan& p, hipStream_t s) {
    switch (op) {
        case DNH_MAX_ELEMWISE: return map_numeric<OpMax>(dt, p, s);
        case DNH_MIN_ELEMWISE: return map_numeric<OpMin>(dt, p, s);
    }
    return fail(DNH_ERR_INVALID_ARG, "dnh_binary: unknown op %d", op);
}
