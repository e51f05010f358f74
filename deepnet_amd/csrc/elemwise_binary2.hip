// More of dnh_binary's ops: ITensorBackend Divide, Modulo (Tensor/Tensor/TensorBackend.fs:100-101).
#include "map_kernels.h"
#include "ops.h"

using namespace dnh;

int32_t dnh::binary_second_unit(int32_t op, int dt, const MapPlan& p, hipStream_t s) {
    switch (op) {
        case DNH_DIVIDE: return map_numeric<OpDiv>(dt, p, s);
        case DNH_MODULO: return map_numeric<OpMod>(dt, p, s);
    }
    return fail(DNH_ERR_INVALID_ARG, "dnh_binary: unknown op %d", op);
}
