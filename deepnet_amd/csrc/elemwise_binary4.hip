// More of dnh_binary's ops: ITensorBackend Multiply, Power (Tensor/Tensor/TensorBackend.fs:99, 102).
#include "map_kernels.h"
#include "ops.h"

using namespace dnh;

int32_t dnh::binary_fourth_unit(int32_t op, int dt, const MapPlan& p, hipStream_t s) {
    switch (op) {
        case DNH_MULTIPLY: return map_numeric<OpMul>(dt, p, s);
        case DNH_POWER:
            if (dt == DNH_F32) return launch_map(OpPow<float>{}, p, s);
            if (dt == DNH_F64) return launch_map(OpPow<double>{}, p, s);
            return fail(DNH_ERR_NOT_SUPPORTED, "Power is defined for single and double only, not %s", dtype_name(dt));
    }
    return fail(DNH_ERR_INVALID_ARG, "dnh_binary: unknown op %d", op);
}
