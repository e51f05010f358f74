// dnh_unary, dnh_is_finite: ITensorBackend UnaryPlus..Truncate, Negate, IsFinite (Tensor/Tensor/TensorBackend.fs:74-95, 113).
#include "map_kernels.h"
#include "ops.h"

using namespace dnh;

namespace {

template <template <class> class OpT, class X>
int32_t run1(const MapPlan& p, hipStream_t s) { return launch_map(OpT<X>{}, p, s); }

template <template <class> class OpT>
int32_t run_fp(int dt, const MapPlan& p, hipStream_t s) {
    if (dt == DNH_F32) return run1<OpT, float>(p, s);
    if (dt == DNH_F64) return run1<OpT, double>(p, s);
    return fail(DNH_ERR_NOT_SUPPORTED, "unary op is defined for single and double only, not %s", dtype_name(dt));
}

template <template <class> class OpT>
int32_t run_signed(int dt, const MapPlan& p, hipStream_t s, bool with_i8) {
    switch (dt) {
        case DNH_I8: if (with_i8) return run1<OpT, int8_t>(p, s); break;
        case DNH_I16: return run1<OpT, int16_t>(p, s);
        case DNH_I32: return run1<OpT, int32_t>(p, s);
        case DNH_I64: return run1<OpT, int64_t>(p, s);
        case DNH_F32: return run1<OpT, float>(p, s);
        case DNH_F64: return run1<OpT, double>(p, s);
    }
    return fail(DNH_ERR_NOT_SUPPORTED, "unary op is not defined for %s", dtype_name(dt));
}

}  // namespace

extern "C" int32_t dnh_unary(int32_t op, const DnhTensor* t, const DnhTensor* a, void* stream) {
    DNH_TRY(ensure_init());
    const DnhTensor* ops[2] = {t, a};
    MapPlan p;
    DNH_TRY(make_map_plan(&p, 2, ops, "dnh_unary"));
    if (t->dtype != a->dtype) return fail(DNH_ERR_INVALID_ARG, "dnh_unary: target is %s but source is %s", dtype_name(t->dtype), dtype_name(a->dtype));
    hipStream_t s = (hipStream_t)stream;
    const int dt = t->dtype;
    if (op == DNH_NEGATE) {
        if (dt != DNH_BOOL) return fail(DNH_ERR_NOT_SUPPORTED, "Negate is defined for bool only");
        return launch_map(OpNot{}, p, s);
    }
    if (dt == DNH_BOOL) return fail(DNH_ERR_NOT_SUPPORTED, "arithmetic unary op on bool");
    switch (op) {
        case DNH_UNARY_PLUS:
            // identity on any numeric type: move by element width
            switch (dtype_size(dt)) {
                case 1: return run1<OpIdentity, uint8_t>(p, s);
                case 2: return run1<OpIdentity, uint16_t>(p, s);
                case 4: return run1<OpIdentity, uint32_t>(p, s);
                default: return run1<OpIdentity, uint64_t>(p, s);
            }
        case DNH_UNARY_MINUS: return run_signed<OpNeg>(dt, p, s, true);
        case DNH_ABS: return run_signed<OpAbs>(dt, p, s, true);
        case DNH_SGN: return run_signed<OpSgn>(dt, p, s, false);  // Sgn.fs covers int16/32/64, single, double
        case DNH_LOG: return run_fp<OpLog>(dt, p, s);
        case DNH_LOG10: return run_fp<OpLog10>(dt, p, s);
        case DNH_EXP: return run_fp<OpExp>(dt, p, s);
        case DNH_SIN: return run_fp<OpSin>(dt, p, s);
        case DNH_COS: return run_fp<OpCos>(dt, p, s);
        case DNH_TAN: return run_fp<OpTan>(dt, p, s);
        case DNH_ASIN: return run_fp<OpAsin>(dt, p, s);
        case DNH_ACOS: return run_fp<OpAcos>(dt, p, s);
        case DNH_ATAN: return run_fp<OpAtan>(dt, p, s);
        case DNH_SINH: return run_fp<OpSinh>(dt, p, s);
        case DNH_COSH: return run_fp<OpCosh>(dt, p, s);
        case DNH_TANH: return run_fp<OpTanh>(dt, p, s);
        case DNH_SQRT: return run_fp<OpSqrt>(dt, p, s);
        case DNH_CEILING: return run_fp<OpCeil>(dt, p, s);
        case DNH_FLOOR: return run_fp<OpFloor>(dt, p, s);
        case DNH_ROUND: return run_fp<OpRound>(dt, p, s);
        case DNH_TRUNCATE: return run_fp<OpTrunc>(dt, p, s);
    }
    return fail(DNH_ERR_INVALID_ARG, "dnh_unary: unknown op %d", op);
}

extern "C" int32_t dnh_is_finite(const DnhTensor* t, const DnhTensor* a, void* stream) {
    DNH_TRY(ensure_init());
    const DnhTensor* ops[2] = {t, a};
    MapPlan p;
    DNH_TRY(make_map_plan(&p, 2, ops, "dnh_is_finite"));
    if (t->dtype != DNH_BOOL) return fail(DNH_ERR_INVALID_ARG, "dnh_is_finite: target must be bool");
    hipStream_t s = (hipStream_t)stream;
    switch (a->dtype) {
        case DNH_F32: return launch_map(OpIsFinite<float>{}, p, s);
        case DNH_F64: return launch_map(OpIsFinite<double>{}, p, s);
        case DNH_BOOL: return fail(DNH_ERR_NOT_SUPPORTED, "IsFinite on bool");
        default: {
            // every integer is finite: a constant fill of the target
            const DnhTensor* only[1] = {t};
            MapPlan pf;
            DNH_TRY(make_map_plan(&pf, 1, only, "dnh_is_finite"));
            return launch_map(OpFill<uint8_t>{1}, pf, s);
        }
    }
}
