// Element functors.  Semantics follow the reference's Host device: Tensor/Tensor/Host/ScalarOps.fs:363-581,
// Tensor/Tensor/ScalarPrimitives.fs:50-246, Tensor/Tensor/Sgn.fs:11-15.  Integer arithmetic wraps (unchecked
// expression trees); integer / and % truncate toward zero; x/0, x%0 and MinValue/-1 raise on .NET and are defined here
// as 0 so that no input can fault the device.  fp32 + - * / sqrt are correctly rounded (no contraction, no fast-math).
#pragma once

#include <hip/hip_runtime.h>

#include <limits>
#include <type_traits>

namespace dnh {

template <class X> struct UnsignedOf { using type = typename std::make_unsigned<X>::type; };
template <> struct UnsignedOf<float> { using type = float; };
template <> struct UnsignedOf<double> { using type = double; };

template <class X> constexpr bool kIsFp = std::is_floating_point<X>::value;

#define DNH_OP_HEAD1(X) using T = X; using A = X; using B = char; using C = char; static constexpr int NSRC = 1;
#define DNH_OP_HEAD2(X) using T = X; using A = X; using B = X; using C = char; static constexpr int NSRC = 2;

template <class X> struct OpIdentity { DNH_OP_HEAD1(X) __device__ X operator()(X a) const { return a; } };

template <class X> struct OpNeg {
    DNH_OP_HEAD1(X)
    __device__ X operator()(X a) const {
        if constexpr (kIsFp<X>) return -a;
        else { using U = typename UnsignedOf<X>::type; return (X)(U(0) - (U)a); }
    }
};
template <class X> struct OpAbs {
    DNH_OP_HEAD1(X)
    __device__ X operator()(X a) const {
        if constexpr (std::is_same<X, float>::value) return fabsf(a);
        else if constexpr (std::is_same<X, double>::value) return fabs(a);
        else { using U = typename UnsignedOf<X>::type; return a < 0 ? (X)(U(0) - (U)a) : a; }
    }
};
template <class X> struct OpSgn {
    DNH_OP_HEAD1(X)
    __device__ X operator()(X a) const { return a < X(0) ? X(-1) : (a > X(0) ? X(1) : X(0)); }
};

#define DNH_FP_OP(NAME, F32, F64)                                                    \
    template <class X> struct NAME {                                                 \
        DNH_OP_HEAD1(X)                                                              \
        __device__ X operator()(X a) const {                                         \
            if constexpr (std::is_same<X, float>::value) return F32(a);              \
            else return F64(a);                                                      \
        }                                                                            \
    };
DNH_FP_OP(OpLog, logf, log)
DNH_FP_OP(OpLog10, log10f, log10)
DNH_FP_OP(OpExp, expf, exp)
DNH_FP_OP(OpSin, sinf, sin)
DNH_FP_OP(OpCos, cosf, cos)
DNH_FP_OP(OpTan, tanf, tan)
DNH_FP_OP(OpAsin, asinf, asin)
DNH_FP_OP(OpAcos, acosf, acos)
DNH_FP_OP(OpAtan, atanf, atan)
DNH_FP_OP(OpSinh, sinhf, sinh)
DNH_FP_OP(OpCosh, coshf, cosh)
DNH_FP_OP(OpTanh, tanhf, tanh)
DNH_FP_OP(OpSqrt, sqrtf, sqrt)
DNH_FP_OP(OpCeil, ceilf, ceil)
DNH_FP_OP(OpFloor, floorf, floor)
DNH_FP_OP(OpRound, rintf, rint)  // ties to even, as .NET Math.Round
DNH_FP_OP(OpTrunc, truncf, trunc)

struct OpNot {
    using T = uint8_t; using A = uint8_t; using B = char; using C = char; static constexpr int NSRC = 1;
    __device__ uint8_t operator()(uint8_t a) const { return a ? 0 : 1; }
};

template <class X> struct OpAdd {
    DNH_OP_HEAD2(X)
    __device__ X operator()(X a, X b) const {
        if constexpr (kIsFp<X>) return a + b;
        else { using U = typename UnsignedOf<X>::type; return (X)((U)a + (U)b); }
    }
};
template <class X> struct OpSub {
    DNH_OP_HEAD2(X)
    __device__ X operator()(X a, X b) const {
        if constexpr (kIsFp<X>) return a - b;
        else { using U = typename UnsignedOf<X>::type; return (X)((U)a - (U)b); }
    }
};
template <class X> struct OpMul {
    DNH_OP_HEAD2(X)
    __device__ X operator()(X a, X b) const {
        if constexpr (kIsFp<X>) return a * b;
        else if constexpr (sizeof(X) < 4) return (X)((unsigned)a * (unsigned)b);
        else { using U = typename UnsignedOf<X>::type; return (X)((U)a * (U)b); }
    }
};
template <class X> struct OpDiv {
    DNH_OP_HEAD2(X)
    __device__ X operator()(X a, X b) const {
        if constexpr (kIsFp<X>) return a / b;
        else {
            bool bad = b == 0;
            // (8- and 16-bit operands are widened to 32 bits before the division, so MinValue / -1 does not overflow: it wraps when stored)
            if constexpr (std::is_signed<X>::value && sizeof(X) >= 4) bad = bad || (a == std::numeric_limits<X>::min() && b == X(-1));
            const X bb = bad ? X(1) : b;
            const X q = (X)(a / bb);   // narrow types: int arithmetic, truncated
            return bad ? X(0) : q;
        }
    }
};
template <class X> struct OpMod {
    DNH_OP_HEAD2(X)
    __device__ X operator()(X a, X b) const {
        if constexpr (std::is_same<X, float>::value) return fmodf(a, b);
        else if constexpr (std::is_same<X, double>::value) return fmod(a, b);
        else {
            bool bad = b == 0;
            // (8- and 16-bit operands are widened to 32 bits before the division, so MinValue / -1 does not overflow: it wraps when stored)
            if constexpr (std::is_signed<X>::value && sizeof(X) >= 4) bad = bad || (a == std::numeric_limits<X>::min() && b == X(-1));
            const X bb = bad ? X(1) : b;
            const X r = (X)(a % bb);
            return bad ? X(0) : r;
        }
    }
};
template <class X> struct OpPow {
    DNH_OP_HEAD2(X)
    __device__ X operator()(X a, X b) const {
        if constexpr (std::is_same<X, float>::value) return powf(a, b);
        else return pow(a, b);
    }
};
template <class X> struct OpMax { DNH_OP_HEAD2(X) __device__ X operator()(X a, X b) const { return a > b ? a : b; } };
template <class X> struct OpMin { DNH_OP_HEAD2(X) __device__ X operator()(X a, X b) const { return a < b ? a : b; } };

#define DNH_BOOL_OP(NAME, EXPR)                                                                       \
    struct NAME {                                                                                     \
        using T = uint8_t; using A = uint8_t; using B = uint8_t; using C = char; static constexpr int NSRC = 2; \
        __device__ uint8_t operator()(uint8_t a, uint8_t b) const { return (uint8_t)((EXPR) ? 1 : 0); } \
    };
DNH_BOOL_OP(OpAnd, a && b)
DNH_BOOL_OP(OpOr, a || b)
DNH_BOOL_OP(OpXor, (a != 0) != (b != 0))

#define DNH_CMP_OP(NAME, EXPR)                                                                        \
    template <class X> struct NAME {                                                                  \
        using T = uint8_t; using A = X; using B = X; using C = char; static constexpr int NSRC = 2;    \
        __device__ uint8_t operator()(X a, X b) const { return (uint8_t)((EXPR) ? 1 : 0); }            \
    };
DNH_CMP_OP(OpEq, a == b)
DNH_CMP_OP(OpNe, a != b)
DNH_CMP_OP(OpLt, a < b)
DNH_CMP_OP(OpLe, a <= b)
DNH_CMP_OP(OpGt, a > b)
DNH_CMP_OP(OpGe, a >= b)

template <class X> struct OpIsFinite {
    using T = uint8_t; using A = X; using B = char; using C = char; static constexpr int NSRC = 1;
    __device__ uint8_t operator()(X a) const {
        if constexpr (kIsFp<X>) return (uint8_t)(isfinite(a) ? 1 : 0);
        else return 1;
    }
};

// pure data movement is specialised on the element width only
template <class W> struct OpSelect {
    using T = W; using A = uint8_t; using B = W; using C = W; static constexpr int NSRC = 3;
    __device__ W operator()(uint8_t c, W a, W b) const { return c ? a : b; }
};
template <class W> struct OpFill {
    using T = W; using A = char; using B = char; using C = char; static constexpr int NSRC = 0;
    W value;
    __device__ W operator()() const { return value; }
};
// ITensorBackend.Convert is an unchecked Expression.Convert (Tensor/Tensor/ScalarPrimitives.fs:50-52).  Integer -> integer wraps,
// integer -> float rounds to nearest, float -> float rounds (overflow to infinity): the plain casts.  A float that does not fit the
// integer target is left unspecified by the CLI standard; what the reference's runtime (64-bit x86) does is restated here, since a
// plain cast saturates on this GPU:
//   -> int32 / int64: truncate toward zero; NaN and values outside the range give the minimum value (the cvtt* instructions);
//   -> int8 / uint8 / int16 / uint16: as int32, then the low 8 / 16 bits;   -> uint32: as int64, then the low 32 bits;
//   -> uint64: below 2^63 as int64 (negative values wrap), from 2^63 on (and NaN) int64(x - 2^63) + 2^63, wrapping.
template <class F> __device__ __forceinline__ int32_t fp_to_i32(F x) {
    return (x >= (F)-2147483648.0 && x < (F)2147483648.0) ? (int32_t)x : INT32_MIN;
}
template <class F> __device__ __forceinline__ int64_t fp_to_i64(F x) {
    return (x >= (F)-9223372036854775808.0 && x < (F)9223372036854775808.0) ? (int64_t)x : INT64_MIN;
}
template <class TT, class TA> struct OpConvert {
    using T = TT; using A = TA; using B = char; using C = char; static constexpr int NSRC = 1;
    __device__ TT operator()(TA a) const {
        if constexpr (kIsFp<TA> && !kIsFp<TT>) {
            if constexpr (std::is_same<TT, int32_t>::value) return fp_to_i32(a);
            else if constexpr (std::is_same<TT, int64_t>::value) return fp_to_i64(a);
            else if constexpr (sizeof(TT) <= 2) return (TT)(uint32_t)fp_to_i32(a);
            else if constexpr (std::is_same<TT, uint32_t>::value) return (uint32_t)(uint64_t)fp_to_i64(a);
            else {
                static_assert(std::is_same<TT, uint64_t>::value, "integer target");
                if (a < (TA)9223372036854775808.0) return (uint64_t)fp_to_i64(a);
                return (uint64_t)fp_to_i64(a - (TA)9223372036854775808.0) + 0x8000000000000000ull;
            }
        } else {
            return (TT)a;
        }
    }
};
template <class TA> struct OpToBool {
    using T = uint8_t; using A = TA; using B = char; using C = char; static constexpr int NSRC = 1;
    __device__ uint8_t operator()(TA a) const { return (uint8_t)(a != TA(0) ? 1 : 0); }
};

}  // namespace dnh
