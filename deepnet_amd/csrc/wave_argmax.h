// Largest value of a wavefront together with its row, lowest row on equal values, through DPP lane moves (VALU rate) instead
// of LDS-routed shuffles: shifts by 1, 2, 4, 8 inside each row of 16 lanes leave a row's result in its lane 15, two row
// broadcasts carry it on to lane 31 / 63.  Only lane 63 holds the result.  Combining a candidate twice is harmless (max with
// a lowest-row tie rule is idempotent), so every step runs unmasked inside the rows it targets.
#pragma once
#include <hip/hip_runtime.h>

namespace dnh {

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp_move(int v) {
    // lanes without a source lane under CTRL, or outside ROW_MASK, keep their own value
    return __builtin_amdgcn_update_dpp(v, v, CTRL, ROW_MASK, 0xF, false);
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(dpp_move<CTRL, ROW_MASK>(__float_as_int(v)));
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp_move(double v) {
    const long long b = __double_as_longlong(v);
    const int lo = dpp_move<CTRL, ROW_MASK>((int)(unsigned)(b & 0xFFFFFFFFLL));
    const int hi = dpp_move<CTRL, ROW_MASK>((int)(b >> 32));
    return __longlong_as_double(((long long)hi << 32) | (unsigned)lo);
}

template <int CTRL, int ROW_MASK, class T>
__device__ __forceinline__ void arg_max_step(T& best, int& bi) {
    const T ov = dpp_move<CTRL, ROW_MASK>(best);
    const int oi = dpp_move<CTRL, ROW_MASK>(bi);
    if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
}

// After the call lane 63 holds the wavefront's (largest value, its row).  Every lane of the wavefront must be active.
template <class T>
__device__ __forceinline__ void wave_arg_max_to_lane63(T& best, int& bi) {
    arg_max_step<0x111, 0xF>(best, bi);   // row_shr:1
    arg_max_step<0x112, 0xF>(best, bi);   // row_shr:2
    arg_max_step<0x114, 0xF>(best, bi);   // row_shr:4
    arg_max_step<0x118, 0xF>(best, bi);   // row_shr:8
    arg_max_step<0x142, 0xA>(best, bi);   // row_bcast:15 into rows 1 and 3
    arg_max_step<0x143, 0xC>(best, bi);   // row_bcast:31 into rows 2 and 3
}

// The (largest value, its row) of the first `count` <= 16 entries of two LDS arrays, in every lane: lane l fetches entry l,
// four row shifts leave the result in lane 15, which is then read by all.  Every lane of the wavefront must be active.
template <class T>
__device__ __forceinline__ void arg_max_of_entries(const T* vals, const int* rows, int count, int lane, T& best, int& bi) {
    T v = lane < count ? vals[lane & 15] : T(-2);
    int r = lane < count ? rows[lane & 15] : 0;
    arg_max_step<0x111, 0xF>(v, r);
    arg_max_step<0x112, 0xF>(v, r);
    arg_max_step<0x114, 0xF>(v, r);
    arg_max_step<0x118, 0xF>(v, r);
    bi = __builtin_amdgcn_readlane(r, 15);
    if constexpr (sizeof(T) == 4) {
        best = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 15));
    } else {
        const long long b = __double_as_longlong(v);
        const int lo = __builtin_amdgcn_readlane((int)(unsigned)(b & 0xFFFFFFFFLL), 15);
        const int hi = __builtin_amdgcn_readlane((int)(b >> 32), 15);
        best = __longlong_as_double(((long long)hi << 32) | (unsigned)lo);
    }
}

}  // namespace dnh
