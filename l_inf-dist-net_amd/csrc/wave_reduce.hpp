// Wave-wide reductions on DPP moves, shared by the kernels whose lanes split a reduction (the few-outputs forward
// kernels, the mean shift, the optimizer step).
#pragma once
#include <hip/hip_runtime.h>

namespace ldist {

// Wave-wide reductions with DPP moves (lane-to-lane inside the vector unit, no trip through LDS as ds_bpermute
// makes): swaps inside quads, rotations inside rows of 16, then the last lane of a row broadcast to the next row
// (row_bcast:15 into rows 1 and 3) and of the first half to the second (row_bcast:31 into rows 2 and 3).
// THE RESULT IS IN LANE 63 ONLY.  `old` is what a lane outside the row mask receives: the operation's identity.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp_move(int old, int v) {
    return __builtin_amdgcn_update_dpp(old, v, CTRL, ROW_MASK, 0xF, false);
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float old, float v) {
    return __int_as_float(dpp_move<CTRL, ROW_MASK>(__float_as_int(old), __float_as_int(v)));
}
constexpr int kDppSwap1 = 0xB1, kDppSwap2 = 0x4E, kDppRor4 = 0x124, kDppRor8 = 0x128, kDppBcast15 = 0x142,
              kDppBcast31 = 0x143;

// op(accumulator, value moved in); old: see above
#define LDIST_WAVE_REDUCE(STEP)          \
    STEP(kDppSwap1, 0xF);                \
    STEP(kDppSwap2, 0xF);                \
    STEP(kDppRor4, 0xF);                 \
    STEP(kDppRor8, 0xF);                 \
    STEP(kDppBcast15, 0xA);              \
    STEP(kDppBcast31, 0xC)

__device__ __forceinline__ float wave_max(float v) {   // lane 63
#define LDIST_STEP(C, M) v = __builtin_fmaxf(v, dpp_move<C, M>(v, v))
    LDIST_WAVE_REDUCE(LDIST_STEP);
#undef LDIST_STEP
    return v;
}

__device__ __forceinline__ float wave_sum(float v) {   // lane 63
#define LDIST_STEP(C, M) v += dpp_move<C, M>(0.f, v)
    LDIST_WAVE_REDUCE(LDIST_STEP);
#undef LDIST_STEP
    return v;
}

// Largest value and, among equal values, the lowest k (bits 0..30 of p; bit 31 rides along): lane 63.
__device__ __forceinline__ void wave_best(float& v, int& p) {
#define LDIST_STEP(C, M)                                                                          \
    do {                                                                                          \
        const float ov = dpp_move<C, M>(v, v);                                                    \
        const int op = dpp_move<C, M>(p, p);                                                      \
        const bool take = ov > v || (ov == v && (op & 0x7fffffff) < (p & 0x7fffffff));            \
        v = take ? ov : v;                                                                        \
        p = take ? op : p;                                                                        \
    } while (0)
    LDIST_WAVE_REDUCE(LDIST_STEP);
#undef LDIST_STEP
}

}  // namespace ldist
