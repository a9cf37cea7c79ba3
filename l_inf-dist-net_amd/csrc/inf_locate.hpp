// Argmax location inside one 32-wide chunk of k, shared by the L_inf forward kernels.
#pragma once
#include "tile.hpp"

namespace ldist {

// Lowest k in [0, len) with |x[k] - w[k]| == best, as kb + k with bit 31 carrying the
// sign of the difference; 0 if none.  All 32 operand pairs are fetched before the
// first comparison so the loads overlap.  XVEC: both rows are contiguous, 16-byte
// aligned and len is a multiple of 4.
template <bool XVEC>
__device__ __forceinline__ int locate_in_chunk(const float* __restrict__ xr, int xk, const float* __restrict__ wr,
                                               int len, float best, int kb) {
    float xv[kChunk], wv[kChunk];
    if constexpr (XVEC) {
#pragma unroll
        for (int q = 0; q < kChunk / 4; q++) {
            float4 a = make_float4(0.f, 0.f, 0.f, 0.f), b = a;
            if (q * 4 < len) {
                a = reinterpret_cast<const float4*>(xr)[q];
                b = reinterpret_cast<const float4*>(wr)[q];
            }
            xv[q * 4] = a.x; xv[q * 4 + 1] = a.y; xv[q * 4 + 2] = a.z; xv[q * 4 + 3] = a.w;
            wv[q * 4] = b.x; wv[q * 4 + 1] = b.y; wv[q * 4 + 2] = b.z; wv[q * 4 + 3] = b.w;
        }
    } else {
#pragma unroll
        for (int k = 0; k < kChunk; k++) {
            xv[k] = k < len ? xr[(size_t)k * xk] : 0.f;
            wv[k] = k < len ? wr[k] : 0.f;
        }
    }
    int p = 0;
#pragma unroll
    for (int k = kChunk - 1; k >= 0; k--) {  // descending: the lowest match is written last
        const float df = xv[k] - wv[k];
        if (__builtin_fabsf(df) == best) p = (kb + k) | (__float_as_int(df) & 0x80000000);
    }
    return p;
}

}  // namespace ldist
