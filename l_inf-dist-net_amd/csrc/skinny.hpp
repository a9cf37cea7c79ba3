// Helpers for the "few outputs per group" kernels (NG <= 16, e.g. a 10-way head): a
// workgroup of 256 lanes takes RW rows m of one group and splits k over its lanes; per
// (row, output) partial results are reduced inside each wave and then across the four
// waves through LDS.  These kernels are bound by reading x once and w from L2.
#pragma once
#include "tile.hpp"

namespace ldist {

constexpr int kSkinnyMaxNG = 16;

// Row bookkeeping shared by the skinny kernels.
template <int RW>
struct SkinnyRows {
    int g, m0;
    size_t xoff[RW], ooff[RW];
    __device__ __forceinline__ void init(const Dims& d) {
        const int row_blocks = (d.M + RW - 1) / RW;
        g = blockIdx.x / row_blocks;
        m0 = (blockIdx.x % row_blocks) * RW;
#pragma unroll
        for (int r = 0; r < RW; r++) {
            const int m = min(m0 + r, d.M - 1);  // rows past the end repeat the last one and are not written
            const int b = m / d.HW, hw = m % d.HW;
            xoff[r] = ((size_t)(b * d.G + g) * d.K) * d.HW + hw;
            ooff[r] = ((size_t)(b * d.G + g) * d.NG) * d.HW + hw;
        }
    }
};

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = __builtin_fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

inline unsigned skinny_grid(const Dims& d, int rw) { return (unsigned)((d.M + rw - 1) / rw) * d.G; }

}  // namespace ldist
