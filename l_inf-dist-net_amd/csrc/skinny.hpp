// Helpers for the "few outputs per group" kernels (NG <= 16, e.g. a 10-way head): a
// workgroup of 256 lanes takes RW rows m of one group and splits k over its lanes; per
// (row, output) partial results are reduced inside each wave with DPP moves and then across
// the four waves through LDS.  These kernels are bound by reading x once and w from L2.
#pragma once
#include "tile.hpp"
#include "wave_reduce.hpp"

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

// One walk over k for the lane: f(k, x[NX][RW], w[NB]) for every k of the lane, ascending; NX input tensors of
// one shape (the point, or the lower and upper ends of a box, or all three).
// VEC (fc layout, K % 4 == 0, 16-byte aligned tensors): a lane takes four consecutive k per trip with
// 128-bit loads -- a quarter of the load instructions, in kernels that wait for memory.  Outputs past
// the group's last one repeat it (their results are never written).
template <int NX, int RW, int NB, bool VEC, class F>
__device__ __forceinline__ void skinny_sweep(const float* const (&input)[NX], const float* __restrict__ weight,
                                             const SkinnyRows<RW>& rows, const Dims& d, int nb, int tid, F&& f) {
    const int K = d.K;
    const float* wrow[NB];
#pragma unroll
    for (int j = 0; j < NB; j++) wrow[j] = weight + ((size_t)rows.g * d.NG + min(nb + j, d.NG - 1)) * K;
    if constexpr (VEC) {
        for (int k = tid * 4; k < K; k += 1024) {
            float4 xq[NX][RW], wq[NB];
#pragma unroll
            for (int q = 0; q < NX; q++)
#pragma unroll
                for (int r = 0; r < RW; r++) xq[q][r] = *reinterpret_cast<const float4*>(input[q] + rows.xoff[r] + k);
#pragma unroll
            for (int j = 0; j < NB; j++) wq[j] = *reinterpret_cast<const float4*>(wrow[j] + k);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                float xv[NX][RW], wv[NB];
#pragma unroll
                for (int q = 0; q < NX; q++)
#pragma unroll
                    for (int r = 0; r < RW; r++)
                        xv[q][r] = e == 0 ? xq[q][r].x : e == 1 ? xq[q][r].y : e == 2 ? xq[q][r].z : xq[q][r].w;
#pragma unroll
                for (int j = 0; j < NB; j++) wv[j] = e == 0 ? wq[j].x : e == 1 ? wq[j].y : e == 2 ? wq[j].z : wq[j].w;
                f(k + e, xv, wv);
            }
        }
    } else {
        const int xk = d.HW;
        for (int k = tid; k < K; k += 256) {
            float xv[NX][RW], wv[NB];
#pragma unroll
            for (int q = 0; q < NX; q++)
#pragma unroll
                for (int r = 0; r < RW; r++) xv[q][r] = input[q][rows.xoff[r] + (size_t)k * xk];
#pragma unroll
            for (int j = 0; j < NB; j++) wv[j] = wrow[j][k];
            f(k, xv, wv);
        }
    }
}

// Calls LAUNCH(NB, VEC) with the smallest NB in {4, 8, 12, 16} that holds all outputs of a group in one
// pass over k (the 10-way head: 12).  vec: see skinny_sweep.
#define LDIST_SKINNY_DISPATCH(ng, vec, LAUNCH)                                     \
    do {                                                                           \
        if ((ng) <= 4) { if (vec) LAUNCH(4, true); else LAUNCH(4, false); }        \
        else if ((ng) <= 8) { if (vec) LAUNCH(8, true); else LAUNCH(8, false); }   \
        else if ((ng) <= 12) { if (vec) LAUNCH(12, true); else LAUNCH(12, false); } \
        else { if (vec) LAUNCH(16, true); else LAUNCH(16, false); }                \
    } while (0)

inline unsigned skinny_grid(const Dims& d, int rw) { return (unsigned)((d.M + rw - 1) / rw) * d.G; }

}  // namespace ldist
