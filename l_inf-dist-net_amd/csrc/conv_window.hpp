// The 3x3 window of the convolution-shaped layer read straight from the image: what F.unfold would put in
// column k = (ci*3 + i)*3 + j of row (b, ho, wo) (the reference unfolds first, model/norm_dist.py:132):
//   img[b, g*CG + ci, ho*S + i*D - P, wo*S + j*D - P],  0 outside the image.
// Used by the p-norm kernels, whose terms cost far more than the index arithmetic of a load.
#pragma once
#include <hip/hip_runtime.h>

namespace ldist {

struct ImgWin {
    int C, CG;        // channels of the image, channels per group
    int H, W;         // image
    int HO, WO;       // output positions
    int S, P, D;      // stride, padding, dilation
};

// Row m = (b, ho, wo) of the unfolded matrix, as its window's corner in the image.
struct WinRow {
    int b, h0, w0;    // image, row and column of tap (0, 0); may lie outside the image
    __device__ __forceinline__ void set(const ImgWin& q, int m) {
        const int hw = q.HO * q.WO;
        b = m / hw;
        const int r = m - b * hw, ho = r / q.WO;
        h0 = ho * q.S - q.P;
        w0 = (r - ho * q.WO) * q.S - q.P;
    }
};

// Element offset in the image of column k of a row of group g; false when the tap lies in the padding.
__device__ __forceinline__ bool win_tap(const ImgWin& q, const WinRow& r, int g, int k, size_t& off) {
    const int ci = k / 9, t = k - ci * 9, i = t / 3, j = t - i * 3;
    const int h = r.h0 + i * q.D, w = r.w0 + j * q.D;
    off = (((size_t)r.b * q.C + g * q.CG + ci) * q.H + h) * q.W + w;
    return (unsigned)h < (unsigned)q.H && (unsigned)w < (unsigned)q.W;
}

}  // namespace ldist
