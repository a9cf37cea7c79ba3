// Patch extraction for the convolution-shaped distance layer, and its adjoints.  The reference
// builds the (B, C*kh*kw, L) column tensor with torch's F.unfold (model/norm_dist.py:132,144-145)
// and lets autograd fold the gradient back; both are HBM-bound copies that torch runs at about a
// quarter of what the memory system allows, and for the L_inf layer the 9x inflated gradient of
// the columns need not exist at all.
//
//   unfold:  cols[b, (c*KH + i)*KW + j, h*WO + w] = img[b, c, h*S + i*D - P, w*S + j*D - P]   (0 outside)
//   fold:    gimg[b, c, y, x] = sum over (i, j, h, w) with h*S + i*D - P = y, w*S + j*D - P = x of gcols[...]
//   inf_backward_input_folded: the L_inf scatter (reference model/inf_dist_cuda.cu:143-156) composed
//            with fold: every (b, n, h, w) sends +-grad_output to the image pixel its argmax k = (c, i, j)
//            was read from; contributions that point into the padding are dropped, as fold drops them.
#include "kernels.hpp"

namespace ldist {

// One lane = four consecutive output positions of one (b, row of cols).  4-wide stores need L % 4 == 0.
template <int VEC>
__global__ void __launch_bounds__(256)
unfold_kernel(const float* __restrict__ img, float* __restrict__ cols, ConvGeom q) {
    const int L = q.HO * q.WO;
    const int per_row = (L + VEC - 1) / VEC;
    const long long total = (long long)q.B * q.C * q.KH * q.KW * per_row;
    for (long long id = (long long)blockIdx.x * 256 + threadIdx.x; id < total; id += (long long)gridDim.x * 256) {
        const int v = (int)(id % per_row);
        const long long row = id / per_row;                 // b * (C*KH*KW) + (c*KH + i)*KW + j
        const int j = (int)(row % q.KW);
        const long long r1 = row / q.KW;
        const int i = (int)(r1 % q.KH);
        const long long bc = r1 / q.KH;                     // b * C + c
        const float* plane = img + bc * q.H * q.W;
        float out[VEC];
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            const int l = v * VEC + e;
            const int h = l / q.WO, w = l - h * q.WO;
            const int y = h * q.S + i * q.D - q.P, x = w * q.S + j * q.D - q.P;
            out[e] = (l < L && (unsigned)y < (unsigned)q.H && (unsigned)x < (unsigned)q.W) ? plane[y * q.W + x] : 0.f;
        }
        float* dst = cols + row * L + (long long)v * VEC;
        if constexpr (VEC == 4) {
            *reinterpret_cast<float4*>(dst) = make_float4(out[0], out[1], out[2], out[3]);
        } else {
            dst[0] = out[0];
        }
    }
}

// One lane = one image pixel: gathers the KH*KW column entries that were copied from it.
__global__ void __launch_bounds__(256)
fold_kernel(const float* __restrict__ gcols, float* __restrict__ gimg, ConvGeom q) {
    const int L = q.HO * q.WO;
    const long long total = (long long)q.B * q.C * q.H * q.W;
    for (long long id = (long long)blockIdx.x * 256 + threadIdx.x; id < total; id += (long long)gridDim.x * 256) {
        const int x = (int)(id % q.W);
        const long long r1 = id / q.W;
        const int y = (int)(r1 % q.H);
        const long long bc = r1 / q.H;
        const float* base = gcols + bc * q.KH * q.KW * L;
        float s = 0.f;
        for (int i = 0; i < q.KH; i++) {
            const int hy = y + q.P - i * q.D;
            if (hy < 0 || hy % q.S != 0) continue;
            const int h = hy / q.S;
            if (h >= q.HO) continue;
            for (int j = 0; j < q.KW; j++) {
                const int wx = x + q.P - j * q.D;
                if (wx < 0 || wx % q.S != 0) continue;
                const int w = wx / q.S;
                if (w >= q.WO) continue;
                s += base[(long long)(i * q.KW + j) * L + h * q.WO + w];
            }
        }
        gimg[id] = s;
    }
}

// Workgroup = (image b, group g, R consecutive image rows).  bins[c][r][x] in LDS collect what the
// output rows that can reach those image rows send there; the slab is then stored whole, zeros
// included, so the caller needs no memset.  Output rows near a slab border are scanned by two
// workgroups, each keeping only what lands in its own rows.
__global__ void __launch_bounds__(256)
inf_backward_input_folded_kernel(const float* __restrict__ grad_output, const int32_t* __restrict__ pos,
                                 float* __restrict__ grad_img, ConvGeom q, int G, int NG, int R, int row_tiles) {
    extern __shared__ float bins[];
    const int CG = q.C / G;
    const int tile = blockIdx.x % row_tiles;
    const int bg = blockIdx.x / row_tiles;          // b * G + g
    const int b = bg / G, g = bg - b * G;
    const int y0 = tile * R;
    const int rows = min(R, q.H - y0);
    const int nb = CG * rows * q.W;
    for (int e = threadIdx.x; e < nb; e += 256) bins[e] = 0.f;
    __syncthreads();

    // output rows h with h*S + i*D - P in [y0, y0 + rows) for some i in [0, KH)
    const int lo_num = y0 + q.P - (q.KH - 1) * q.D;
    const int h_lo = lo_num <= 0 ? 0 : (lo_num + q.S - 1) / q.S;
    const int h_hi = min(q.HO - 1, (y0 + rows - 1 + q.P) / q.S);
    const int L = q.HO * q.WO;
    const int span = (h_hi - h_lo + 1) * q.WO;      // contiguous run of output positions per output channel
    if (span > 0) {
        const size_t obase = ((size_t)bg * NG) * L + (size_t)h_lo * q.WO;
        const int total = NG * span;
        const int khw = q.KH * q.KW;
        for (int e = threadIdx.x; e < total; e += 256) {
            const int n = e / span, t = e - n * span;
            const size_t o = obase + (size_t)n * L + t;
            const int p = pos[o];
            const int k = p & 0x7fffffff;
            const int c = k / khw, r = k - c * khw;
            const int i = r / q.KW, j = r - i * q.KW;
            const int h = h_lo + t / q.WO, w = t % q.WO;
            const int y = h * q.S + i * q.D - q.P - y0, x = w * q.S + j * q.D - q.P;
            if ((unsigned)y < (unsigned)rows && (unsigned)x < (unsigned)q.W && c < CG) {
                const float gv = grad_output[o];
                atomicAdd(&bins[(c * rows + y) * q.W + x], p >= 0 ? gv : -gv);
            }
        }
    }
    __syncthreads();

    // bins[c][y][x] -> grad_img[b, g*CG + c, y0 + y, x]: rows of one channel are contiguous in memory
    const int per_c = rows * q.W;
    for (int e = threadIdx.x; e < nb; e += 256) {
        const int c = e / per_c, rest = e - c * per_c;
        grad_img[(((size_t)b * q.C + (size_t)g * CG + c) * q.H + y0) * q.W + rest] = bins[e];
    }
}

static unsigned grid_for(long long items) {
    const long long blocks = (items + 255) / 256;
    return (unsigned)(blocks < 1 ? 1 : (blocks > 65536 ? 65536 : blocks));
}

hipError_t unfold(const float* img, float* cols, const ConvGeom& q, hipStream_t stream) {
    const int L = q.HO * q.WO;
    const long long rows = (long long)q.B * q.C * q.KH * q.KW;
    if (L % 4 == 0 && aligned16(cols)) {
        hipLaunchKernelGGL(unfold_kernel<4>, dim3(grid_for(rows * (L / 4))), dim3(256), 0, stream, img, cols, q);
    } else {
        hipLaunchKernelGGL(unfold_kernel<1>, dim3(grid_for(rows * L)), dim3(256), 0, stream, img, cols, q);
    }
    return hipGetLastError();
}

hipError_t fold(const float* gcols, float* gimg, const ConvGeom& q, hipStream_t stream) {
    hipLaunchKernelGGL(fold_kernel, dim3(grid_for((long long)q.B * q.C * q.H * q.W)), dim3(256), 0, stream, gcols, gimg,
                       q);
    return hipGetLastError();
}

hipError_t inf_backward_input_folded(const float* grad_output, const int32_t* pos, float* grad_img, const ConvGeom& q,
                                     int G, int CO, hipStream_t stream) {
    const int CG = q.C / G, NG = CO / G;
    // as many image rows per workgroup as 64 KB of bins hold
    int R = (int)(16384 / ((long long)CG * q.W));
    if (R < 1) return hipErrorInvalidValue;          // the API layer screens this out
    if (R > q.H) R = q.H;
    const int row_tiles = (q.H + R - 1) / R;
    const size_t lds = (size_t)CG * R * q.W * sizeof(float);
    hipLaunchKernelGGL(inf_backward_input_folded_kernel, dim3((unsigned)(q.B * G * row_tiles)), dim3(256), lds, stream,
                       grad_output, pos, grad_img, q, G, NG, R, row_tiles);
    return hipGetLastError();
}

}  // namespace ldist
