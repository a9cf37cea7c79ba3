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

// Exact n / d for 0 <= n < 65536 by one multiply-high (d >= 1): q = (n * ceil(2^32 / d)) >> 32.
// Larger n take the plain division.
struct SmallDiv {
    unsigned d, magic;
    __host__ explicit SmallDiv(int div = 1) : d((unsigned)div), magic((unsigned)((0x100000000ULL + div - 1) / div)) {}
    __device__ __forceinline__ int div(int n) const {
        return d == 1 ? n : ((unsigned)n < 65536u ? (int)__umulhi((unsigned)n, magic) : (int)((unsigned)n / d));
    }
};

// A lane takes VEC consecutive output positions of one image plane (b, c) and writes them to all
// KH*KW rows of cols that belong to that plane: the window positions overlap, so the loads of one
// lane mostly hit the lines its previous window position fetched, and a wave's stores to one row are
// one contiguous kilobyte.  4-wide stores need L % 4 == 0.
template <int VEC>
__global__ void __launch_bounds__(256)
unfold_kernel(const float* __restrict__ img, float* __restrict__ cols, ConvGeom q, int blocks_per_plane,
              SmallDiv by_wo) {
    const int L = q.HO * q.WO;
    const long long bc = blockIdx.x / blocks_per_plane;       // b * C + c
    const int v = (blockIdx.x % blocks_per_plane) * 256 + threadIdx.x;
    if ((long long)v * VEC >= L) return;
    const float* plane = img + bc * q.H * q.W;
    int y0[VEC], x0[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++) {
        const int l = min(v * VEC + e, L - 1);
        const int h = by_wo.div(l), w = l - h * q.WO;
        y0[e] = h * q.S - q.P;
        x0[e] = w * q.S - q.P;
    }
    float* dst = cols + bc * q.KH * q.KW * L + (long long)v * VEC;
    for (int i = 0; i < q.KH; i++)
        for (int j = 0; j < q.KW; j++) {
            float out[VEC];
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                const int y = y0[e] + i * q.D, x = x0[e] + j * q.D;
                out[e] = ((unsigned)y < (unsigned)q.H && (unsigned)x < (unsigned)q.W) ? plane[y * q.W + x] : 0.f;
            }
            float* row = dst + (long long)(i * q.KW + j) * L;
            if constexpr (VEC == 4) {
                *reinterpret_cast<float4*>(row) = make_float4(out[0], out[1], out[2], out[3]);
            } else {
                row[0] = out[0];
            }
        }
}

// The common window: 3 x 3, stride 1, dilation 1, padding 1, W % 4 == 0, 16-byte aligned tensors.
// A lane takes four neighbouring pixels of one image row; per window row it needs the aligned
// float4 of those pixels and the two pixels next to it, and writes three float4 (the j = 0, 1, 2
// rows of cols): 9 loads for 9 stores instead of 36.
__global__ void __launch_bounds__(256)
unfold_3x3_kernel(const float* __restrict__ img, float* __restrict__ cols, int planes, int H, int W) {
    const int L = H * W, quads = L / 4;
    const long long id = (long long)blockIdx.x * 256 + threadIdx.x;
    if (id >= (long long)planes * quads) return;
    const long long bc = id / quads;
    const int v = (int)(id - bc * quads);
    const int l = v * 4, h = l / W, w = l - h * W;
    const float* plane = img + bc * L;
    float* dst = cols + bc * 9 * L + l;
#pragma unroll
    for (int i = 0; i < 3; i++) {
        const int y = h + i - 1;
        float4 mid = make_float4(0.f, 0.f, 0.f, 0.f);
        float left = 0.f, right = 0.f;
        if ((unsigned)y < (unsigned)H) {
            const float* r = plane + y * W + w;
            mid = *reinterpret_cast<const float4*>(r);
            if (w > 0) left = r[-1];
            if (w + 4 < W) right = r[4];
        }
        *reinterpret_cast<float4*>(dst + (long long)(i * 3 + 0) * L) = make_float4(left, mid.x, mid.y, mid.z);
        *reinterpret_cast<float4*>(dst + (long long)(i * 3 + 1) * L) = mid;
        *reinterpret_cast<float4*>(dst + (long long)(i * 3 + 2) * L) = make_float4(mid.y, mid.z, mid.w, right);
    }
}

// One lane = one image pixel: gathers the KH*KW column entries that were copied from it, sums them in double and
// rounds once (the kernel waits for memory; the result is the correctly rounded sum, in a fixed order).
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
        double s = 0.0;
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
        gimg[id] = (float)s;
    }
}

// Workgroup = (image b, group g, R consecutive image rows).  bins[c][r][x] in LDS collect what the
// output rows that can reach those image rows send there; the slab is then stored whole, zeros
// included, so the caller needs no memset.  Output rows near a slab border are scanned by two
// workgroups, each keeping only what lands in its own rows.
__global__ void __launch_bounds__(256)
inf_backward_input_folded_kernel(const float* __restrict__ grad_output, const int32_t* __restrict__ pos,
                                 float* __restrict__ grad_img, ConvGeom q, int G, int NG, int R, int row_tiles, int vec, int vec_img,
                                 SmallDiv by_khw, SmallDiv by_kw, SmallDiv by_wo) {
    extern __shared__ __align__(16) double bins[];   // doubles: their LDS atomic add retires nine times the lanes of the float one
    const int CG = q.C / G;
    const int tile = blockIdx.x % row_tiles;
    const int bg = blockIdx.x / row_tiles;          // b * G + g
    const int b = bg / G, g = bg - b * G;
    const int y0 = tile * R;
    const int rows = min(R, q.H - y0);
    const int nb = CG * rows * q.W;
    if (vec_img) {                                    // W % 4 == 0: nb is a multiple of four
        for (int e = threadIdx.x * 2; e < nb; e += 512) *reinterpret_cast<double2*>(bins + e) = make_double2(0.0, 0.0);
    } else {
        for (int e = threadIdx.x; e < nb; e += 256) bins[e] = 0.0;
    }
    __syncthreads();

    // output rows h with h*S + i*D - P in [y0, y0 + rows) for some i in [0, KH)
    const int lo_num = y0 + q.P - (q.KH - 1) * q.D;
    const int h_lo = lo_num <= 0 ? 0 : (lo_num + q.S - 1) / q.S;
    const int h_hi = min(q.HO - 1, (y0 + rows - 1 + q.P) / q.S);
    const int L = q.HO * q.WO;
    const int span = (h_hi - h_lo + 1) * q.WO;      // contiguous run of output positions per output channel
    if (span > 0) {
        const size_t obase = ((size_t)bg * NG) * L + (size_t)h_lo * q.WO;
        const int khw = q.KH * q.KW;
        auto scatter = [&](int p, float gv, int t) {
            const int k = p & 0x7fffffff;
            const int c = by_khw.div(k), r = k - c * khw;
            const int i = by_kw.div(r), j = r - i * q.KW;
            const int th = by_wo.div(t);
            const int h = h_lo + th, w = t - th * q.WO;
            const int y = h * q.S + i * q.D - q.P - y0, x = w * q.S + j * q.D - q.P;
            if ((unsigned)y < (unsigned)rows && (unsigned)x < (unsigned)q.W && c < CG)
                atomicAdd(&bins[(c * rows + y) * q.W + x], (double)(p >= 0 ? gv : -gv));
        };
        // lanes run along the positions of one output channel, channels are shared out over the waves
        if (vec) {
            // four positions per lane and two such groups in flight: one position per trip, the index first and
            // the gradient after it, left a wave waiting out two memory latencies per 256 bytes
            const int quads = span / 4;                   // WO % 4 == 0
            for (int n = threadIdx.x >> 6; n < NG; n += 4) {
                const int4* pq = reinterpret_cast<const int4*>(pos + obase + (size_t)n * L);
                const float4* gq = reinterpret_cast<const float4*>(grad_output + obase + (size_t)n * L);
                for (int t4 = threadIdx.x & 63; t4 < quads; t4 += 128) {
                    const bool second = t4 + 64 < quads;
                    const int4 p0 = pq[t4], p1 = pq[second ? t4 + 64 : t4];
                    const float4 g0 = gq[t4], g1 = gq[second ? t4 + 64 : t4];
                    scatter(p0.x, g0.x, 4 * t4); scatter(p0.y, g0.y, 4 * t4 + 1);
                    scatter(p0.z, g0.z, 4 * t4 + 2); scatter(p0.w, g0.w, 4 * t4 + 3);
                    if (second) {
                        const int u = 4 * (t4 + 64);
                        scatter(p1.x, g1.x, u); scatter(p1.y, g1.y, u + 1);
                        scatter(p1.z, g1.z, u + 2); scatter(p1.w, g1.w, u + 3);
                    }
                }
            }
        } else {
            for (int n = threadIdx.x >> 6; n < NG; n += 4)
                for (int t = threadIdx.x & 63; t < span; t += 64) {
                    const size_t o = obase + (size_t)n * L + t;
                    scatter(pos[o], grad_output[o], t);
                }
        }
    }
    __syncthreads();

    // bins[c][y][x] -> grad_img[b, g*CG + c, y0 + y, x]: rows of one channel are contiguous in memory
    const int per_c = rows * q.W;
    if (vec_img) {
        for (int e = threadIdx.x * 4; e < nb; e += 1024) {
            const int c = e / per_c, rest = e - c * per_c;
            const double2 lo = *reinterpret_cast<const double2*>(bins + e), hi = *reinterpret_cast<const double2*>(bins + e + 2);
            *reinterpret_cast<float4*>(grad_img + (((size_t)b * q.C + (size_t)g * CG + c) * q.H + y0) * q.W + rest) =
                make_float4((float)lo.x, (float)lo.y, (float)hi.x, (float)hi.y);
        }
    } else {
        for (int e = threadIdx.x; e < nb; e += 256) {
            const int c = e / per_c, rest = e - c * per_c;
            grad_img[(((size_t)b * q.C + (size_t)g * CG + c) * q.H + y0) * q.W + rest] = (float)bins[e];
        }
    }
}

static unsigned grid_for(long long items) {
    const long long blocks = (items + 255) / 256;
    return (unsigned)(blocks < 1 ? 1 : (blocks > 65536 ? 65536 : blocks));
}

hipError_t unfold(const float* img, float* cols, const ConvGeom& q, hipStream_t stream) {
    const int L = q.HO * q.WO;
    const long long planes = (long long)q.B * q.C;
    if (q.KH == 3 && q.KW == 3 && q.S == 1 && q.D == 1 && q.P == 1 && q.W % 4 == 0 && aligned16(img) &&
        aligned16(cols)) {
        const long long lanes = planes * (q.H * q.W / 4);
        hipLaunchKernelGGL(unfold_3x3_kernel, dim3((unsigned)((lanes + 255) / 256)), dim3(256), 0, stream, img, cols,
                           (int)planes, q.H, q.W);
        return hipGetLastError();
    }
    const SmallDiv by_wo(q.WO);
    if (L % 4 == 0 && aligned16(cols)) {
        const int bpp = (L / 4 + 255) / 256;
        hipLaunchKernelGGL(unfold_kernel<4>, dim3((unsigned)(planes * bpp)), dim3(256), 0, stream, img, cols, q, bpp,
                           by_wo);
    } else {
        const int bpp = (L + 255) / 256;
        hipLaunchKernelGGL(unfold_kernel<1>, dim3((unsigned)(planes * bpp)), dim3(256), 0, stream, img, cols, q, bpp,
                           by_wo);
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
    // as many image rows per workgroup as 64 KB of bins (doubles) hold (two workgroups per CU: their zeroing,
    // scanning and write-out phases overlap); a single row may take up to 128 KB
    if ((long long)CG * q.W > 16384) return hipErrorInvalidValue;          // the API layer screens this out
    int R = (int)(8192 / ((long long)CG * q.W));
    if (R < 1) R = 1;
    if (R > q.H) R = q.H;
    const int row_tiles = (q.H + R - 1) / R;
    const size_t lds = (size_t)CG * R * q.W * sizeof(double);
    static LdsRecord lds_allowed = {};
    int device = 0;
    if (hipError_t e = hipGetDevice(&device); e != hipSuccess) return e;
    if (hipError_t e = allow_lds(inf_backward_input_folded_kernel, 128 * 1024, device, lds_allowed); e != hipSuccess) return e;
    // 128-bit loads of four neighbouring positions: every run of output rows starts on a multiple of four
    const int vec = q.WO % 4 == 0 && aligned16(grad_output) && aligned16(pos);
    const int vec_img = q.W % 4 == 0 && aligned16(grad_img);   // the slab of a channel starts and ends on multiples of four
    hipLaunchKernelGGL(inf_backward_input_folded_kernel, dim3((unsigned)(q.B * G * row_tiles)), dim3(256), lds, stream,
                       grad_output, pos, grad_img, q, G, NG, R, row_tiles, vec, vec_img, SmallDiv(q.KH * q.KW), SmallDiv(q.KW),
                       SmallDiv(q.WO));
    return hipGetLastError();
}

}  // namespace ldist
