// Interval-bound forward of the L_inf distance layer on images, without the unfolded tensors (the reference
// unfolds lower and upper with F.unfold, model/norm_dist.py:144-145, and calls inf_dist_bound_forward_cuda):
//   U[b, g*NG + n, h*WO + w] = max_k max(|l_k - w_nk|, |u_k - w_nk|)
//   L[...]                   = max_k min(|l_k - w_nk|, |u_k - w_nk|) over the k where not (l_k - w_nk < 0 < u_k - w_nk), else 0
// with l_k, u_k the window pixels of the lower / upper image (0 outside the image) and k = (c*3 + i)*3 + j.
// Semantics follow the reference kernel model/inf_dist_cuda.cu:73-141 exactly as the column kernel
// (bound_forward.hip) does: a regular box (l <= u, everything finite) takes two subtractions and two v_max3_f32
// per (position, output, k); a stage that holds l > u, a NaN or an infinity anywhere is reduced with the
// reference's literal predicate.  Results equal the column path's bit for bit.
//
// Structure as the staged variant of inf_conv_forward.hip: a workgroup owns R output rows of one (image, group)
// and up to 64 outputs; four channels at a time of the lower rows, the upper rows and the weights travel through
// double-buffered LDS stages (global -> registers before a stage's arithmetic, registers -> LDS after it, one
// barrier per stage, which also carries the "irregular" vote for the next stage).  A lane owns 8 neighbouring
// positions of one output row times 4 outputs and reads the 10 pixels its positions cover in a window row with
// three (stride 2: five) aligned 128-bit reads per image.  A last stage with fewer than four channels loads zeros
// for the missing ones (lower = upper = weight = 0 is neutral).
#include "conv_image.hpp"

namespace ldist {

namespace {

using namespace convimg;

template <int S>
__global__ void __launch_bounds__(kMaxThreads, 2)
bound_conv_forward_kernel(const float* __restrict__ lower, const float* __restrict__ upper,
                          const float* __restrict__ weight, float* __restrict__ out_lower,
                          float* __restrict__ out_upper, ConvFwd a) {
    constexpr int NXR = (7 * S + 2) / 4 + 1;          // 128-bit reads per window row: pixels 0 .. 7*S + 2
    constexpr int XR = x_regs(S);
    constexpr int BNP = kBNP;
    constexpr float INF = __builtin_inff();
    extern __shared__ __align__(16) float lds[];
    float* xl = lds;                                    // 2 x [xhalf]: lower rows of the stage's channels
    float* xu = lds + a.xwords;                         // 2 x [xhalf]: upper rows
    float* wst = lds + 2 * a.xwords;                    // 2 x [kKC][kBNP]
    const int xhalf = a.xwords / 2;
    const int tid = threadIdx.x, NT = blockDim.x;

    int id = blockIdx.x;
    const int tn = id % a.tiles_n; id /= a.tiles_n;
    const int th = id % a.tiles_h; id /= a.tiles_h;
    const int g = id % a.G, b = id / a.G;
    const int h0 = th * a.R, n0 = tn * a.BN;
    const int y0 = h0 * S - a.P;
    const int NR = a.NR, WP = a.WP, K = a.K;
    const int plane = NR * WP;

    // ---- weights: global -> registers -> LDS stage, k-major ----
    const float* wgrp = weight + ((size_t)g * a.NG + n0) * K;
    const int nvalid = min(a.NG - n0, a.BN);
    float wreg[kWRegs];
    auto wload = [&](int ch) {
        const int kb = ch * kKC;
#pragma unroll
        for (int r = 0; r < kWRegs; r++) {
            const int idx = tid + r * NT;
            const int n = idx / kKC, kk = idx - n * kKC;
            const bool real = n < nvalid && kb + kk < K;
            const float v = wgrp[real ? (unsigned)(n * K + kb + kk) : 0u];
            wreg[r] = real ? v : 0.f;
        }
    };
    auto wstore = [&](float* stage) {
#pragma unroll
        for (int r = 0; r < kWRegs; r++) {
            const int idx = tid + r * NT;
            const int n = idx / kKC, kk = idx - n * kKC;
            stage[kk * BNP + n] = wreg[r];   // n <= 63 (idx < kWRegs * 256 = 36 * 64): inside the stage
        }
    };

    // ---- image rows: what a lane moves per stage is the same every time, only the channel base advances ----
    const size_t grp_off = ((size_t)b * a.G + g) * a.CG * a.H * a.W;
    const float* srcl = lower + grp_off;
    const float* srcu = upper + grp_off;
    int goff[XR];    // (channel inside the stage << 28) | element offset inside the stage's channels; -1 = padding
    float lreg[XR], ureg[XR];
#pragma unroll
    for (int r = 0; r < XR; r++) {
        const int idx = tid + r * NT;
        const int c = idx / plane, rem = idx - c * plane;
        const int row = rem / WP, col = rem - row * WP;
        const int y = y0 + row, x = col - a.P;
        const bool real = c < kCC && (unsigned)y < (unsigned)a.H && (unsigned)x < (unsigned)a.W;
        goff[r] = real ? ((c << 28) | ((c * a.H + y) * a.W + x)) : -1;
    }
    auto xload = [&](int ch) {
        const size_t base = (size_t)ch * kCC * a.H * a.W;
        const unsigned left = (unsigned)min(a.CG - ch * kCC, kCC);   // channels this stage really has (1..4)
#pragma unroll
        for (int r = 0; r < XR; r++) {
            const bool real = ((unsigned)goff[r] >> 28) < left;   // -1 reads as channel 15: never real
            const size_t off = base + (real ? (unsigned)goff[r] & 0x0fffffffu : 0u);
            const float lv = srcl[real ? off : 0], uv = srcu[real ? off : 0];
            lreg[r] = real ? lv : 0.f;
            ureg[r] = real ? uv : 0.f;
        }
    };
    auto xstore = [&](float* sl, float* su) {
#pragma unroll
        for (int r = 0; r < XR; r++) {
            sl[tid + r * NT] = lreg[r];   // < XR*NT <= xhalf
            su[tid + r * NT] = ureg[r];
        }
    };
    // true when something this lane just loaded breaks lower <= upper, or is NaN or infinite (weights included)
    auto loaded_irregular = [&]() {
        bool bad = false;
#pragma unroll
        for (int r = 0; r < XR; r++)
            bad |= !(lreg[r] <= ureg[r] && __builtin_fabsf(lreg[r]) < INF && __builtin_fabsf(ureg[r]) < INF);
#pragma unroll
        for (int r = 0; r < kWRegs; r++) bad |= !(__builtin_fabsf(wreg[r]) < INF);
        return bad;
    };
    // A workgroup too small to carry a whole stage in registers (tiny images) moves the rest directly and checks
    // it on the way; with 256 lanes these loops are empty.
    auto rest = [&](int ch, float* sl, float* su, float* sw) {
        bool bad = false;
        const size_t base = (size_t)ch * kCC * a.H * a.W;
        const int left = a.CG - ch * kCC;
        for (int idx = tid + XR * NT; idx < kCC * plane; idx += NT) {
            const int c = idx / plane, rem = idx - c * plane;
            const int row = rem / WP, col = rem - row * WP;
            const int y = y0 + row, x = col - a.P;
            const bool real = c < left && (unsigned)y < (unsigned)a.H && (unsigned)x < (unsigned)a.W;
            const size_t off = base + (size_t)(c * a.H + y) * a.W + x;
            const float lv = real ? srcl[off] : 0.f, uv = real ? srcu[off] : 0.f;
            sl[idx] = lv;
            su[idx] = uv;
            bad |= !(lv <= uv && __builtin_fabsf(lv) < INF && __builtin_fabsf(uv) < INF);
        }
        const int kb = ch * kKC;
        for (int idx = tid + kWRegs * NT; idx < kKC * a.BN; idx += NT) {
            const int n = idx / kKC, kk = idx - n * kKC;
            const bool real = n < nvalid && kb + kk < K;
            const float v = real ? wgrp[(unsigned)(n * K + kb + kk)] : 0.f;
            sw[kk * BNP + n] = v;
            bad |= !(__builtin_fabsf(v) < INF);
        }
        return bad;
    };

    wload(0);
    xload(0);
    bool bad0 = loaded_irregular();
    xstore(xl, xu);
    wstore(wst);
    bad0 |= rest(0, xl, xu, wst);
    int irregular = __syncthreads_or(bad0);

    // ---- lane geometry ----
    const int nl = tid % a.NL, ml = tid / a.NL;
    const int hr = ml / a.SEG, w0 = (ml - hr * a.SEG) * kTM;
    const int xlane_off = (hr * S) * WP + w0 * S;              // + (c*NR + i)*WP: 16-byte aligned (WP % 4 == 0)

    float lo[kTM][kTN], up[kTM][kTN];
#pragma unroll
    for (int e = 0; e < kTM; e++)
#pragma unroll
        for (int t = 0; t < kTN; t++) { lo[e][t] = 0.f; up[e][t] = 0.f; }

    struct Row { float l[NXR * 4], u[NXR * 4], w[3][kTN]; };
    const int nstage = a.CGP / kCC;
    for (int ch = 0; ch < nstage; ch++) {
        if (ch + 1 < nstage) {
            wload(ch + 1);
            xload(ch + 1);
        }
        const float* wrow = wst + (ch & 1) * kKC * BNP + kTN * nl;   // walks down the 9*kCC rows of the stage
        const float* lrow = xl + (ch & 1) * xhalf + xlane_off;       // walk down the window rows of its channels
        const float* urow = xu + (ch & 1) * xhalf + xlane_off;
        auto fetch = [&](Row& f, int r) {         // window row r of the channel the pointers stand at
#pragma unroll
            for (int q = 0; q < NXR; q++) {
                const float4 vl = *reinterpret_cast<const float4*>(lrow + r * WP + 4 * q);
                const float4 vu = *reinterpret_cast<const float4*>(urow + r * WP + 4 * q);
                f.l[4 * q] = vl.x; f.l[4 * q + 1] = vl.y; f.l[4 * q + 2] = vl.z; f.l[4 * q + 3] = vl.w;
                f.u[4 * q] = vu.x; f.u[4 * q + 1] = vu.y; f.u[4 * q + 2] = vu.z; f.u[4 * q + 3] = vu.w;
            }
#pragma unroll
            for (int j = 0; j < 3; j++) {
                const float4 w4 = *reinterpret_cast<const float4*>(wrow + (3 * r + j) * BNP);
                f.w[j][0] = w4.x; f.w[j][1] = w4.y; f.w[j][2] = w4.z; f.w[j][3] = w4.w;
            }
        };
        if (!irregular) {
            // One channel per trip (rolled: its registers are all the compiler has to keep), its three window rows
            // unrolled.  A row is 9 LDS reads for 384 arithmetic instructions, and the two bound accumulators
            // leave no room for a second row in flight: the other wave of the SIMD covers the read latency.
#pragma unroll 1
            for (int cc = 0; cc < kCC; cc++) {
#pragma unroll 1
                for (int r = 0; r < 3; r++) {
                    Row cur;
                    fetch(cur, r);
#pragma unroll
                    for (int j = 0; j < 3; j++) {
                        __builtin_amdgcn_sched_barrier(0);   // one j at a time: bounds the differences in flight
#pragma unroll
                        for (int e = 0; e < kTM; e++)
#pragma unroll
                            for (int t = 0; t < kTN; t++) {
                                const float tl = cur.l[e * S + j] - cur.w[j][t];
                                const float tu = cur.u[e * S + j] - cur.w[j][t];
                                up[e][t] = __builtin_fmaxf(__builtin_fmaxf(up[e][t], __builtin_fabsf(tl)),
                                                           __builtin_fabsf(tu));
                                lo[e][t] = __builtin_fmaxf(__builtin_fmaxf(lo[e][t], tl), -tu);
                            }
                    }
                }
                lrow += NR * WP;
                urow += NR * WP;
                wrow += 9 * BNP;
            }
        } else {
            // rare path, kept lean: one window row per trip, no prefetch, the reference's literal predicate
#pragma unroll 1
            for (int cr = 0; cr < 3 * kCC; cr++) {
                Row f;
                fetch(f, 0);
#pragma unroll
                for (int j = 0; j < 3; j++)
#pragma unroll
                    for (int e = 0; e < kTM; e++) {
                        __builtin_amdgcn_sched_barrier(0);   // four outputs at a time: this path must not cost the other registers
#pragma unroll
                        for (int t = 0; t < kTN; t++) {
                            const float tl = f.l[e * S + j] - f.w[j][t];
                            const float tu = f.u[e * S + j] - f.w[j][t];
                            const float al = __builtin_fabsf(tl), au = __builtin_fabsf(tu);
                            up[e][t] = __builtin_fmaxf(up[e][t], __builtin_fmaxf(al, au));
                            if (!(tl < 0.f && tu > 0.f)) lo[e][t] = __builtin_fmaxf(lo[e][t], __builtin_fminf(al, au));
                        }
                    }
                const bool last_row = cr % 3 == 2;              // on to the next window row, or the next channel
                lrow += last_row ? (NR - 2) * WP : WP;
                urow += last_row ? (NR - 2) * WP : WP;
                wrow += 3 * BNP;
            }
        }
        bool bad = false;
        if (ch + 1 < nstage) {
            bad = loaded_irregular();
            float* sw = wst + ((ch + 1) & 1) * kKC * BNP;
            xstore(xl + ((ch + 1) & 1) * xhalf, xu + ((ch + 1) & 1) * xhalf);
            wstore(sw);
            bad |= rest(ch + 1, xl + ((ch + 1) & 1) * xhalf, xu + ((ch + 1) & 1) * xhalf, sw);
        }
        irregular = __syncthreads_or(bad);
    }

    const int h = h0 + hr;
    if (h >= a.HO) return;
    const int L = a.HO * a.WO;
#pragma unroll
    for (int t = 0; t < kTN; t++) {
        const int n = n0 + kTN * nl + t;
        if (n >= a.NG) break;
        const size_t at = (((size_t)b * a.G + g) * a.NG + n) * L + (size_t)h * a.WO + w0;
        if (a.vec_out) {
            *reinterpret_cast<float4*>(out_lower + at) = make_float4(lo[0][t], lo[1][t], lo[2][t], lo[3][t]);
            *reinterpret_cast<float4*>(out_lower + at + 4) = make_float4(lo[4][t], lo[5][t], lo[6][t], lo[7][t]);
            *reinterpret_cast<float4*>(out_upper + at) = make_float4(up[0][t], up[1][t], up[2][t], up[3][t]);
            *reinterpret_cast<float4*>(out_upper + at + 4) = make_float4(up[4][t], up[5][t], up[6][t], up[7][t]);
        } else {
#pragma unroll
            for (int e = 0; e < kTM; e++)
                if (w0 + e < a.WO) { out_lower[at + e] = lo[e][t]; out_upper[at + e] = up[e][t]; }
        }
    }
}

}  // namespace

bool bound_conv_forward_supported(const ConvGeom& q, int G, int CO) {
    ConvFwd a{};
    return plan(q, G, CO, a, 2);
}

hipError_t bound_conv_forward(const float* lower, const float* upper, const float* weight, float* out_lower,
                              float* out_upper, const ConvGeom& q, int G, int CO, int device, hipStream_t stream) {
    ConvFwd a{};
    if (!plan(q, G, CO, a, 2)) return hipErrorInvalidValue;   // the API layer asks bound_conv_forward_supported first
    a.vec_in = 0;
    a.vec_out = q.WO % kTM == 0 && aligned16(out_lower) && aligned16(out_upper);   // every run of 8 positions whole and aligned
    const size_t lds = (2 * (size_t)a.xwords + 2 * (size_t)kKC * kBNP) * sizeof(float);
    // The dynamic-LDS limit is raised to what the largest launch so far needed, not to the whole 160 KB: the
    // workgroup-wide vote keeps a little static LDS of its own, and the two must fit together.
    static std::atomic<size_t> raised[64][2] = {};   // callers may come from several threads
    const int ki = q.S - 1;
    auto kern = q.S == 1 ? bound_conv_forward_kernel<1> : bound_conv_forward_kernel<2>;
    const int di = device >= 0 && device < 64 ? device : 0;
    if (lds > raised[di][ki].load(std::memory_order_acquire) || di != device) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)lds);
        if (e != hipSuccess) return e;
        if (di == device) {   // keep the largest: another thread may have raised it further meanwhile
            size_t seen = raised[di][ki].load(std::memory_order_relaxed);
            while (seen < lds && !raised[di][ki].compare_exchange_weak(seen, lds, std::memory_order_release)) {}
        }
    }
    const unsigned grid = (unsigned)((long long)q.B * G * a.tiles_h * a.tiles_n);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(a.ML * a.NL), lds, stream, lower, upper, weight, out_lower, out_upper, a);
    return hipGetLastError();
}

}  // namespace ldist
