// The general p-norm backward kernel (any p > 1, either gradient, every layout) and its launcher, shared by the
// column entry points (norm_backward.hip) and those that read the image of a convolution-shaped layer (norm_conv.hip).
#pragma once
#include "conv_window.hpp"
#include "kernels.hpp"
#include "pow.hpp"

namespace ldist {


struct NbDims {
    int B, G, K, NG, HW, M;
};

constexpr int RB = 32;  // stage depth (rows of the reduction per LDS panel)

// Exponents from which the kernels test whether a row of terms can matter before raising them to the power.
// Below, so many terms matter (normalised differences above 2^(-36/p)) that the test only costs.
constexpr float kBackwardSparseMinP = 64.f;

// WEIGHT = false: grad_input.  WEIGHT = true: grad_weight.  IMG: x is the image of a convolution-shaped layer
// (3x3 window) and row m, column k of the unfolded input is looked up in it; out and grad_output keep the conv layout.
template <bool WEIGHT, bool CONV, bool IMG>
struct Views {
    const float* x; const float* w; const float* out; const float* go;
    NbDims d; int g; ImgWin win;
    // rows of P: a in [0, A); reduction: r in [0, R)
    __device__ __forceinline__ int A() const { return WEIGHT ? d.NG : d.M; }
    // address of x[m][k], w[n][k], and of the (m,n) element of out / grad_output
    // IMG: false when the element lies in the padding (it reads as 0 and takes no gradient)
    __device__ __forceinline__ bool x_tap(int m, int k, size_t& off) const {
        WinRow r;
        r.set(win, m);
        return win_tap(win, r, g, k, off);
    }
    __device__ __forceinline__ size_t x_at(int m, int k) const {
        if (CONV) { const int b = m / d.HW, hw = m - b * d.HW; return ((size_t)(b * d.G + g) * d.K + k) * d.HW + hw; }
        return ((size_t)m * d.G + g) * d.K + k;
    }
    __device__ __forceinline__ size_t w_at(int n, int k) const { return ((size_t)g * d.NG + n) * d.K + k; }
    __device__ __forceinline__ size_t o_at(int m, int n) const {
        if (CONV) { const int b = m / d.HW, hw = m - b * d.HW; return ((size_t)(b * d.G + g) * d.NG + n) * d.HW + hw; }
        return ((size_t)m * d.G + g) * d.NG + n;
    }
};

// BA = rows of P per workgroup (64, or 32 when 64 would leave the device short of
// workgroups), BKO = its columns (64, or 128 when P has so few rows that a 32-row tile is all there
// is: the wider tile restores sixteen terms per lane and step); a lane owns BA/16 rows x BKO/16 columns.
// IMG, grad_input: the sums are added onto the image gradient (a pixel collects up to nine columns, from several
// workgroups), which the caller zero-fills.
template <bool WEIGHT, bool CONV, bool SPLIT, int BA, int BKO, bool IMG>
__global__ void __launch_bounds__(256)
norm_backward_kernel(const float* __restrict__ grad_output, const float* __restrict__ input,
                     const float* __restrict__ weight, const float* __restrict__ output, float* __restrict__ grad,
                     float p, NbDims d, int tiles_a, int tiles_k, int r_per_wg, ImgWin win) {
    static_assert(!IMG || CONV, "an image has positions");
    constexpr int LDP = BKO + 1, LDA = BA + 1;   // padded LDS rows
    constexpr int CK = BKO / 16;                 // columns per lane
    __shared__ float Os[RB * LDP];  // O[r][k]
    __shared__ float Cs[RB * LDA];  // c[r][a]     = grad_output
    __shared__ float Rs[RB * LDA];  // rinv[r][a]  = 1 / output
    __shared__ float Fs[RB * LDA];  // c * rinv^(p-1) for the small integer exponents, limits for the large ones (see below)
    const int tid = threadIdx.x;
    const int ta = blockIdx.x % tiles_a;
    const int rest = blockIdx.x / tiles_a;
    const int tk = rest % tiles_k;
    const int g = rest / tiles_k;
    const int a0 = ta * BA, k0 = tk * BKO;
    const Views<WEIGHT, CONV, IMG> v{input, weight, output, grad_output, d, g, win};
    const int A = v.A();
    const int R = WEIGHT ? d.M : d.NG;
    const int r_begin = blockIdx.y * r_per_wg;
    const int r_end = min(R, r_begin + r_per_wg);
    constexpr int PA = BA / 16;              // rows per lane
    const int tx = tid & 15, ty = tid >> 4;  // lane's patch: rows a0 + ty*PA.., columns k0 + tx, k0 + tx + 16, ...
    const float e = p - 1.0f;
    const int ie = small_int_power(e);
    // every (a, r) pair has its own largest term among its K differences, and a row of the test holds 256 of them
    // per wave: with a short K most rows hold one and the tests only cost
    const bool sparse = p >= kBackwardSparseMinP && d.K >= 1024;
    const float cut = __builtin_exp2f(-36.0f / e);   // |u| <= cut  =>  |u|^(p-1) <= 2^-36

    float q[PA][CK], acc[PA][CK];
#pragma unroll
    for (int i = 0; i < PA; i++)
#pragma unroll
        for (int j = 0; j < CK; j++) {
            const int a = a0 + ty * PA + i, k = k0 + tx + 16 * j;
            acc[i][j] = 0.f;
            if constexpr (IMG && !WEIGHT) {
                size_t off;
                q[i][j] = (a < A && k < d.K && v.x_tap(a, k, off)) ? input[off] : 0.f;
            } else {
                q[i][j] = (a < A && k < d.K) ? (WEIGHT ? weight[v.w_at(a, k)] : input[v.x_at(a, k)]) : 0.f;
            }
        }

    // In memory the k axis is contiguous for w (always) and for x when HW == 1;
    // the a/r axes of out and grad_output are contiguous along n when HW == 1 and
    // along m (= hw) otherwise.  Lanes follow the contiguous axis of each panel.
    constexpr bool O_K_CONTIG = !(WEIGHT && CONV);         // O = w, or x in the fc layout
    constexpr bool C_A_CONTIG = WEIGHT ? !CONV : CONV;     // is `a` the contiguous axis of out/grad_output
    // grad_weight in the conv layout: every panel element this lane loads belongs to row m = r0 + (tid & 31)
    // of the reduction, so its image b and position hw are kept up to date from stage to stage instead of
    // being divided out per element
    constexpr bool ROW_PER_LANE = WEIGHT && CONV;
    int mb = 0, mhw = 0;
    if constexpr (ROW_PER_LANE) {
        const int m = r_begin + (tid & (RB - 1));
        mb = m / d.HW;
        mhw = m - mb * d.HW;
    }
    for (int r0 = r_begin; r0 < r_end; r0 += RB) {
        __syncthreads();
        bool unsafe = !(ie == 1 || ie == 2 || ie == 3 || ie == 7);
        const size_t xrow = ((size_t)(mb * d.G + g) * d.K) * d.HW + mhw;    // ROW_PER_LANE: x[m][0]
        WinRow wrow;                                                         // ROW_PER_LANE, IMG: the window of row m
        if constexpr (IMG && ROW_PER_LANE) {
            const int ho = mhw / win.WO;
            wrow.b = mb;
            wrow.h0 = ho * win.S - win.P;
            wrow.w0 = (mhw - ho * win.WO) * win.S - win.P;
        }
        const size_t orow = ((size_t)(mb * d.G + g) * d.NG) * d.HW + mhw;   // ROW_PER_LANE: out[m][0]
#pragma unroll
        for (int it = 0; it < RB * BKO / 256; it++) {
            const int id = tid + it * 256;
            const int rr = O_K_CONTIG ? id / BKO : id & (RB - 1);
            const int cc = O_K_CONTIG ? id % BKO : id / RB;
            const int r = r0 + rr, k = k0 + cc;
            float val = 0.f;
            if constexpr (IMG && ROW_PER_LANE) {
                size_t off;
                if (r < r_end && k < d.K && win_tap(win, wrow, g, k, off)) val = input[off];
            } else if (r < r_end && k < d.K)
                val = ROW_PER_LANE ? input[xrow + (size_t)k * d.HW] : (WEIGHT ? input[v.x_at(r, k)] : weight[v.w_at(r, k)]);
            Os[rr * LDP + cc] = val;
        }
#pragma unroll
        for (int it = 0; it < RB * BA / 256; it++) {
            const int id = tid + it * 256;
            {
                const int rr = C_A_CONTIG ? id / BA : id & (RB - 1);
                const int cc = C_A_CONTIG ? id % BA : id / RB;
                const int r = r0 + rr, a = a0 + cc;
                float c = 0.f, ri = 0.f, lim = 3.0e38f;   // padding never passes the test of the sparse sweep
                if (r < r_end && a < A) {
                    const size_t o = ROW_PER_LANE ? orow + (size_t)a * d.HW : (WEIGHT ? v.o_at(r, a) : v.o_at(a, r));
                    c = grad_output[o];
                    const float out = output[o];
                    ri = __builtin_amdgcn_rcpf(out);
                    // the factored form below needs rinv^(p-1) and (Q-O)^(p-1) well inside the float range
                    unsafe |= !(out >= 0x1p-12f && out <= 0x1p12f);
                    lim = cut * out;
                }
                const float r2 = ri * ri, r3 = r2 * ri;
                Cs[rr * LDA + cc] = c;
                Rs[rr * LDA + cc] = ri;
                Fs[rr * LDA + cc] = sparse ? lim : c * (ie == 1 ? ri : ie == 2 ? r2 : ie == 3 ? r3 : r3 * r3 * ri);
            }
        }
        if constexpr (ROW_PER_LANE) {
            mhw += RB;
            while (mhw >= d.HW) { mhw -= d.HW; mb++; }
        }
        // With p - 1 = 1, 2, 3 or 7 and every output of the stage within [2^-12, 2^12], the term
        // c * ((Q-O) * rinv)^(p-1) is taken as (c * rinv^(p-1)) * (Q-O)^(p-1): the first factor is per (a, r) and
        // sits in LDS, which saves the multiplication by rinv per term (6 instead of 7 instructions at p = 8) and
        // one LDS read per row and step.  |Q-O| <= output up to rounding, so (Q-O)^7 stays below 2^84, and where it
        // underflows the normalised difference is below 2^-6 and its seventh power below the tolerance.
        const bool factored = !__syncthreads_or(unsafe);
        auto reduce_factored = [&](auto spower) {
#pragma unroll 2
            for (int rr = 0; rr < RB; rr++) {
                float o[CK], f[PA];
#pragma unroll
                for (int j = 0; j < CK; j++) o[j] = Os[rr * LDP + tx + 16 * j];
#pragma unroll
                for (int i = 0; i < PA; i++) f[i] = Fs[rr * LDA + ty * PA + i];
#pragma unroll
                for (int i = 0; i < PA; i++)
#pragma unroll
                    for (int j = 0; j < CK; j++) acc[i][j] += f[i] * spower(q[i][j] - o[j]);
            }
        };
        // spower(u) = sign(u) * |u|^(p-1) for the signed, normalised difference u = (Q - O) * rinv.
        // Odd integer exponents keep the sign by themselves, even ones take one factor as |u|.
        auto reduce = [&](auto spower) {
#pragma unroll 2
            for (int rr = 0; rr < RB; rr++) {
                float o[CK], c[PA], ri[PA];
#pragma unroll
                for (int j = 0; j < CK; j++) o[j] = Os[rr * LDP + tx + 16 * j];   // neighbouring lanes, neighbouring banks
#pragma unroll
                for (int i = 0; i < PA; i++) { c[i] = Cs[rr * LDA + ty * PA + i]; ri[i] = Rs[rr * LDA + ty * PA + i]; }
#pragma unroll
                for (int i = 0; i < PA; i++)
#pragma unroll
                    for (int j = 0; j < CK; j++) acc[i][j] += c[i] * spower((q[i][j] - o[j]) * ri[i]);
            }
        };
        // Large exponents: a normalised difference |u| <= 1 with |u|^(p-1) below 2^-36 adds less to a sum than the
        // rounding of one term of unit size, and nearly all differences are that small -- while the logarithm and the
        // exponential are most of a term's cost.  One row of the lane's patch at a time (CK terms that share c and
        // rinv): when no lane of the wave has |Q - O| above its limit 2^(-36/(p-1)) * output (the Fs panel), the
        // wave passes over the row.  The four tests of a step are made before the first branch, so that the
        // branches wait for scalar registers only.
        auto reduce_sparse = [&]() {
#pragma unroll 2
            for (int rr = 0; rr < RB; rr++) {
                float o[CK], lim[PA], df[PA][CK];
#pragma unroll
                for (int j = 0; j < CK; j++) o[j] = Os[rr * LDP + tx + 16 * j];
#pragma unroll
                for (int i = 0; i < PA; i++) lim[i] = Fs[rr * LDA + ty * PA + i];
                unsigned long long hot[PA], any = 0;
#pragma unroll
                for (int i = 0; i < PA; i++) {
                    float top = 0.f;
#pragma unroll
                    for (int j = 0; j < CK; j++) {
                        df[i][j] = q[i][j] - o[j];
                        top = __builtin_fmaxf(top, __builtin_fabsf(df[i][j]));
                    }
                    hot[i] = __builtin_amdgcn_ballot_w64(top > lim[i]);
                    any |= hot[i];
                }
                if (any == 0) continue;
#pragma unroll
                for (int i = 0; i < PA; i++) {
                    if (hot[i] == 0) continue;
                    const float c = Cs[rr * LDA + ty * PA + i], ri = Rs[rr * LDA + ty * PA + i];
#pragma unroll
                    for (int j = 0; j < CK; j++) {
                        const float u = df[i][j] * ri;
                        acc[i][j] += c * __builtin_copysignf(pow_pos(__builtin_fabsf(u), e), u);
                    }
                }
            }
        };
        if (sparse) {
            reduce_sparse();
            continue;
        }
        if (factored) {
            switch (ie) {
                case 1: reduce_factored([](float u) { return u; }); break;
                case 2: reduce_factored([](float u) { return u * __builtin_fabsf(u); }); break;
                case 3: reduce_factored([](float u) { return pow_int<3>(u); }); break;
                default: reduce_factored([](float u) { return pow_int<7>(u); }); break;
            }
            continue;
        }
        switch (ie) {
            case 1: reduce([](float u) { return u; }); break;
            case 2: reduce([](float u) { return u * __builtin_fabsf(u); }); break;
            case 3: reduce([](float u) { return pow_int<3>(u); }); break;
            case 7: reduce([](float u) { return pow_int<7>(u); }); break;
            default:   // at u == 0 the power is 0 and the sign is irrelevant
                reduce([e](float u) { return __builtin_copysignf(pow_pos(__builtin_fabsf(u), e), u); });
                break;
        }
    }

#pragma unroll
    for (int i = 0; i < PA; i++)
#pragma unroll
        for (int j = 0; j < CK; j++) {
            const int a = a0 + ty * PA + i, k = k0 + tx + 16 * j;
            if (a < A && k < d.K) {
                if (WEIGHT) {
                    float* dst = grad + v.w_at(a, k);
                    if (SPLIT) atomicAdd(dst, acc[i][j]);
                    else *dst += acc[i][j];
                } else if constexpr (IMG) {
                    size_t off;
                    if (v.x_tap(a, k, off)) atomicAdd(grad + off, acc[i][j]);
                } else {
                    grad[v.x_at(a, k)] = acc[i][j];
                }
            }
        }
}

template <bool WEIGHT, int BA, int BKO, bool IMG>
static hipError_t launch_norm_backward_ba(const float* grad_output, const float* input, const float* weight,
                                          const float* output, float* grad, float p, const Problem& pr,
                                          hipStream_t stream, const ImgWin& win) {
    const NbDims d{pr.B, pr.G, pr.K, pr.NG, pr.HW, pr.B * pr.HW};
    const int A = WEIGHT ? d.NG : d.M;
    const int R = WEIGHT ? d.M : d.NG;
    const int tiles_a = (A + BA - 1) / BA, tiles_k = (d.K + BKO - 1) / BKO;
    const long tiles = (long)tiles_a * tiles_k * d.G;
    int splits = 1;
    if (WEIGHT && tiles < 2L * pr.num_cu) {  // few output tiles, long reduction over the rows: share it out
        const long want = (4L * pr.num_cu + tiles - 1) / tiles;
        const long most = max(1L, (long)R / (4 * RB));
        splits = (int)min(want, most);
    }
    int r_per_wg = (R + splits - 1) / splits;
    r_per_wg = (r_per_wg + RB - 1) / RB * RB;
    splits = (R + r_per_wg - 1) / r_per_wg;
    const dim3 grid((unsigned)tiles, (unsigned)splits);
    const bool conv = pr.HW != 1;
#define LDIST_LAUNCH(W, C, S)                                                                                      \
    hipLaunchKernelGGL((norm_backward_kernel<W, C, S, BA, BKO, IMG && C>), grid, dim3(256), 0, stream, grad_output, input,  \
                       weight, output, grad, p, d, tiles_a, tiles_k, r_per_wg, win)
    if constexpr (IMG) {   // an image always has the conv layout (a single position included)
        (void)conv;
        if (WEIGHT && splits > 1) LDIST_LAUNCH(WEIGHT, true, true); else LDIST_LAUNCH(WEIGHT, true, false);
    } else if (WEIGHT) {
        if (splits > 1) { if (conv) LDIST_LAUNCH(WEIGHT, true, true); else LDIST_LAUNCH(WEIGHT, false, true); }
        else { if (conv) LDIST_LAUNCH(WEIGHT, true, false); else LDIST_LAUNCH(WEIGHT, false, false); }
    } else {
        if (conv) LDIST_LAUNCH(WEIGHT, true, false); else LDIST_LAUNCH(WEIGHT, false, false);
    }
#undef LDIST_LAUNCH
    return hipGetLastError();
}

template <bool WEIGHT, bool IMG>
static hipError_t launch_norm_backward(const float* grad_output, const float* input, const float* weight,
                                       const float* output, float* grad, float p, const Problem& pr,
                                       hipStream_t stream, const ImgWin& win) {
    // 64-row tiles unless they would give fewer than four workgroups per CU (and the rows allow halving);
    // P with at most 32 rows (grad_weight of a grouped layer with few outputs per group): 32 x 128 tiles
    const int A = WEIGHT ? pr.NG : pr.B * pr.HW;
    if (A <= 32 && pr.K > 64)
        return launch_norm_backward_ba<WEIGHT, 32, 128, IMG>(grad_output, input, weight, output, grad, p, pr, stream, win);
    const long tiles64 = (long)((A + 63) / 64) * ((pr.K + 63) / 64) * pr.G;
    if (tiles64 < 4L * pr.num_cu && A > 32)
        return launch_norm_backward_ba<WEIGHT, 32, 64, IMG>(grad_output, input, weight, output, grad, p, pr, stream, win);
    return launch_norm_backward_ba<WEIGHT, 64, 64, IMG>(grad_output, input, weight, output, grad, p, pr, stream, win);
}

}  // namespace ldist
