// Interval-bound forward of the L_inf distance layer:
//   U[m,n] = max_k max(|l-w|, |u-w|)
//   L[m,n] = max_k min(|l-w|, |u-w|) over the k where not (l-w < 0 < u-w), else 0
// with l, u the lower/upper ends of the input box.  Semantics follow the
// reference kernel model/inf_dist_cuda.cu:73-141.
//
// For a regular box (l <= u, everything finite) the lower bound equals
// max_k max(l-w, w-u, 0), so the hot loop is two subtractions and two v_max3_f32
// per (m,n,k): U = max3(U, |tl|, |tu|), L = max3(L, tl, -tu)  (L starts at 0).
// Each stage checks what it loads; a stage that holds l > u, a NaN or an
// infinity anywhere in its panels is reduced with the reference's literal
// predicate instead, so results match the reference for every input.
#include "fwd_engine.hpp"
#include "skinny.hpp"

namespace ldist {

template <class GEO, bool CONV, int VEC>
__global__ void __launch_bounds__(GEO::NT, 2)
bound_forward_kernel(const float* __restrict__ lower, const float* __restrict__ upper,
                     const float* __restrict__ weight, float* __restrict__ out_lower, float* __restrict__ out_upper,
                     Dims d) {
    constexpr int BM = GEO::BM, BN = GEO::BN, TM = GEO::TM, TN = GEO::TN, KS = GEO::KS, KK = GEO::KK;
    constexpr int NGRP = GEO::NGRP;
    using Stage = Stager<GEO, CONV, VEC, 2>;
    constexpr int STAGE = Stage::STAGE, NBUF = Stage::NBUF;
    static_assert(2 * (KS - 1) * TM * TN * NGRP <= NBUF * STAGE, "merge area fits in the panels");
    extern __shared__ __align__(16) float lds[];

    int tm, tn, g;
    tile_of_block(d, tm, tn, g);
    const int m0 = tm * BM, n0 = tn * BN;
    const int tid = threadIdx.x;
    const int grp = tid / NGRP, t = tid % NGRP;
    const int tx = t % GEO::TX, ty = t / GEO::TX;

    Stage st;
    const float* const ins[2] = {lower, upper};
    st.init(ins, weight, d, m0, n0, g, tid);

    float lo[TM][TN], up[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) { lo[i][j] = 0.f; up[i][j] = 0.f; }

    const int nstage = (d.K + KK - 1) / KK;
    st.load(0);
    st.store(lds);
    int irregular = __syncthreads_or(st.interval_is_irregular());
    for (int s = 0; s < nstage; s++) {
        const float* stage = lds + (s % NBUF) * STAGE;
        if (s + 1 < nstage) st.load((s + 1) * KK);
        const float* xp = stage + grp * kChunk * GEO::SM;
        const float* wp = stage + 2 * GEO::XS + grp * kChunk * GEO::SN;
        if (!irregular) {
            sweep_chunk<GEO, 2, 1>(xp, wp, tx, ty, [&](const Frag<GEO, 2, 1>& f, int) {
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        {
                            const float tl = f.x[0][0][i] - f.w[0][j];
                            const float tu = f.x[1][0][i] - f.w[0][j];
                            up[i][j] = __builtin_fmaxf(__builtin_fmaxf(up[i][j], __builtin_fabsf(tl)),
                                                       __builtin_fabsf(tu));
                            lo[i][j] = __builtin_fmaxf(__builtin_fmaxf(lo[i][j], tl), -tu);
                        }
                    }
            });
        } else {
            // rare path, kept lean: a second pipelined sweep here would push the hot loop into scratch
            sweep_chunk_plain<GEO, 2>(xp, wp, tx, ty, [&](const Frag<GEO, 2, 1>& f, int) {
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        {
                            const float tl = f.x[0][0][i] - f.w[0][j];
                            const float tu = f.x[1][0][i] - f.w[0][j];
                            const float al = __builtin_fabsf(tl), au = __builtin_fabsf(tu);
                            up[i][j] = __builtin_fmaxf(up[i][j], __builtin_fmaxf(al, au));
                            if (!(tl < 0.f && tu > 0.f)) lo[i][j] = __builtin_fmaxf(lo[i][j], __builtin_fminf(al, au));
                        }
                    }
            });
        }
        bool next_irregular = false;
        if (NBUF == 1) __syncthreads();  // everyone is done reading the only buffer
        if (s + 1 < nstage) {
            next_irregular = st.interval_is_irregular();
            st.store(lds + ((s + 1) % NBUF) * STAGE);
        }
        irregular = __syncthreads_or(next_irregular);
    }

    if constexpr (KS > 1) {
        float* ml = lds;  // [KS-1][TM*TN][NGRP] lower bounds, then as many upper bounds
        float* mu = lds + (KS - 1) * TM * TN * NGRP;
        if (grp > 0) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const int o = ((grp - 1) * TM * TN + i * TN + j) * NGRP + t;
                    ml[o] = lo[i][j];
                    mu[o] = up[i][j];
                }
        }
        __syncthreads();
        if (grp > 0) return;
#pragma unroll
        for (int q = 0; q < KS - 1; q++)
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const int o = (q * TM * TN + i * TN + j) * NGRP + t;
                    lo[i][j] = __builtin_fmaxf(lo[i][j], ml[o]);
                    up[i][j] = __builtin_fmaxf(up[i][j], mu[o]);
                }
    }

    store_patch<GEO, CONV>(out_lower, lo, d, m0, n0, g, tx, ty, d.ovec != 0);
    store_patch<GEO, CONV>(out_upper, up, d, m0, n0, g, tx, ty, d.ovec != 0);
}

// Few outputs per group: lanes split k and apply the reference's literal predicate.
template <int RW, int NB, bool VEC>
__global__ void __launch_bounds__(256)
bound_forward_skinny_kernel(const float* __restrict__ lower, const float* __restrict__ upper,
                            const float* __restrict__ weight, float* __restrict__ out_lower,
                            float* __restrict__ out_upper, Dims d) {
    __shared__ float sl[4][RW * NB], su[4][RW * NB];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    SkinnyRows<RW> rows;
    rows.init(d);
    for (int nb = 0; nb < d.NG; nb += NB) {
        float lo[RW][NB], up[RW][NB];
#pragma unroll
        for (int r = 0; r < RW; r++)
#pragma unroll
            for (int j = 0; j < NB; j++) { lo[r][j] = 0.f; up[r][j] = 0.f; }
        const float* const ins[2] = {lower, upper};
        skinny_sweep<2, RW, NB, VEC>(ins, weight, rows, d, nb, tid, [&](int, const float (&xv)[2][RW], const float (&wv)[NB]) {
#pragma unroll
            for (int r = 0; r < RW; r++)
#pragma unroll
                for (int j = 0; j < NB; j++) {
                    const float tl = xv[0][r] - wv[j], tu = xv[1][r] - wv[j];
                    const float al = __builtin_fabsf(tl), au = __builtin_fabsf(tu);
                    up[r][j] = __builtin_fmaxf(up[r][j], __builtin_fmaxf(al, au));
                    if (!(tl < 0.f && tu > 0.f)) lo[r][j] = __builtin_fmaxf(lo[r][j], __builtin_fminf(al, au));
                }
        });
#pragma unroll
        for (int r = 0; r < RW; r++)
#pragma unroll
            for (int j = 0; j < NB; j++) {
                const float l = wave_max(lo[r][j]), u = wave_max(up[r][j]);
                if (lane == 63) { sl[wave][r * NB + j] = l; su[wave][r * NB + j] = u; }
            }
        __syncthreads();
        if (tid < RW * NB) {
            float l = sl[0][tid], u = su[0][tid];
#pragma unroll
            for (int q = 1; q < 4; q++) { l = __builtin_fmaxf(l, sl[q][tid]); u = __builtin_fmaxf(u, su[q][tid]); }
            const int r = tid / NB, j = tid % NB;
            if (rows.m0 + r < d.M && nb + j < d.NG) {
                out_lower[rows.ooff[r] + (size_t)(nb + j) * d.HW] = l;
                out_upper[rows.ooff[r] + (size_t)(nb + j) * d.HW] = u;
            }
        }
        __syncthreads();
    }
}

template <class GEO, bool CONV, int VEC>
struct BoundForward {
    static constexpr int X_PANELS = 2;   // lower and upper
    static hipError_t launch(unsigned grid, const Dims& d, int device, hipStream_t stream, const float* lower,
                             const float* upper, const float* weight, float* out_lower, float* out_upper) {
        const size_t lds = Stager<GEO, CONV, VEC, 2>::LDS_BYTES;
        auto kern = bound_forward_kernel<GEO, CONV, VEC>;
        static LdsRecord lds_allowed = {};   // per instantiation of this launcher, i.e. per kernel
        if (hipError_t e = allow_lds(kern, lds, device, lds_allowed); e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3(grid), dim3(GEO::NT), lds, stream, lower, upper, weight, out_lower, out_upper,
                           d);
        return hipGetLastError();
    }
};

hipError_t bound_forward(const float* lower, const float* upper, const float* weight, float* out_lower,
                         float* out_upper, const Problem& pr, hipStream_t stream) {
    if (pr.NG <= kSkinnyMaxNG) {
        const Dims d = make_dims(pr);
        const bool vec = pr.HW == 1 && pr.K % 4 == 0 && aligned16(lower) && aligned16(upper) && aligned16(weight);
#define LDIST_LAUNCH_RW(RW, NB, VEC)                                                                                          \
    hipLaunchKernelGGL((bound_forward_skinny_kernel<RW, NB, VEC>), dim3(skinny_grid(d, RW)), dim3(256), 0, stream, lower, \
                       upper, weight, out_lower, out_upper, d)
        // two rows per workgroup share the weight loads; with few rows (up to eight per CU) one each: more workgroups hide more latency
#define LDIST_LAUNCH_1(NB, VEC) LDIST_LAUNCH_RW(1, NB, VEC)
#define LDIST_LAUNCH_2(NB, VEC) LDIST_LAUNCH_RW(2, NB, VEC)
        if ((long)d.M * d.G <= 8L * pr.num_cu) LDIST_SKINNY_DISPATCH(pr.NG, vec, LDIST_LAUNCH_1);
        else LDIST_SKINNY_DISPATCH(pr.NG, vec, LDIST_LAUNCH_2);
#undef LDIST_LAUNCH_1
#undef LDIST_LAUNCH_2
#undef LDIST_LAUNCH_RW
        return hipGetLastError();
    }
    return dispatch_forward<BoundForward>(pr, can_vec4(pr, lower, upper, weight),
                                          can_vec4_out(pr, out_lower, out_upper), stream, lower, upper, weight,
                                          out_lower, out_upper);
}

}  // namespace ldist
