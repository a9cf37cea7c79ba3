// Values and interval bounds of the L_inf distance layer in one pass over the weights:
//   Y[m,n] = max_k |x-w|
//   U[m,n] = max_k max(|l-w|, |u-w|)
//   L[m,n] = max_k min(|l-w|, |u-w|) over the k where not (l-w < 0 < u-w), else 0
// for a point x and the box [l, u] around it -- what certification evaluates per layer (reference
// model/norm_dist.py:134,144-155 calls the value kernel and the bound kernel one after the other;
// the results here are those of model/inf_dist_cuda.cu:10-68 without the index and :73-141).
// The evaluation-mode epilogue of the layer is part of the kernel: every output channel c may have
// a mean subtracted and then a bias added, (v - mean[c]) + bias[c] in that order, as MeanNorm and
// the bias do in the reference (model/norm_dist.py:146-155).
//
// Three input panels (x, l, u) and the weight panel per stage; the hot loop is three subtractions,
// two v_max3_f32 and one v_max_f32 per (m,n,k).  No index is kept: certification runs without a
// backward pass.  Irregular boxes are handled as in the bound kernel.
#include "fwd_engine.hpp"
#include "skinny.hpp"

namespace ldist {

// (v - mean[c]) + bias[c] for the lane's patch; either pointer may be null.
template <class GEO>
__device__ __forceinline__ void shift_patch(float (&val)[GEO::TM][GEO::TN], const float* __restrict__ mean,
                                            const float* __restrict__ bias, const Dims& d, int n0, int g, int tx) {
#pragma unroll
    for (int j = 0; j < GEO::TN; j++) {
        const int n = n0 + GEO::col(tx, j);
        if (n >= d.NG) continue;
        const int c = g * d.NG + n;
        const float mu = mean ? mean[c] : 0.f, b = bias ? bias[c] : 0.f;
#pragma unroll
        for (int i = 0; i < GEO::TM; i++) {
            float v = val[i][j];
            if (mean) v -= mu;
            if (bias) v += b;
            val[i][j] = v;
        }
    }
}

template <class GEO, bool CONV, int VEC>
__global__ void __launch_bounds__(GEO::NT, 2)
value_bound_forward_kernel(const float* __restrict__ input, const float* __restrict__ lower,
                           const float* __restrict__ upper, const float* __restrict__ weight,
                           const float* __restrict__ mean, const float* __restrict__ bias,
                           float* __restrict__ out, float* __restrict__ out_lower, float* __restrict__ out_upper,
                           Dims d) {
    constexpr int BM = GEO::BM, BN = GEO::BN, TM = GEO::TM, TN = GEO::TN, KS = GEO::KS, KK = GEO::KK;
    constexpr int NGRP = GEO::NGRP;
    using Stage = Stager<GEO, CONV, VEC, 3>;
    constexpr int STAGE = Stage::STAGE, NBUF = Stage::NBUF;
    static_assert(3 * (KS - 1) * TM * TN * NGRP <= NBUF * STAGE, "merge area fits in the panels");
    extern __shared__ __align__(16) float lds[];

    int tm, tn, g;
    tile_of_block(d, tm, tn, g);
    const int m0 = tm * BM, n0 = tn * BN;
    const int tid = threadIdx.x;
    const int grp = tid / NGRP, t = tid % NGRP;
    const int tx = t % GEO::TX, ty = t / GEO::TX;

    Stage st;
    const float* const ins[3] = {input, lower, upper};
    st.init(ins, weight, d, m0, n0, g, tid);

    float val[TM][TN], lo[TM][TN], up[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) { val[i][j] = 0.f; lo[i][j] = 0.f; up[i][j] = 0.f; }

    const int nstage = (d.K + KK - 1) / KK;
    st.load(0);
    st.store(lds);
    int irregular = __syncthreads_or(st.interval_is_irregular());
    // Unlike the other forward kernels this one fetches the next stage only after the sweep: three accumulator sets
    // and the operands of three panels leave no registers for a stage in flight (58 more per lane with the 8 x 5
    // patch; kept in flight, a sixth of the hot loop's values lived in scratch).  The 256-lane tiles run two
    // workgroups per CU, one of which sweeps while the other fetches.
    for (int s = 0; s < nstage; s++) {
        const float* stage = lds + (s % NBUF) * STAGE;
        const float* xp = stage + grp * kChunk * GEO::SM;
        const float* wp = stage + 3 * GEO::XS + grp * kChunk * GEO::SN;
        if (!irregular) {
            sweep_chunk<GEO, 3, 1>(xp, wp, tx, ty, [&](const Frag<GEO, 3, 1>& f, int) {
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        const float tv = f.x[0][0][i] - f.w[0][j];
                        const float tl = f.x[1][0][i] - f.w[0][j];
                        const float tu = f.x[2][0][i] - f.w[0][j];
                        val[i][j] = __builtin_fmaxf(val[i][j], __builtin_fabsf(tv));
                        up[i][j] = __builtin_fmaxf(__builtin_fmaxf(up[i][j], __builtin_fabsf(tl)), __builtin_fabsf(tu));
                        lo[i][j] = __builtin_fmaxf(__builtin_fmaxf(lo[i][j], tl), -tu);
                    }
            });
        } else {
            // rare path, kept lean: the reference's literal predicate for the lower bound
            sweep_chunk_plain<GEO, 3>(xp, wp, tx, ty, [&](const Frag<GEO, 3, 1>& f, int) {
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        const float tv = f.x[0][0][i] - f.w[0][j];
                        const float tl = f.x[1][0][i] - f.w[0][j];
                        const float tu = f.x[2][0][i] - f.w[0][j];
                        const float al = __builtin_fabsf(tl), au = __builtin_fabsf(tu);
                        val[i][j] = __builtin_fmaxf(val[i][j], __builtin_fabsf(tv));
                        up[i][j] = __builtin_fmaxf(up[i][j], __builtin_fmaxf(al, au));
                        if (!(tl < 0.f && tu > 0.f)) lo[i][j] = __builtin_fmaxf(lo[i][j], __builtin_fminf(al, au));
                    }
            });
        }
        bool next_irregular = false;
        if (NBUF == 1) __syncthreads();  // everyone is done reading the only buffer
        if (s + 1 < nstage) {
            st.load((s + 1) * KK);
            next_irregular = st.interval_is_irregular();
            st.store(lds + ((s + 1) % NBUF) * STAGE);
        }
        irregular = __syncthreads_or(next_irregular);
    }

    if constexpr (KS > 1) {
        constexpr int PLANE = (KS - 1) * TM * TN * NGRP;   // values, then lower bounds, then upper bounds
        if (grp > 0) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const int o = ((grp - 1) * TM * TN + i * TN + j) * NGRP + t;
                    lds[o] = val[i][j];
                    lds[PLANE + o] = lo[i][j];
                    lds[2 * PLANE + o] = up[i][j];
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
                    val[i][j] = __builtin_fmaxf(val[i][j], lds[o]);
                    lo[i][j] = __builtin_fmaxf(lo[i][j], lds[PLANE + o]);
                    up[i][j] = __builtin_fmaxf(up[i][j], lds[2 * PLANE + o]);
                }
    }

    if (mean || bias) {
        shift_patch<GEO>(val, mean, bias, d, n0, g, tx);
        shift_patch<GEO>(lo, mean, bias, d, n0, g, tx);
        shift_patch<GEO>(up, mean, bias, d, n0, g, tx);
    }
    store_patch<GEO, CONV>(out, val, d, m0, n0, g, tx, ty, d.ovec != 0);
    store_patch<GEO, CONV>(out_lower, lo, d, m0, n0, g, tx, ty, d.ovec != 0);
    store_patch<GEO, CONV>(out_upper, up, d, m0, n0, g, tx, ty, d.ovec != 0);
}

// Few outputs per group: lanes split k and apply the reference's literal predicate.
template <int RW, int NB, bool VEC>
__global__ void __launch_bounds__(256)
value_bound_forward_skinny_kernel(const float* __restrict__ input, const float* __restrict__ lower,
                                  const float* __restrict__ upper, const float* __restrict__ weight,
                                  const float* __restrict__ mean, const float* __restrict__ bias,
                                  float* __restrict__ out, float* __restrict__ out_lower,
                                  float* __restrict__ out_upper, Dims d) {
    __shared__ float sv[4][RW * NB], sl[4][RW * NB], su[4][RW * NB];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    SkinnyRows<RW> rows;
    rows.init(d);
    for (int nb = 0; nb < d.NG; nb += NB) {
        float val[RW][NB], lo[RW][NB], up[RW][NB];
#pragma unroll
        for (int r = 0; r < RW; r++)
#pragma unroll
            for (int j = 0; j < NB; j++) { val[r][j] = 0.f; lo[r][j] = 0.f; up[r][j] = 0.f; }
        const float* const ins[3] = {input, lower, upper};
        skinny_sweep<3, RW, NB, VEC>(ins, weight, rows, d, nb, tid, [&](int, const float (&xv)[3][RW], const float (&wv)[NB]) {
#pragma unroll
            for (int r = 0; r < RW; r++)
#pragma unroll
                for (int j = 0; j < NB; j++) {
                    const float tl = xv[1][r] - wv[j], tu = xv[2][r] - wv[j];
                    const float al = __builtin_fabsf(tl), au = __builtin_fabsf(tu);
                    val[r][j] = __builtin_fmaxf(val[r][j], __builtin_fabsf(xv[0][r] - wv[j]));
                    up[r][j] = __builtin_fmaxf(up[r][j], __builtin_fmaxf(al, au));
                    if (!(tl < 0.f && tu > 0.f)) lo[r][j] = __builtin_fmaxf(lo[r][j], __builtin_fminf(al, au));
                }
        });
#pragma unroll
        for (int r = 0; r < RW; r++)
#pragma unroll
            for (int j = 0; j < NB; j++) {
                const float v = wave_max(val[r][j]), l = wave_max(lo[r][j]), u = wave_max(up[r][j]);
                if (lane == 63) { sv[wave][r * NB + j] = v; sl[wave][r * NB + j] = l; su[wave][r * NB + j] = u; }
            }
        __syncthreads();
        if (tid < RW * NB) {
            float v = sv[0][tid], l = sl[0][tid], u = su[0][tid];
#pragma unroll
            for (int q = 1; q < 4; q++) {
                v = __builtin_fmaxf(v, sv[q][tid]);
                l = __builtin_fmaxf(l, sl[q][tid]);
                u = __builtin_fmaxf(u, su[q][tid]);
            }
            const int r = tid / NB, j = tid % NB;
            if (rows.m0 + r < d.M && nb + j < d.NG) {
                const int c = rows.g * d.NG + nb + j;
                if (mean) { const float mu = mean[c]; v -= mu; l -= mu; u -= mu; }
                if (bias) { const float b = bias[c]; v += b; l += b; u += b; }
                const size_t o = rows.ooff[r] + (size_t)(nb + j) * d.HW;
                out[o] = v;
                out_lower[o] = l;
                out_upper[o] = u;
            }
        }
        __syncthreads();
    }
}

template <class GEO, bool CONV, int VEC>
struct ValueBoundForward {
    static constexpr int X_PANELS = 3;   // the point, lower and upper
    static hipError_t launch(unsigned grid, const Dims& d, int device, hipStream_t stream, const float* input,
                             const float* lower, const float* upper, const float* weight, const float* mean,
                             const float* bias, float* out, float* out_lower, float* out_upper) {
        const size_t lds = Stager<GEO, CONV, VEC, 3>::LDS_BYTES;
        auto kern = value_bound_forward_kernel<GEO, CONV, VEC>;
        static LdsRecord lds_allowed = {};   // per instantiation of this launcher, i.e. per kernel
        if (hipError_t e = allow_lds(kern, lds, device, lds_allowed); e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3(grid), dim3(GEO::NT), lds, stream, input, lower, upper, weight, mean, bias, out,
                           out_lower, out_upper, d);
        return hipGetLastError();
    }
};

hipError_t value_bound_forward(const float* input, const float* lower, const float* upper, const float* weight,
                               const float* mean, const float* bias, float* out, float* out_lower, float* out_upper,
                               const Problem& pr, hipStream_t stream) {
    if (pr.NG <= kSkinnyMaxNG) {
        const Dims d = make_dims(pr);
        const bool vec = pr.HW == 1 && pr.K % 4 == 0 && aligned16(input) && aligned16(lower) && aligned16(upper) &&
                         aligned16(weight);
#define LDIST_LAUNCH_RW(RW, NB, VEC)                                                                                       \
    hipLaunchKernelGGL((value_bound_forward_skinny_kernel<RW, NB, VEC>), dim3(skinny_grid(d, RW)), dim3(256), 0, stream, \
                       input, lower, upper, weight, mean, bias, out, out_lower, out_upper, d)
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
    const bool vec_in = can_vec4(pr, input, lower, upper) && aligned16(weight);
    const bool vec_out = can_vec4_out(pr, out, out_lower) && aligned16(out_upper);
    return dispatch_forward<ValueBoundForward>(pr, vec_in, vec_out, stream, input, lower, upper, weight, mean, bias,
                                               out, out_lower, out_upper);
}

}  // namespace ldist
