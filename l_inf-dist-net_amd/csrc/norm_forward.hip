// p-norm distance forward, p > 1:  out[m,n] = (sum_k |x[m,k] - w[n,k]|^p)^(1/p),
// evaluated as  mx * (sum_k (|x-w|/mx)^p)^(1/p)  with a running maximum mx so
// that no power can overflow for any p.  Semantics follow the reference kernel
// model/norm_dist_cuda.cu:228-292: mx and the sum are seeded with 1e-10 (:232-233),
// and whenever a block of k raises mx the sum is rescaled by (mx_old/mx_new)^p
// (:257-261).  Here the block is a 32-wide chunk: sweep one finds the chunk
// maximum (sub + half a max3 per element), the rescale runs once per output,
// sweep two adds (|x-w| / mx)^p.  p = 2, 3, 4, 8 use multiplies only; any other
// p goes through v_log_f32 / v_exp_f32.
#include "fwd_engine.hpp"
#include "pow.hpp"

namespace ldist {

template <class GEO, bool CONV, int VEC>
__global__ void __launch_bounds__(GEO::NT, 2)
norm_forward_kernel(const float* __restrict__ input, const float* __restrict__ weight, float* __restrict__ output,
                    float p, Dims d) {
    constexpr int BM = GEO::BM, BN = GEO::BN, TM = GEO::TM, TN = GEO::TN, KS = GEO::KS, KK = GEO::KK;
    constexpr int NGRP = GEO::NGRP;
    using Stage = Stager<GEO, CONV, VEC, 1>;
    constexpr int STAGE = Stage::STAGE, NBUF = Stage::NBUF;
    static_assert(2 * (KS - 1) * TM * TN * NGRP <= NBUF * STAGE, "merge area fits in the panels");
    extern __shared__ __align__(16) float lds[];

    int tm, tn, g;
    tile_of_block(d, tm, tn, g);
    const int m0 = tm * BM, n0 = tn * BN;
    const int tid = threadIdx.x;
    const int grp = tid / NGRP, t = tid % NGRP;
    const int tx = t % GEO::TX, ty = t / GEO::TX;
    const int ip = small_int_power(p);

    Stage st;
    const float* const ins[1] = {input};
    st.init(ins, weight, d, m0, n0, g, tid);

    float acc[TM][TN], mx[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) { acc[i][j] = grp == 0 ? 1e-10f : 0.f; mx[i][j] = 1e-10f; }

    const int nstage = (d.K + KK - 1) / KK;
    st.load(0);
    st.store(lds);
    __syncthreads();
    for (int s = 0; s < nstage; s++) {
        const float* stage = lds + (s % NBUF) * STAGE;
        if (s + 1 < nstage) st.load((s + 1) * KK);
        const float* xp = stage + grp * kChunk * GEO::SM;
        const float* wp = stage + GEO::XS + grp * kChunk * GEO::SN;
        float cm[TM][TN];  // chunk maximum, then 1 / running maximum
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) cm[i][j] = 0.f;
        sweep_chunk<GEO, 1, 2>(xp, wp, tx, ty, [&](const Frag<GEO, 1, 2>& f) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const float d0 = __builtin_fabsf(f.x[0][0][i] - f.w[0][j]);
                    const float d1 = __builtin_fabsf(f.x[0][1][i] - f.w[1][j]);
                    cm[i][j] = __builtin_fmaxf(__builtin_fmaxf(cm[i][j], d0), d1);
                }
        });
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) {
                if (cm[i][j] > mx[i][j]) {
                    acc[i][j] *= pow_pos(mx[i][j] * __builtin_amdgcn_rcpf(cm[i][j]), p);
                    mx[i][j] = cm[i][j];
                }
                cm[i][j] = __builtin_amdgcn_rcpf(mx[i][j]);
            }
        auto add_powers = [&](auto power) {
            sweep_chunk<GEO, 1, 2>(xp, wp, tx, ty, [&](const Frag<GEO, 1, 2>& f) {
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        const float v0 = __builtin_fabsf(f.x[0][0][i] - f.w[0][j]) * cm[i][j];
                        const float v1 = __builtin_fabsf(f.x[0][1][i] - f.w[1][j]) * cm[i][j];
                        acc[i][j] += power(v0);
                        acc[i][j] += power(v1);
                    }
            });
        };
        switch (ip) {
            case 2: add_powers([](float v) { return pow_int<2>(v); }); break;
            case 3: add_powers([](float v) { return pow_int<3>(v); }); break;
            case 4: add_powers([](float v) { return pow_int<4>(v); }); break;
            case 8: add_powers([](float v) { return pow_int<8>(v); }); break;
            default: add_powers([p](float v) { return pow_pos(v, p); }); break;
        }
        if (NBUF == 1) __syncthreads();  // everyone is done reading the only buffer
        if (s + 1 < nstage) st.store(lds + ((s + 1) % NBUF) * STAGE);
        __syncthreads();
    }

    // Merge the k-groups onto the common maximum.
    if constexpr (KS > 1) {
        float* ma = lds;  // [KS-1][TM*TN][NGRP] sums, then as many maxima
        float* mm = lds + (KS - 1) * TM * TN * NGRP;
        if (grp > 0) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const int o = ((grp - 1) * TM * TN + i * TN + j) * NGRP + t;
                    ma[o] = acc[i][j];
                    mm[o] = mx[i][j];
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
                    const float a2 = ma[o], m2 = mm[o];
                    const float m = __builtin_fmaxf(mx[i][j], m2);
                    const float r = __builtin_amdgcn_rcpf(m);
                    acc[i][j] = acc[i][j] * pow_pos(mx[i][j] * r, p) + a2 * pow_pos(m2 * r, p);
                    mx[i][j] = m;
                }
    }

    const float inv_p = 1.0f / p;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = pow_pos(acc[i][j], inv_p) * mx[i][j];
    store_patch<GEO, CONV>(output, acc, d, m0, n0, g, tx, ty, 0xFFu, d.ovec != 0);
}

template <class GEO, bool CONV, int VEC>
struct NormForward {
    static hipError_t launch(unsigned grid, const Dims& d, int device, hipStream_t stream, const float* input,
                             const float* weight, float* output, float p) {
        const size_t lds = Stager<GEO, CONV, VEC, 1>::LDS_BYTES;
        auto kern = norm_forward_kernel<GEO, CONV, VEC>;
        if (hipError_t e = allow_lds(kern, lds, device); e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3(grid), dim3(GEO::NT), lds, stream, input, weight, output, p, d);
        return hipGetLastError();
    }
};

hipError_t norm_forward(const float* input, const float* weight, float* output, float p, const Problem& pr,
                        hipStream_t stream) {
    return dispatch_forward<NormForward>(pr, can_vec4(pr, input, weight), can_vec4_out(pr, output), stream, input,
                                         weight, output, p);
}

}  // namespace ldist
