// L_inf distance forward with argmax: out[m,n] = max_k |x[m,k] - w[n,k]|,
// pos[m,n] = lowest k attaining it (bit 31 set when x - w < 0 there).
// Semantics follow the reference kernel model/inf_dist_cuda.cu:10-68.
//
// Hot loop: per (m,n,k) one v_sub_f32 plus half a v_max3_f32 (|.| is a free
// source modifier), with no index bookkeeping.  Only once per 32-wide chunk of
// k is the chunk maximum compared with the running maximum; a strict '>' there
// records the chunk.  After the k loop the lowest k with |x-w| == out is found
// by scanning that one chunk again, which reproduces "scan k ascending, update
// on strict >" exactly (the first chunk to reach the final maximum contains the
// first k to reach it).
#include "fwd_engine.hpp"

namespace ldist {

template <class GEO, bool CONV, int VEC>
__global__ void __launch_bounds__(GEO::NT, 2)
inf_forward_kernel(const float* __restrict__ input, const float* __restrict__ weight, float* __restrict__ output,
                   int32_t* __restrict__ pos, Dims d) {
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
    const int K = d.K;

    Stage st;
    const float* const ins[1] = {input};
    st.init(ins, weight, d, m0, n0, g, tid);

    float acc[TM][TN];
    int cidx[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) { acc[i][j] = 0.f; cidx[i][j] = 0; }

    const int nstage = (K + KK - 1) / KK;
    st.load(0);
    st.store(lds);
    __syncthreads();
    for (int s = 0; s < nstage; s++) {
        const float* stage = lds + (s % NBUF) * STAGE;
        if (s + 1 < nstage) st.load((s + 1) * KK);
        float cm[TM][TN];
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) cm[i][j] = 0.f;
        sweep_chunk<GEO, 1, 2>(stage + grp * kChunk * GEO::SM, stage + GEO::XS + grp * kChunk * GEO::SN, tx, ty,
                            [&](const Frag<GEO, 1, 2>& f) {
#pragma unroll
                                for (int i = 0; i < TM; i++)
#pragma unroll
                                    for (int j = 0; j < TN; j++) {
                                        const float d0 = __builtin_fabsf(f.x[0][0][i] - f.w[0][j]);
                                        const float d1 = __builtin_fabsf(f.x[0][1][i] - f.w[1][j]);
                                        cm[i][j] = __builtin_fmaxf(__builtin_fmaxf(cm[i][j], d0), d1);
                                    }
                            });
        const int c = s * KS + grp;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) {
                if (cm[i][j] > acc[i][j]) { acc[i][j] = cm[i][j]; cidx[i][j] = c; }
            }
        if (NBUF == 1) __syncthreads();  // everyone is done reading the only buffer
        if (s + 1 < nstage) st.store(lds + ((s + 1) % NBUF) * STAGE);
        __syncthreads();
    }

    // Merge the k-groups: the larger value wins, equal values keep the lower chunk.
    if constexpr (KS > 1) {
        float* mv = lds;  // [KS-1][TM*TN][NGRP] values, then as many chunk ids
        int* mi = reinterpret_cast<int*>(lds) + (KS - 1) * TM * TN * NGRP;
        if (grp > 0) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const int o = ((grp - 1) * TM * TN + i * TN + j) * NGRP + t;
                    mv[o] = acc[i][j];
                    mi[o] = cidx[i][j];
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
                    const float v = mv[o];
                    const int ci = mi[o];
                    if (v > acc[i][j] || (v == acc[i][j] && ci < cidx[i][j])) { acc[i][j] = v; cidx[i][j] = ci; }
                }
    }

    // Locate the argmax inside the recorded chunk and write both outputs.
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int m = m0 + GEO::row(ty, i);
        if (m >= d.M) continue;
        const RowAddr<CONV> ra(d, m, g);
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int n = n0 + GEO::col(tx, j);
            if (n >= d.NG) continue;
            const float best = acc[i][j];
            int p = 0;
            if (best > 0.f) {
                const int kb = cidx[i][j] * kChunk;
                const int ke = min(kb + kChunk, K);
                const float* xr = input + ra.x + (size_t)kb * ra.xk;
                const float* wr = weight + ((size_t)g * d.NG + n) * K + kb;
                for (int k = ke - kb - 1; k >= 0; k--) {  // descending: the lowest match is written last
                    const float df = xr[(size_t)k * ra.xk] - wr[k];
                    if (__builtin_fabsf(df) == best) p = (kb + k) | (__float_as_int(df) & 0x80000000);
                }
            }
            output[ra.o + (size_t)n * ra.on] = best;
            pos[ra.o + (size_t)n * ra.on] = p;
        }
    }
}

template <class GEO, bool CONV, int VEC>
struct InfForward {
    static hipError_t launch(unsigned grid, const Dims& d, int device, hipStream_t stream, const float* input,
                             const float* weight, float* output, int32_t* pos) {
        const size_t lds = Stager<GEO, CONV, VEC, 1>::LDS_BYTES;
        auto kern = inf_forward_kernel<GEO, CONV, VEC>;
        if (hipError_t e = allow_lds(kern, lds, device); e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3(grid), dim3(GEO::NT), lds, stream, input, weight, output, pos, d);
        return hipGetLastError();
    }
};

// ---------------------------------------------------------------------------
// Few outputs per group (the 10-way classification head): one wave per row m,
// lanes split k, each lane keeps the exact (value, k) pair per output and the
// wave reduces with "larger value, then lower k".  Memory bound by design.
// ---------------------------------------------------------------------------
template <int NB>
__global__ void __launch_bounds__(256)
inf_forward_skinny_kernel(const float* __restrict__ input, const float* __restrict__ weight,
                          float* __restrict__ output, int32_t* __restrict__ pos, Dims d) {
    const int lane = threadIdx.x & 63;
    const int wave = (blockIdx.x * 256 + threadIdx.x) >> 6;
    const int rows = d.M * d.G;
    if (wave >= rows) return;
    const int m = wave / d.G, g = wave % d.G;
    const int b = m / d.HW, hw = m % d.HW;
    const int K = d.K, xk = d.HW;
    const float* xr = input + ((size_t)(b * d.G + g) * K) * d.HW + hw;
    const size_t ooff = ((size_t)(b * d.G + g) * d.NG) * d.HW + hw;
    for (int nb = 0; nb < d.NG; nb += NB) {
        float best[NB];
        int bk[NB];
#pragma unroll
        for (int j = 0; j < NB; j++) { best[j] = 0.f; bk[j] = 0; }
        for (int k = lane; k < K; k += 64) {
            const float xv = xr[(size_t)k * xk];
#pragma unroll
            for (int j = 0; j < NB; j++) {
                if (nb + j < d.NG) {
                    const float df = xv - weight[((size_t)g * d.NG + nb + j) * K + k];
                    const float a = __builtin_fabsf(df);
                    if (a > best[j]) { best[j] = a; bk[j] = k | (__float_as_int(df) & 0x80000000); }
                }
            }
        }
#pragma unroll
        for (int j = 0; j < NB; j++) {
            float v = best[j];
            int p = bk[j];
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) {
                const float ov = __shfl_xor(v, off, 64);
                const int op = __shfl_xor(p, off, 64);
                const bool take = ov > v || (ov == v && (op & 0x7fffffff) < (p & 0x7fffffff));
                if (take) { v = ov; p = op; }
            }
            if (lane == 0 && nb + j < d.NG) {
                output[ooff + (size_t)(nb + j) * d.HW] = v;
                pos[ooff + (size_t)(nb + j) * d.HW] = v > 0.f ? p : 0;
            }
        }
    }
}

hipError_t inf_forward(const float* input, const float* weight, float* output, int32_t* pos, const Problem& pr,
                       hipStream_t stream) {
    if (pr.NG <= 16) {
        const Dims d = make_dims(pr);
        const int rows = d.M * d.G;
        const unsigned grid = (unsigned)((rows + 3) / 4);
        hipLaunchKernelGGL(inf_forward_skinny_kernel<8>, dim3(grid), dim3(256), 0, stream, input, weight, output, pos,
                           d);
        return hipGetLastError();
    }
    return dispatch_forward<InfForward>(pr, can_vec4(pr, input, weight), stream, input, weight, output, pos);
}

}  // namespace ldist
