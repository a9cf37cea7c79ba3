// p-norm distance forward, p > 1:  out[m,n] = (sum_k |x[m,k] - w[n,k]|^p)^(1/p),
// evaluated as  mx * (sum_k (|x-w|/mx)^p)^(1/p)  with a running maximum mx so
// that no power can overflow for any p.  Semantics follow the reference kernel
// model/norm_dist_cuda.cu:228-292: mx and the sum are seeded with 1e-10 (:232-233),
// and whenever a block of k raises mx the sum is rescaled by (mx_old/mx_new)^p
// (:257-261).  Here the block is a 32-wide chunk.  Below p = 128 a chunk is normally
// swept once with the scale left by earlier chunks (see the kernel; a chunk that
// overflows is swept again the reference's way: maximum, rescale, powers);
// from p = 128 the kernel first
// finds the maxima over all of k and then takes only the powers that can matter
// (see MODE 2 in the kernel).  p = 2, 3, 4, 8 use multiplies only; any other p goes
// through v_log_f32 / v_exp_f32.
#include "norm_forward_kernel.hpp"
#include "skinny.hpp"

namespace ldist {

// Few outputs per group: two passes over k, first the exact maximum per (row, output),
// then the sum of (|x-w| / max)^p; lanes split k in both.
template <int RW, int NB, bool VEC>
__global__ void __launch_bounds__(256)
norm_forward_skinny_kernel(const float* __restrict__ input, const float* __restrict__ weight,
                           float* __restrict__ output, float p, Dims d) {
    __shared__ float red[4][RW * NB];
    __shared__ float bcast[RW * NB];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    SkinnyRows<RW> rows;
    rows.init(d);
    for (int nb = 0; nb < d.NG; nb += NB) {
        float acc[RW][NB], rmx[RW][NB];
        // pass 0: maximum; pass 1: power sum
        for (int pass = 0; pass < 2; pass++) {
#pragma unroll
            for (int r = 0; r < RW; r++)
#pragma unroll
                for (int j = 0; j < NB; j++) acc[r][j] = 0.f;
            const float* const ins[1] = {input};
            skinny_sweep<1, RW, NB, VEC>(ins, weight, rows, d, nb, tid, [&](int, const float (&xv)[1][RW], const float (&wv)[NB]) {
#pragma unroll
                for (int r = 0; r < RW; r++)
#pragma unroll
                    for (int j = 0; j < NB; j++) {
                        const float a = __builtin_fabsf(xv[0][r] - wv[j]);
                        if (pass == 0) acc[r][j] = __builtin_fmaxf(acc[r][j], a);
                        else acc[r][j] += pow_pos(a * rmx[r][j], p);
                    }
            });
#pragma unroll
            for (int r = 0; r < RW; r++)
#pragma unroll
                for (int j = 0; j < NB; j++) {
                    const float v = pass == 0 ? wave_max(acc[r][j]) : wave_sum(acc[r][j]);
                    if (lane == 63) red[wave][r * NB + j] = v;
                }
            __syncthreads();
            if (tid < RW * NB) {
                float v = red[0][tid];
#pragma unroll
                for (int q = 1; q < 4; q++) v = pass == 0 ? __builtin_fmaxf(v, red[q][tid]) : v + red[q][tid];
                if (pass == 0) {
                    bcast[tid] = __builtin_fmaxf(v, 1e-10f);   // the reference's seed for the maximum
                } else {
                    const float mx = bcast[tid];
                    const float sum = v + 1e-10f * pow_pos(1e-10f * __builtin_amdgcn_rcpf(mx), p);  // seeded sum
                    const int r = tid / NB, j = tid % NB;
                    if (rows.m0 + r < d.M && nb + j < d.NG)
                        output[rows.ooff[r] + (size_t)(nb + j) * d.HW] = pow_pos(sum, 1.0f / p) * mx;
                }
            }
            __syncthreads();
            if (pass == 0) {
#pragma unroll
                for (int r = 0; r < RW; r++)
#pragma unroll
                    for (int j = 0; j < NB; j++) rmx[r][j] = __builtin_amdgcn_rcpf(bcast[r * NB + j]);
            }
            __syncthreads();
        }
    }
}

template <class GEO, bool CONV, int VEC>
struct NormForward {
    static hipError_t launch(unsigned grid, const Dims& d, int device, hipStream_t stream, const float* input,
                             const float* weight, float* output, float p) {
        return NormForwardLaunch<GEO, CONV, VEC, false>::launch(grid, d, device, stream, input, weight, output, p, ImgWin{});
    }
};

hipError_t norm_forward(const float* input, const float* weight, float* output, float p, const Problem& pr,
                        hipStream_t stream) {
    if (pr.NG <= kSkinnyMaxNG) {
        const Dims d = make_dims(pr);
        const bool vec = pr.HW == 1 && pr.K % 4 == 0 && aligned16(input) && aligned16(weight);
#define LDIST_LAUNCH_RW(RW, NB, VEC)                                                                                        \
    hipLaunchKernelGGL((norm_forward_skinny_kernel<RW, NB, VEC>), dim3(skinny_grid(d, RW)), dim3(256), 0, stream, input, \
                       weight, output, p, d)
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
    return dispatch_forward<NormForward>(pr, can_vec4(pr, input, weight), can_vec4_out(pr, output), stream, input,
                                         weight, output, p);
}

}  // namespace ldist
