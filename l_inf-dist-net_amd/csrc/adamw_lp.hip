// One AdamW step with the reference's row-wise l_p weight decay, fused into a single pass over
// the parameter (reference adamw.py:36-85, which spends about sixteen elementwise torch kernels
// per tensor).  The parameter is viewed as (rows, cols); decay first, on the parameter itself:
//   mode PLAIN   (the owning module has no p):  w *= 1 - lr*wd                         (:42-43)
//   mode FINITE  (:44-50):  a = w^2 + eps, s = a / max_row(a), q = s^(p/2 - 1),
//                           w += -lr*wd * (sum_row s*q)^(2/p - 1) * q * w
//   mode INF     (:51-55):  only the first element of largest |w| in the row: w -= lr*wd * w
// then Adam on the decayed value (:73-85):
//   m = b1*m + (1-b1)*g,  v = b2*v + (1-b2)*g*g,  w -= lr/(1-b1^t) * m / (sqrt(v)/sqrt(1-b2^t) + eps)
// HBM-bound: w, g, m, v are read once and w, m, v written once; the row statistics need two more
// sweeps over the row, which come from cache (a row of 5120 floats is 20 KB).
#include <cmath>

#include "kernels.hpp"
#include "pow.hpp"
#include "wave_reduce.hpp"

namespace ldist {

enum : int { kDecayPlain = 0, kDecayFinite = 1, kDecayInf = 2 };

struct AdamArgs {
    float neg_lr_wd;       // -lr * weight_decay
    float plain_factor;    // 1 - lr * weight_decay, formed in double (PLAIN)
    float beta1, beta2, eps;
    float one_minus_beta1, one_minus_beta2;   // formed in double on the host
    float step_size;       // lr / (1 - beta1^t)
    float inv_sqrt_bc2;    // 1 / sqrt(1 - beta2^t)
    float half_p;          // p / 2            (FINITE)
    float outer;           // 2 / p - 1        (FINITE)
    int with_adam;         // 0: decay only (grad, exp_avg, exp_avg_sq unused)
};

__device__ __forceinline__ float adam_update(float w, float g, float& m, float& v, const AdamArgs& a) {
    m = a.beta1 * m + a.one_minus_beta1 * g;
    v = a.beta2 * v + a.one_minus_beta2 * g * g;
    const float denom = __builtin_sqrtf(v) * a.inv_sqrt_bc2 + a.eps;
    return w - a.step_size * (m / denom);
}

__device__ __forceinline__ float block_max(float v, float* red) {
    v = wave_max(v);                // lane 63 holds the wave's maximum
    __syncthreads();
    if ((threadIdx.x & 63) == 63) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = red[0];
    for (int q = 1; q < (int)(blockDim.x >> 6); q++) r = __builtin_fmaxf(r, red[q]);
    return r;
}

__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);                // lane 63 holds the wave's sum
    __syncthreads();
    if ((threadIdx.x & 63) == 63) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = 0.f;
    for (int q = 0; q < (int)(blockDim.x >> 6); q++) r += red[q];
    return r;
}

// One workgroup per row.  VEC = 4 needs cols % 4 == 0 and 16-byte aligned tensors.
template <int MODE, int VEC>
__global__ void __launch_bounds__(256)
adamw_lp_rows_kernel(float* __restrict__ param, const float* __restrict__ grad, float* __restrict__ exp_avg,
                     float* __restrict__ exp_avg_sq, int cols, AdamArgs a) {
    __shared__ float red[4];
    __shared__ int red_i[4];
    const size_t base = (size_t)blockIdx.x * cols;
    float* w = param + base;
    const int nvec = cols / VEC;
    auto load = [&](const float* p, int i, float (&v)[VEC]) {
        if constexpr (VEC == 4) {
            const float4 t = reinterpret_cast<const float4*>(p)[i];
            v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
        } else {
            v[0] = p[i];
        }
    };
    auto store = [&](float* p, int i, const float (&v)[VEC]) {
        if constexpr (VEC == 4) reinterpret_cast<float4*>(p)[i] = make_float4(v[0], v[1], v[2], v[3]);
        else p[i] = v[0];
    };

    float rinv_max = 0.f, coef = 0.f;   // FINITE: 1 / max_row(w^2 + eps), (sum_row s^(p/2))^(2/p - 1)
    int decayed = -1;                   // INF: the column that decays
    if constexpr (MODE == kDecayFinite) {
        float mx = 0.f;
        for (int i = threadIdx.x; i < nvec; i += 256) {
            float v[VEC];
            load(w, i, v);
#pragma unroll
            for (int e = 0; e < VEC; e++) mx = __builtin_fmaxf(mx, v[e] * v[e] + a.eps);
        }
        mx = block_max(mx, red);
        rinv_max = 1.0f / mx;
        float sum = 0.f;
        for (int i = threadIdx.x; i < nvec; i += 256) {
            float v[VEC];
            load(w, i, v);
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                const float s = (v[e] * v[e] + a.eps) * rinv_max;
                if (s > 0.f) sum += pow_pos(s, a.half_p);   // s * s^(p/2-1)
            }
        }
        sum = block_sum(sum, red);
        coef = pow_pos(sum, a.outer);
    } else if constexpr (MODE == kDecayInf) {
        float best = -1.f;
        int where = 0x7fffffff;
        for (int i = threadIdx.x; i < nvec; i += 256) {
            float v[VEC];
            load(w, i, v);
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                const float m = __builtin_fabsf(v[e]);
                if (m > best) { best = m; where = i * VEC + e; }   // ascending columns per lane: first maximum kept
            }
        }
        wave_best(best, where);     // larger value, then lower column: lane 63
        if ((threadIdx.x & 63) == 63) { red[threadIdx.x >> 6] = best; red_i[threadIdx.x >> 6] = where; }
        __syncthreads();
        best = red[0];
        where = red_i[0];
        for (int q = 1; q < 4; q++)
            if (red[q] > best || (red[q] == best && red_i[q] < where)) { best = red[q]; where = red_i[q]; }
        decayed = where;
    }

    for (int i = threadIdx.x; i < nvec; i += 256) {
        float v[VEC], g[VEC], m[VEC], s2[VEC];
        load(w, i, v);
        if (a.with_adam) {
            load(grad + base, i, g);
            load(exp_avg + base, i, m);
            load(exp_avg_sq + base, i, s2);
        }
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            float x = v[e];
            if constexpr (MODE == kDecayPlain) {
                x = x * a.plain_factor;
            } else if constexpr (MODE == kDecayFinite) {
                const float s = (x * x + a.eps) * rinv_max;
                // s == 0 needs eps == 0 and w == 0: torch.pow(0, e) is 1 for e == 0, else 0
                const float q = s > 0.f ? pow_pos(s, a.half_p - 1.0f) : (a.half_p == 1.0f ? 1.0f : 0.0f);
                x = x + a.neg_lr_wd * (coef * q) * x;
            } else {
                if (i * VEC + e == decayed) x = x + a.neg_lr_wd * x;
            }
            if (a.with_adam) x = adam_update(x, g[e], m[e], s2[e], a);
            v[e] = x;
        }
        store(w, i, v);
        if (a.with_adam) {
            store(exp_avg + base, i, m);
            store(exp_avg_sq + base, i, s2);
        }
    }
}

// cols == 1 (biases): every row is its own maximum, so all three modes decay every element by
// lr*wd (PLAIN as a product, the others as the reference's w + (-lr*wd)*w).
__global__ void __launch_bounds__(256)
adamw_lp_scalar_rows_kernel(float* __restrict__ param, const float* __restrict__ grad, float* __restrict__ exp_avg,
                            float* __restrict__ exp_avg_sq, int rows, int plain, AdamArgs a) {
    const int r = blockIdx.x * 256 + threadIdx.x;
    if (r >= rows) return;
    float x = param[r];
    x = plain ? x * a.plain_factor : x + a.neg_lr_wd * x;
    if (a.with_adam) {
        float m = exp_avg[r], v = exp_avg_sq[r];
        x = adam_update(x, grad[r], m, v, a);
        exp_avg[r] = m;
        exp_avg_sq[r] = v;
    }
    param[r] = x;
}

hipError_t adamw_lp_step(float* param, const float* grad, float* exp_avg, float* exp_avg_sq, int rows, int cols,
                         double p_norm, double lr, double beta1, double beta2, double eps, double weight_decay, int step,
                         hipStream_t stream) {
    AdamArgs a{};
    a.neg_lr_wd = (float)(-lr * weight_decay);
    a.plain_factor = (float)(1.0 - lr * weight_decay);
    a.beta1 = (float)beta1;
    a.beta2 = (float)beta2;
    a.one_minus_beta1 = (float)(1.0 - beta1);
    a.one_minus_beta2 = (float)(1.0 - beta2);
    a.eps = (float)eps;
    a.step_size = (float)(lr / (1.0 - std::pow(beta1, (double)step)));
    a.inv_sqrt_bc2 = (float)(1.0 / std::sqrt(1.0 - std::pow(beta2, (double)step)));
    a.with_adam = grad != nullptr;
    const int mode = !(p_norm > 0.0) ? kDecayPlain : (std::isinf(p_norm) ? kDecayInf : kDecayFinite);
    if (mode == kDecayFinite) {
        a.half_p = (float)(0.5 * p_norm);
        a.outer = (float)(2.0 / p_norm - 1.0);
    }
    if (cols == 1) {
        hipLaunchKernelGGL(adamw_lp_scalar_rows_kernel, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, stream,
                           param, grad, exp_avg, exp_avg_sq, rows, mode == kDecayPlain ? 1 : 0, a);
        return hipGetLastError();
    }
    const bool vec = cols % 4 == 0 && aligned16(param) && aligned16(grad) && aligned16(exp_avg) && aligned16(exp_avg_sq);
#define LDIST_LAUNCH(MODE)                                                                                         \
    do {                                                                                                           \
        if (vec)                                                                                                   \
            hipLaunchKernelGGL((adamw_lp_rows_kernel<MODE, 4>), dim3((unsigned)rows), dim3(256), 0, stream, param, \
                               grad, exp_avg, exp_avg_sq, cols, a);                                                \
        else                                                                                                       \
            hipLaunchKernelGGL((adamw_lp_rows_kernel<MODE, 1>), dim3((unsigned)rows), dim3(256), 0, stream, param, \
                               grad, exp_avg, exp_avg_sq, cols, a);                                                \
    } while (0)
    if (mode == kDecayPlain) LDIST_LAUNCH(kDecayPlain);
    else if (mode == kDecayFinite) LDIST_LAUNCH(kDecayFinite);
    else LDIST_LAUNCH(kDecayInf);
#undef LDIST_LAUNCH
    return hipGetLastError();
}

}  // namespace ldist
