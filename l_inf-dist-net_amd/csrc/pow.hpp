// v^e for v >= 0 on the transcendental unit, and exact small integer powers.
#pragma once
#include <hip/hip_runtime.h>

namespace ldist {

// exp2(e * log2(v)): v_log_f32, v_mul_f32, v_exp_f32.  v == 0 gives exp2(-inf) = 0
// for e > 0.  Both hardware functions are accurate to about one ulp; the product
// e * log2(v) carries a relative error of about 1e-7, so terms that still matter
// to a sum (|e * log2 v| < 30) come out with a relative error of a few 1e-6.
__device__ __forceinline__ float pow_pos(float v, float e) {
    return __builtin_amdgcn_exp2f(e * __builtin_amdgcn_logf(v));
}

// Keeps a wave-uniform factor in a vector register.  As a scalar-register operand it turns v_mul_f32 into a form that
// issues at little more than half the rate (measured: 4.2 against 2.4 clocks per wave instruction at two waves per
// SIMD), and the exponent multiplies every term.
__device__ __forceinline__ float in_vgpr(float e) {
    asm volatile("" : "+v"(e));
    return e;
}

// sign(u) * |u|^e written as u * |u|^(e-1), em1 = e - 1 > 0: the sign comes with the last multiplication (one plain
// v_mul_f32) instead of a v_bfi_b32 with a scalar mask (4.4 clocks).  u == 0: exp2(-inf) = 0 and 0 * 0 = 0.  em1 must
// be positive (p > 2 for a gradient), or u == 0 would multiply 0 by infinity.
__device__ __forceinline__ float spow_by_mul(float u, float em1) {
    return u * __builtin_amdgcn_exp2f(em1 * __builtin_amdgcn_logf(__builtin_fabsf(u)));
}

// v^N by repeated multiplication; N is a compile-time constant.
template <int N>
__device__ __forceinline__ float pow_int(float v) {
    if constexpr (N == 1) return v;
    else if constexpr (N % 2 == 0) { const float h = pow_int<N / 2>(v); return h * h; }
    else return v * pow_int<N - 1>(v);
}

// Integer exponents that get a multiply-only inner loop (others use pow_pos).
__host__ __device__ inline int small_int_power(float e) {
    const int i = (int)e;
    if ((float)i != e) return 0;
    return (i == 1 || i == 2 || i == 3 || i == 4 || i == 7 || i == 8) ? i : 0;
}

}  // namespace ldist
