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
