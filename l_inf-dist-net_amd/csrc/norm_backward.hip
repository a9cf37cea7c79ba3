// p-norm distance backward, p > 1 (reference model/norm_dist_cuda.cu:294-425):
//   grad_input [m,k]  = sum_n g[m,n] * (|x-w| / out[m,n])^(p-1) * sign(x-w)     (:294-297, every element written)
//   grad_weight[n,k] += sum_m g[m,n] * (|w-x| / out[m,n])^(p-1) * sign(w-x)     (:363-366, added to the buffer)
// Both are the same reduction with the roles of x and w exchanged:
//   P[a,k] = sum_r c[a,r] * (|Q[a,k] - O[r,k]| * rinv[a,r])^(p-1) * sign(Q - O)
// grad_input: a = m, r = n, Q = x, O = w;  grad_weight: a = n, r = m, Q = w, O = x.
// A workgroup owns a 64 x 64 tile of P; each lane keeps a 4 x 4 patch of Q and of
// the sums in registers and walks r in stages of 32 whose O, c and rinv panels sit
// in LDS.  The work is bound by the transcendental unit (one v_log_f32 and one
// v_exp_f32 per term; p-1 = 1, 2, 3, 7 use multiplies only), so the loads are
// plain coalesced 32-bit accesses.
#include "norm_backward_kernel.hpp"

namespace ldist {

hipError_t norm_backward_input(const float* grad_output, const float* input, const float* weight,
                               const float* output, float* grad_input, float p, const Problem& pr,
                               hipStream_t stream) {
    if (norm_backward_input_tiled_applicable(pr, p, grad_output, input, weight, output, grad_input))
        return norm_backward_input_tiled(grad_output, input, weight, output, grad_input, p, pr, stream);
    return launch_norm_backward<false, false>(grad_output, input, weight, output, grad_input, p, pr, stream, ImgWin{});
}

hipError_t norm_backward_weight(const float* grad_output, const float* input, const float* weight,
                                const float* output, float* grad_weight, float p, const Problem& pr,
                                hipStream_t stream) {
    if (norm_backward_weight_tiled_applicable(pr, p, grad_output, input, weight, output, grad_weight))
        return norm_backward_weight_tiled(grad_output, input, weight, output, grad_weight, p, pr, stream);
    return launch_norm_backward<true, false>(grad_output, input, weight, output, grad_weight, p, pr, stream, ImgWin{});
}

}  // namespace ldist
