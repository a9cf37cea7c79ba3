// p-norm distance layer of convolution shape straight from the image: forward and both gradients without the
// unfolded tensor.  The reference unfolds for every p (F.unfold at model/norm_dist.py:132, nine times the image for
// a 3x3 window) and runs its column kernels on the result (model/norm_dist_cuda.cu:228-425); autograd then folds
// the gradient of the columns back.  Here the kernels of norm_forward.hip and norm_backward.hip take the image
// itself: wherever they would read column k of row (b, ho, wo) they look up tap k of that window (conv_window.hpp),
// and the gradient with respect to the input is added onto the image pixel a column was read from (columns that
// lie in the padding are dropped, as fold drops them).  Same terms, same order of summation inside a workgroup as
// the column kernels; only the nine partial sums a pixel collects from different columns are added in no fixed
// order (float atomics), which moves a gradient by a few units in the last place from run to run.
//
// A term of these kernels costs 5 to 20 instructions and a loaded value is used by every output of the tile, so
// the index arithmetic of a gathered load (about fifteen instructions) is a few per cent of a stage; the image is
// read nine times over, from L2.
#include "norm_backward_kernel.hpp"
#include "norm_forward_kernel.hpp"

namespace ldist {

namespace {

template <class GEO, bool CONV, int VEC>
struct NormForwardImage {
    static hipError_t launch(unsigned grid, const Dims& d, int device, hipStream_t stream, const float* img,
                             const float* weight, float* output, float p, ImgWin win) {
        if constexpr (CONV) return NormForwardLaunch<GEO, true, VEC, true>::launch(grid, d, device, stream, img, weight, output, p, win);
        else return hipErrorInvalidValue;   // a single output position: norm_conv_supported says no
    }
};

ImgWin window_of(const ConvGeom& q, int G) { return ImgWin{q.C, q.C / G, q.H, q.W, q.HO, q.WO, q.S, q.P, q.D}; }

Problem problem_of(const ConvGeom& q, int G, int CO, int num_cu, int device) {
    return Problem{q.B, G, q.C / G * 9, CO / G, q.HO * q.WO, num_cu, device};
}

__global__ void __launch_bounds__(256) zero_fill_kernel(float* __restrict__ p, size_t n, bool vec) {
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (vec && i + 3 < n) {
        *reinterpret_cast<float4*>(p + i) = make_float4(0.f, 0.f, 0.f, 0.f);
    } else {
        for (size_t j = i; j < n && j < i + 4; j++) p[j] = 0.f;
    }
}

}  // namespace

// 3x3 windows (any stride, padding, dilation) with more than one output position.  Layers with few outputs per
// group, for which the column entry point has a kernel of its own, run on the tiled kernel here.
bool norm_conv_supported(const ConvGeom& q, int G, int CO) {
    if (q.KH != 3 || q.KW != 3) return false;
    if (G <= 0 || q.C % G != 0 || CO % G != 0) return false;
    return (long long)q.HO * q.WO > 1;
}

hipError_t norm_conv_forward(const float* img, const float* weight, float* output, float p, const ConvGeom& q, int G,
                             int CO, int num_cu, int device, hipStream_t stream) {
    const Problem pr = problem_of(q, G, CO, num_cu, device);
    const bool wvec = pr.K % 4 == 0 && aligned16(weight);
    return dispatch_forward<NormForwardImage>(pr, wvec, can_vec4_out(pr, output), stream, img, weight, output, p,
                                              window_of(q, G));
}

// grad_img need not be initialised: it is zero-filled here (by a kernel, so that the call can be captured in a graph).
hipError_t norm_conv_backward_input(const float* grad_output, const float* img, const float* weight,
                                    const float* output, float* grad_img, float p, const ConvGeom& q, int G, int CO,
                                    int num_cu, int device, hipStream_t stream) {
    const Problem pr = problem_of(q, G, CO, num_cu, device);
    const size_t n = (size_t)q.B * q.C * q.H * q.W;
    hipLaunchKernelGGL(zero_fill_kernel, dim3((unsigned)((n + 1023) / 1024)), dim3(256), 0, stream, grad_img, n,
                       aligned16(grad_img));
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    return launch_norm_backward<false, true>(grad_output, img, weight, output, grad_img, p, pr, stream, window_of(q, G));
}

// grad_weight is added to, as in the column entry point.
hipError_t norm_conv_backward_weight(const float* grad_output, const float* img, const float* weight,
                                     const float* output, float* grad_weight, float p, const ConvGeom& q, int G, int CO,
                                     int num_cu, int device, hipStream_t stream) {
    const Problem pr = problem_of(q, G, CO, num_cu, device);
    return launch_norm_backward<true, true>(grad_output, img, weight, output, grad_weight, p, pr, stream, window_of(q, G));
}

}  // namespace ldist
