// Internal interface between the C ABI (ldist_api.hip) and the kernel files.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace ldist {

struct Problem {
    int B, G, K, NG, HW;  // K = CI/G, NG = CO/G
    int num_cu;           // compute units of the current device
    int device;
};

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

enum class TileChoice { M128N80K2, M128N64K1, M256N32K1, M32N32K8 };

// Picks the workgroup tiling that leaves the fewest padded (m,n) cells per CU.
// M128N80K2 (512 lanes, two k-groups) fills a CU with one workgroup and divides
// 512 x 5120 into exactly 256 tiles; M128N64K1 is the general shape;
// M256N32K1 serves grouped layers with few outputs per group.
// M32N32K8 (512 lanes, eight k-groups of one wave, 4x4 values per lane) is for few rows and outputs with
// a long reduction (the first fully connected layer behind a conv stack: 128 x 1024 outputs, K = 49152):
// it makes 80 times more workgroups than the big tiles, at twice their LDS traffic per difference.
// -1 = choose by shape; 0, 1, 2, 3 force M128N80K2, M128N64K1, M256N32K1, M32N32K8 (tests and tuning), which also
// keeps the L_inf forward of the unfolded-conv layout on the tiled kernels instead of the short-reduction kernel.
// 4 forces the 64 x 80 tiles that the L_inf forward of a fully connected layer runs two workgroups per CU with
// (inf_forward.hip; by itself it takes them where M128N80K2 would be chosen) and leaves every other kernel's choice alone.
extern int g_tile_override;
extern int g_xcd_remap;  // 1 (default): XCD-aware tile order; 0: plain order (tuning)

inline TileChoice choose_tile(int M, int NG, int G, int num_cu) {
    if (g_tile_override >= 0 && g_tile_override <= 3) return static_cast<TileChoice>(g_tile_override);
    struct Cand { TileChoice c; int bm, bn; bool two_groups; double price; };
    const Cand cands[4] = {{TileChoice::M128N80K2, 128, 80, true, 1.0},
                           {TileChoice::M128N64K1, 128, 64, false, 1.0},
                           {TileChoice::M256N32K1, 256, 32, false, 1.0},
                           {TileChoice::M32N32K8, 32, 32, true, 1.6}};   // a cell of the small tile costs more
    double best = 1e300;
    TileChoice pick = TileChoice::M128N64K1;
    for (const Cand& c : cands) {
        const long tiles = (long)((M + c.bm - 1) / c.bm) * ((NG + c.bn - 1) / c.bn) * G;
        const long rounds = (tiles + num_cu - 1) / num_cu;
        double cost = (double)rounds * c.bm * c.bn * c.price;
        // a lone single-group workgroup leaves one wave per SIMD: latency shows
        if (!c.two_groups && tiles < 2L * num_cu) cost *= 1.25;
        if (cost < best) { best = cost; pick = c.c; }
    }
    return pick;
}

// Sets the dynamic-LDS limit of a kernel once per device.  `done` is the caller's record for that one
// kernel (a function-local static of the launcher instantiated per kernel): kernels share their
// function-pointer type, so a record kept here per type would be shared between them.
// The entry points may be called from several threads at once (a forward thread and autograd's backward thread):
// the record is atomic, and two threads that both find it unset both set the attribute, which is harmless.
using LdsRecord = std::atomic<bool>[64];
template <class Kern>
inline hipError_t allow_lds(Kern kern, size_t bytes, int device, LdsRecord& done) {
    if (device >= 0 && device < 64 && done[device].load(std::memory_order_acquire)) return hipSuccess;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e == hipSuccess && device >= 0 && device < 64) done[device].store(true, std::memory_order_release);
    return e;
}

hipError_t inf_forward(const float* input, const float* weight, float* output, int32_t* pos, const Problem& pr,
                       hipStream_t stream);
// Values without pos, for forward passes that no gradient follows (inf_forward.hip); the fc layout with 128-bit loads.
bool inf_forward_values_applicable(const Problem& pr, const void* input, const void* weight);
hipError_t inf_forward_values(const float* input, const float* weight, float* output, const Problem& pr,
                              hipStream_t stream);
bool inf_forward_shortk_applicable(const Problem& pr, const void* input, const void* output, const void* pos);
hipError_t inf_forward_shortk(const float* input, const float* weight, float* output, int32_t* pos, const Problem& pr,
                              hipStream_t stream);
hipError_t value_bound_forward(const float* input, const float* lower, const float* upper, const float* weight,
                               const float* mean, const float* bias, float* out, float* out_lower, float* out_upper,
                               const Problem& pr, hipStream_t stream);
hipError_t bound_forward(const float* lower, const float* upper, const float* weight, float* out_lower,
                         float* out_upper, const Problem& pr, hipStream_t stream);
// Both L_inf scatters, each gradient written whole; one launch where the layout allows (inf_backward.hip).
hipError_t inf_backward_both(const float* grad_output, const int32_t* pos, float* grad_input, float* grad_weight,
                             const Problem& pr, hipStream_t stream);
hipError_t inf_backward_input(const float* grad_output, const int32_t* pos, float* grad_input, const Problem& pr,
                              bool overwrite, hipStream_t stream);
hipError_t inf_backward_weight(const float* grad_output, const int32_t* pos, float* grad_weight, const Problem& pr,
                               bool overwrite, hipStream_t stream);
hipError_t norm_forward(const float* input, const float* weight, float* output, float p, const Problem& pr,
                        hipStream_t stream);
hipError_t norm_backward_input(const float* grad_output, const float* input, const float* weight,
                               const float* output, float* grad_input, float p, const Problem& pr,
                               hipStream_t stream);
bool norm_backward_input_tiled_applicable(const Problem& pr, float p, const void* grad_output, const void* input,
                                          const void* weight, const void* output, const void* grad_input);
hipError_t norm_backward_input_tiled(const float* grad_output, const float* input, const float* weight,
                                     const float* output, float* grad_input, float p, const Problem& pr,
                                     hipStream_t stream);
bool norm_backward_weight_tiled_applicable(const Problem& pr, float p, const void* grad_output, const void* input,
                                           const void* weight, const void* output, const void* grad_weight);
hipError_t norm_backward_weight_tiled(const float* grad_output, const float* input, const float* weight,
                                      const float* output, float* grad_weight, float p, const Problem& pr,
                                      hipStream_t stream);
hipError_t norm_backward_weight(const float* grad_output, const float* input, const float* weight,
                                const float* output, float* grad_weight, float p, const Problem& pr,
                                hipStream_t stream);

hipError_t mean_shift(const float* x, float* y, float* mean_out, float* running_mean, float momentum, int B, int C,
                      int L, hipStream_t stream);

hipError_t adamw_lp_step(float* param, const float* grad, float* exp_avg, float* exp_avg_sq, int rows, int cols,
                         double p_norm, double lr, double beta1, double beta2, double eps, double weight_decay, int step,
                         hipStream_t stream);

// Geometry of a convolution-shaped layer working on an image tensor (B, C, H, W).
struct ConvGeom {
    int B, C, H, W;        // image
    int KH, KW, S, P, D;   // window, stride, padding, dilation
    int HO, WO;            // output positions
};
hipError_t unfold(const float* img, float* cols, const ConvGeom& q, hipStream_t stream);
hipError_t fold(const float* gcols, float* gimg, const ConvGeom& q, hipStream_t stream);
// L_inf forward straight from the image (3x3 window, dilation 1, stride 1 or 2; a group's channels
// either few enough to stay in LDS or a multiple of four); inf_conv_forward_supported tells whether a geometry is covered.
// Both p-norm gradients in one pass over the terms (norm_backward_fused.hip; the fc layout).
bool norm_backward_fused_applicable(const Problem& pr, float p, const void* grad_output, const void* input,
                                    const void* weight, const void* output, const void* grad_input,
                                    const void* grad_weight);
hipError_t norm_backward_fused(const float* grad_output, const float* input, const float* weight, const float* output,
                               float* grad_input, float* grad_weight, float p, const Problem& pr, hipStream_t stream);
// Both p-norm gradients of a convolution-shaped layer in one pass (norm_conv_backward.hip), from the unfolded
// input or from the image.
bool norm_conv_backward_fused_applicable(const Problem& pr);
bool norm_conv_backward_fused_image_applicable(const ConvGeom& q, int G, int CO, int num_cu);
hipError_t norm_conv_backward_fused_columns(const float* grad_output, const float* input, const float* weight,
                                            const float* output, float* grad_input, float* grad_weight, float p,
                                            const Problem& pr, hipStream_t stream);
hipError_t norm_conv_backward_fused_image(const float* grad_output, const float* img, const float* weight,
                                          const float* output, float* grad_img, float* grad_weight, float p,
                                          const ConvGeom& q, int G, int CO, int num_cu, int device, hipStream_t stream);
// p-norm layer of convolution shape straight from the image (norm_conv.hip): 3x3 windows, more than one output
// position; norm_conv_supported tells whether a geometry is covered.
bool norm_conv_supported(const ConvGeom& q, int G, int CO);
hipError_t norm_conv_forward(const float* img, const float* weight, float* output, float p, const ConvGeom& q, int G,
                             int CO, int num_cu, int device, hipStream_t stream);
hipError_t norm_conv_backward_input(const float* grad_output, const float* img, const float* weight,
                                    const float* output, float* grad_img, float p, const ConvGeom& q, int G, int CO,
                                    int num_cu, int device, hipStream_t stream);
hipError_t norm_conv_backward_weight(const float* grad_output, const float* img, const float* weight,
                                     const float* output, float* grad_weight, float p, const ConvGeom& q, int G, int CO,
                                     int num_cu, int device, hipStream_t stream);
extern int g_conv_rows_override;
extern int g_conv_staging_override;
bool inf_conv_forward_supported(const ConvGeom& q, int G, int CO);
hipError_t inf_conv_forward(const float* img, const float* weight, float* out, int32_t* pos, const ConvGeom& q, int G,
                            int CO, int device, hipStream_t stream);
// Interval-bound forward straight from the lower and upper images (same geometries; channels always staged).
bool bound_conv_forward_supported(const ConvGeom& q, int G, int CO);
hipError_t bound_conv_forward(const float* lower, const float* upper, const float* weight, float* out_lower,
                              float* out_upper, const ConvGeom& q, int G, int CO, int device, hipStream_t stream);
hipError_t inf_backward_input_folded(const float* grad_output, const int32_t* pos, float* grad_img, const ConvGeom& q,
                                     int G, int CO, hipStream_t stream);

}  // namespace ldist
