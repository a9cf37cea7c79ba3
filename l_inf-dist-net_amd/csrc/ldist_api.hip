// C ABI of libldist_hip.so (declared in include/ldist.h): argument checks, device
// lookup and error mapping around the kernel launchers.  Nothing here allocates
// device memory or synchronises; every call only enqueues work on `stream`.
#include "../../include/ldist.h"

#include <atomic>
#include <cmath>
#include <string>

#include "kernels.hpp"

namespace ldist {
int g_tile_override = -1;
int g_xcd_remap = 1;
}

namespace {

thread_local int g_last_hip_error = 0;

// Compute-unit count and architecture of the current device, looked up once per device and kept in one atomic word
// per device (0 = not looked up yet, else num_cu << 1 | is_gfx950): callers may come from several threads.
int current_device(ldist::Problem& pr) {
    static std::atomic<int> info[64] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { g_last_hip_error = (int)e; return LDIST_ELAUNCH; }
    int word = (dev >= 0 && dev < 64) ? info[dev].load(std::memory_order_acquire) : 0;
    if (word == 0) {
        hipDeviceProp_t prop;
        e = hipGetDeviceProperties(&prop, dev);
        if (e != hipSuccess) { g_last_hip_error = (int)e; return LDIST_ELAUNCH; }
        const int num_cu = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
        word = (num_cu << 1) | (std::string(prop.gcnArchName).rfind("gfx950", 0) == 0 ? 1 : 0);
        if (dev >= 0 && dev < 64) info[dev].store(word, std::memory_order_release);
    }
    if (!(word & 1)) return LDIST_EDEVICE;
    pr.num_cu = word >> 1;
    pr.device = dev;
    return LDIST_OK;
}

int check_dims(int B, int CO, int CI, int G, int HW, ldist::Problem& pr) {
    if (B <= 0 || CO <= 0 || CI <= 0 || G <= 0 || HW <= 0) return LDIST_EINVAL;
    if (CI % G != 0 || CO % G != 0) return LDIST_EINVAL;
    const long long lim = 1LL << 31;
    const long long rows = (long long)B * HW;
    if (rows >= lim || rows * CI >= lim || rows * CO >= lim || (long long)CO * (CI / G) >= lim) return LDIST_ERANGE;
    pr.B = B; pr.G = G; pr.K = CI / G; pr.NG = CO / G; pr.HW = HW;
    return current_device(pr);
}

int finish(hipError_t e) {
    if (e == hipSuccess) return LDIST_OK;
    g_last_hip_error = (int)e;
    return LDIST_ELAUNCH;
}

bool valid_p(float p) { return p > 1.0f && std::isfinite(p); }

// Fills q from the image and window sizes; the number of output positions follows torch's unfold.
int conv_geometry(int B, int C, int H, int W, int KH, int KW, int stride, int padding, int dilation, ldist::ConvGeom& q) {
    if (B <= 0 || C <= 0 || H <= 0 || W <= 0 || KH <= 0 || KW <= 0 || stride <= 0 || padding < 0 || dilation <= 0)
        return LDIST_EINVAL;
    const long long ho = ((long long)H + 2LL * padding - (long long)dilation * (KH - 1) - 1) / stride + 1;
    const long long wo = ((long long)W + 2LL * padding - (long long)dilation * (KW - 1) - 1) / stride + 1;
    if ((long long)H + 2LL * padding < (long long)dilation * (KH - 1) + 1 ||
        (long long)W + 2LL * padding < (long long)dilation * (KW - 1) + 1)
        return LDIST_EINVAL;   // the window does not fit the padded image
    const long long lim = 1LL << 31;
    if ((long long)B * C * H * W >= lim || (long long)B * C * KH * KW * ho * wo >= lim) return LDIST_ERANGE;
    q = ldist::ConvGeom{B, C, H, W, KH, KW, stride, padding, dilation, (int)ho, (int)wo};
    return LDIST_OK;
}

}  // namespace

extern "C" {

int ldist_version(void) { return LDIST_VERSION; }

const char* ldist_strerror(int code) {
    switch (code) {
        case LDIST_OK: return "ok";
        case LDIST_EINVAL: return "invalid argument (null pointer, non-positive size, CI % G or CO % G != 0, or p not > 1)";
        case LDIST_ERANGE: return "tensor too large (2^31 or more elements)";
        case LDIST_ELAUNCH: return "HIP runtime error at launch";
        case LDIST_EDEVICE: return "current device is not gfx950";
        case LDIST_EUNSUPPORTED: return "this entry point does not cover the geometry (use the general path)";
        default: return "unknown error";
    }
}

int ldist_last_hip_error(void) { return g_last_hip_error; }

int ldist_set_xcd_remap(int on) {
    ldist::g_xcd_remap = on ? 1 : 0;
    return LDIST_OK;
}

int ldist_set_tile_override(int choice) {
    if (choice < -1 || choice > 5) return LDIST_EINVAL;
    ldist::g_tile_override = choice;
    return LDIST_OK;
}

int ldist_inf_dist_forward(const float* input, const float* weight, int B, int CO, int CI, int G, int HW,
                           float* output, int32_t* pos, ldist_stream_t stream) {
    if (!input || !weight || !output || !pos) return LDIST_EINVAL;
    ldist::Problem pr{};
    if (int rc = check_dims(B, CO, CI, G, HW, pr)) return rc;
    return finish(ldist::inf_forward(input, weight, output, pos, pr, (hipStream_t)stream));
}

int ldist_inf_dist_forward_values(const float* input, const float* weight, int B, int CO, int CI, int G, int HW,
                                  float* output, ldist_stream_t stream) {
    if (!input || !weight || !output) return LDIST_EINVAL;
    ldist::Problem pr{};
    if (int rc = check_dims(B, CO, CI, G, HW, pr)) return rc;
    if (!ldist::inf_forward_values_applicable(pr, input, weight)) return LDIST_EUNSUPPORTED;
    return finish(ldist::inf_forward_values(input, weight, output, pr, (hipStream_t)stream));
}

int ldist_inf_dist_bound_forward(const float* input_lower, const float* input_upper, const float* weight, int B,
                                 int CO, int CI, int G, int HW, float* output_lower, float* output_upper,
                                 ldist_stream_t stream) {
    if (!input_lower || !input_upper || !weight || !output_lower || !output_upper) return LDIST_EINVAL;
    ldist::Problem pr{};
    if (int rc = check_dims(B, CO, CI, G, HW, pr)) return rc;
    return finish(ldist::bound_forward(input_lower, input_upper, weight, output_lower, output_upper, pr,
                                       (hipStream_t)stream));
}

int ldist_inf_dist_value_bound_forward(const float* input, const float* input_lower, const float* input_upper,
                                       const float* weight, int B, int CO, int CI, int G, int HW, const float* mean,
                                       const float* bias, float* output, float* output_lower, float* output_upper,
                                       ldist_stream_t stream) {
    if (!input || !input_lower || !input_upper || !weight || !output || !output_lower || !output_upper)
        return LDIST_EINVAL;
    ldist::Problem pr{};
    if (int rc = check_dims(B, CO, CI, G, HW, pr)) return rc;
    return finish(ldist::value_bound_forward(input, input_lower, input_upper, weight, mean, bias, output, output_lower,
                                             output_upper, pr, (hipStream_t)stream));
}

static int inf_backward_input_impl(const float* grad_output, const int32_t* pos, int B, int CO, int CI, int G,
                                   int HW, float* grad_input, bool overwrite, ldist_stream_t stream) {
    if (!grad_output || !pos || !grad_input) return LDIST_EINVAL;
    ldist::Problem pr{};
    if (int rc = check_dims(B, CO, CI, G, HW, pr)) return rc;
    return finish(ldist::inf_backward_input(grad_output, pos, grad_input, pr, overwrite, (hipStream_t)stream));
}

static int inf_backward_weight_impl(const float* grad_output, const int32_t* pos, int B, int CO, int CI, int G,
                                    int HW, float* grad_weight, bool overwrite, ldist_stream_t stream) {
    if (!grad_output || !pos || !grad_weight) return LDIST_EINVAL;
    ldist::Problem pr{};
    if (int rc = check_dims(B, CO, CI, G, HW, pr)) return rc;
    return finish(ldist::inf_backward_weight(grad_output, pos, grad_weight, pr, overwrite, (hipStream_t)stream));
}

int ldist_inf_dist_backward_input(const float* grad_output, const int32_t* pos, int B, int CO, int CI, int G, int HW,
                                  float* grad_input, ldist_stream_t stream) {
    return inf_backward_input_impl(grad_output, pos, B, CO, CI, G, HW, grad_input, false, stream);
}

int ldist_inf_dist_backward_weight(const float* grad_output, const int32_t* pos, int B, int CO, int CI, int G, int HW,
                                   float* grad_weight, ldist_stream_t stream) {
    return inf_backward_weight_impl(grad_output, pos, B, CO, CI, G, HW, grad_weight, false, stream);
}

int ldist_inf_dist_backward_input_overwrite(const float* grad_output, const int32_t* pos, int B, int CO, int CI,
                                            int G, int HW, float* grad_input, ldist_stream_t stream) {
    return inf_backward_input_impl(grad_output, pos, B, CO, CI, G, HW, grad_input, true, stream);
}

int ldist_inf_dist_backward_weight_overwrite(const float* grad_output, const int32_t* pos, int B, int CO, int CI,
                                             int G, int HW, float* grad_weight, ldist_stream_t stream) {
    return inf_backward_weight_impl(grad_output, pos, B, CO, CI, G, HW, grad_weight, true, stream);
}

int ldist_inf_dist_backward_overwrite(const float* grad_output, const int32_t* pos, int B, int CO, int CI, int G, int HW,
                                      float* grad_input, float* grad_weight, ldist_stream_t stream) {
    if (!grad_output || !pos || !grad_input || !grad_weight) return LDIST_EINVAL;
    ldist::Problem pr{};
    if (int rc = check_dims(B, CO, CI, G, HW, pr)) return rc;
    return finish(ldist::inf_backward_both(grad_output, pos, grad_input, grad_weight, pr, (hipStream_t)stream));
}

int ldist_norm_dist_forward(const float* input, const float* weight, int B, int CO, int CI, int G, int HW,
                            float* output, float p, ldist_stream_t stream) {
    if (!input || !weight || !output || !valid_p(p)) return LDIST_EINVAL;
    ldist::Problem pr{};
    if (int rc = check_dims(B, CO, CI, G, HW, pr)) return rc;
    return finish(ldist::norm_forward(input, weight, output, p, pr, (hipStream_t)stream));
}

int ldist_norm_dist_backward_input(const float* grad_output, const float* input, const float* weight,
                                   const float* output, int B, int CO, int CI, int G, int HW, float* grad_input,
                                   float p, ldist_stream_t stream) {
    if (!grad_output || !input || !weight || !output || !grad_input || !valid_p(p)) return LDIST_EINVAL;
    ldist::Problem pr{};
    if (int rc = check_dims(B, CO, CI, G, HW, pr)) return rc;
    return finish(ldist::norm_backward_input(grad_output, input, weight, output, grad_input, p, pr,
                                             (hipStream_t)stream));
}

int ldist_norm_dist_backward_weight(const float* grad_output, const float* input, const float* weight,
                                    const float* output, int B, int CO, int CI, int G, int HW, float* grad_weight,
                                    float p, ldist_stream_t stream) {
    if (!grad_output || !input || !weight || !output || !grad_weight || !valid_p(p)) return LDIST_EINVAL;
    ldist::Problem pr{};
    if (int rc = check_dims(B, CO, CI, G, HW, pr)) return rc;
    return finish(ldist::norm_backward_weight(grad_output, input, weight, output, grad_weight, p, pr,
                                              (hipStream_t)stream));
}

int ldist_norm_dist_backward(const float* grad_output, const float* input, const float* weight, const float* output,
                             int B, int CO, int CI, int G, int HW, float* grad_input, float* grad_weight, float p,
                             ldist_stream_t stream) {
    if (!grad_output || !input || !weight || !output || !grad_input || !grad_weight || !valid_p(p)) return LDIST_EINVAL;
    ldist::Problem pr{};
    if (int rc = check_dims(B, CO, CI, G, HW, pr)) return rc;
    if (ldist::norm_backward_fused_applicable(pr, p, grad_output, input, weight, output, grad_input, grad_weight))
        return finish(ldist::norm_backward_fused(grad_output, input, weight, output, grad_input, grad_weight, p, pr,
                                                 (hipStream_t)stream));
    if (ldist::norm_conv_backward_fused_applicable(pr))
        return finish(ldist::norm_conv_backward_fused_columns(grad_output, input, weight, output, grad_input, grad_weight,
                                                              p, pr, (hipStream_t)stream));
    if (hipError_t e = ldist::norm_backward_input(grad_output, input, weight, output, grad_input, p, pr, (hipStream_t)stream);
        e != hipSuccess)
        return finish(e);
    return finish(ldist::norm_backward_weight(grad_output, input, weight, output, grad_weight, p, pr,
                                              (hipStream_t)stream));
}

int ldist_mean_shift(const float* x, int B, int C, int L, float* y, float* mean_out, float* running_mean,
                     float momentum, ldist_stream_t stream) {
    if (!x || !y || B <= 0 || C <= 0 || L <= 0 || !(momentum >= 0.0f && momentum <= 1.0f)) return LDIST_EINVAL;
    if ((long long)B * C * L >= (1LL << 31)) return LDIST_ERANGE;
    ldist::Problem pr{};
    if (int rc = current_device(pr)) return rc;
    return finish(ldist::mean_shift(x, y, mean_out, running_mean, momentum, B, C, L, (hipStream_t)stream));
}

int ldist_adamw_lp_step(float* param, const float* grad, float* exp_avg, float* exp_avg_sq, int rows, int cols,
                        double p_norm, double lr, double beta1, double beta2, double eps, double weight_decay, int step,
                        ldist_stream_t stream) {
    if (!param || rows <= 0 || cols <= 0 || step < 1) return LDIST_EINVAL;
    if (grad && (!exp_avg || !exp_avg_sq)) return LDIST_EINVAL;
    if (!(lr >= 0.0) || !(eps >= 0.0) || !(weight_decay >= 0.0) || !(beta1 >= 0.0 && beta1 < 1.0) ||
        !(beta2 >= 0.0 && beta2 < 1.0))
        return LDIST_EINVAL;   // the reference constructor's checks, adamw.py:15-24
    if ((long long)rows * cols >= (1LL << 31)) return LDIST_ERANGE;
    ldist::Problem pr{};
    if (int rc = current_device(pr)) return rc;
    return finish(ldist::adamw_lp_step(param, grad, exp_avg, exp_avg_sq, rows, cols, p_norm, lr, beta1, beta2, eps,
                                       weight_decay, step, (hipStream_t)stream));
}

int ldist_unfold(const float* img, int B, int C, int H, int W, int KH, int KW, int stride, int padding, int dilation,
                 float* cols, ldist_stream_t stream) {
    ldist::ConvGeom q{};
    if (!img || !cols) return LDIST_EINVAL;
    if (int rc = conv_geometry(B, C, H, W, KH, KW, stride, padding, dilation, q)) return rc;
    ldist::Problem pr{};
    if (int rc = current_device(pr)) return rc;
    return finish(ldist::unfold(img, cols, q, (hipStream_t)stream));
}

int ldist_inf_dist_conv_forward_supported(int C, int H, int W, int CO, int G, int KH, int KW, int stride, int padding,
                                          int dilation) {
    ldist::ConvGeom q{};
    if (CO <= 0 || G <= 0) return 0;
    if (conv_geometry(1, C, H, W, KH, KW, stride, padding, dilation, q) != LDIST_OK) return 0;
    return ldist::inf_conv_forward_supported(q, G, CO) ? 1 : 0;
}

// pos == nullptr: values only
static int inf_conv_forward_entry(const float* img, const float* weight, int B, int C, int H, int W, int CO, int G,
                                  int KH, int KW, int stride, int padding, int dilation, float* output, int32_t* pos,
                                  ldist_stream_t stream) {
    ldist::ConvGeom q{};
    if (!img || !weight || !output || CO <= 0 || G <= 0) return LDIST_EINVAL;
    if (int rc = conv_geometry(B, C, H, W, KH, KW, stride, padding, dilation, q)) return rc;
    if (C % G != 0 || CO % G != 0) return LDIST_EINVAL;
    if ((long long)B * CO * q.HO * q.WO >= (1LL << 31) || (long long)CO * (C / G) * KH * KW >= (1LL << 31))
        return LDIST_ERANGE;
    if (!ldist::inf_conv_forward_supported(q, G, CO)) return LDIST_EUNSUPPORTED;
    ldist::Problem pr{};
    if (int rc = current_device(pr)) return rc;
    return finish(ldist::inf_conv_forward(img, weight, output, pos, q, G, CO, pr.device, (hipStream_t)stream));
}

int ldist_inf_dist_conv_forward(const float* img, const float* weight, int B, int C, int H, int W, int CO, int G,
                                int KH, int KW, int stride, int padding, int dilation, float* output, int32_t* pos,
                                ldist_stream_t stream) {
    if (!pos) return LDIST_EINVAL;
    return inf_conv_forward_entry(img, weight, B, C, H, W, CO, G, KH, KW, stride, padding, dilation, output, pos, stream);
}

int ldist_inf_dist_conv_forward_values(const float* img, const float* weight, int B, int C, int H, int W, int CO, int G,
                                       int KH, int KW, int stride, int padding, int dilation, float* output,
                                       ldist_stream_t stream) {
    return inf_conv_forward_entry(img, weight, B, C, H, W, CO, G, KH, KW, stride, padding, dilation, output, nullptr,
                                  stream);
}

int ldist_inf_dist_bound_conv_forward_supported(int C, int H, int W, int CO, int G, int KH, int KW, int stride,
                                                int padding, int dilation) {
    ldist::ConvGeom q{};
    if (CO <= 0 || G <= 0) return 0;
    if (conv_geometry(1, C, H, W, KH, KW, stride, padding, dilation, q) != LDIST_OK) return 0;
    return ldist::bound_conv_forward_supported(q, G, CO) ? 1 : 0;
}

int ldist_inf_dist_bound_conv_forward(const float* lower_img, const float* upper_img, const float* weight, int B, int C,
                                      int H, int W, int CO, int G, int KH, int KW, int stride, int padding,
                                      int dilation, float* output_lower, float* output_upper, ldist_stream_t stream) {
    ldist::ConvGeom q{};
    if (!lower_img || !upper_img || !weight || !output_lower || !output_upper || CO <= 0 || G <= 0) return LDIST_EINVAL;
    if (int rc = conv_geometry(B, C, H, W, KH, KW, stride, padding, dilation, q)) return rc;
    if (C % G != 0 || CO % G != 0) return LDIST_EINVAL;
    if ((long long)B * CO * q.HO * q.WO >= (1LL << 31) || (long long)CO * (C / G) * KH * KW >= (1LL << 31))
        return LDIST_ERANGE;
    if (!ldist::bound_conv_forward_supported(q, G, CO)) return LDIST_EUNSUPPORTED;
    ldist::Problem pr{};
    if (int rc = current_device(pr)) return rc;
    return finish(ldist::bound_conv_forward(lower_img, upper_img, weight, output_lower, output_upper, q, G, CO,
                                            pr.device, (hipStream_t)stream));
}

int ldist_norm_dist_conv_supported(int C, int H, int W, int CO, int G, int KH, int KW, int stride, int padding,
                                   int dilation) {
    ldist::ConvGeom q{};
    if (CO <= 0 || G <= 0) return 0;
    if (conv_geometry(1, C, H, W, KH, KW, stride, padding, dilation, q) != LDIST_OK) return 0;
    return ldist::norm_conv_supported(q, G, CO) ? 1 : 0;
}

namespace {
// Shared argument checks of the three p-norm entry points that read the image.
int norm_conv_prepare(int B, int C, int H, int W, int CO, int G, int KH, int KW, int stride, int padding, int dilation,
                      float p, ldist::ConvGeom& q, ldist::Problem& pr) {
    if (CO <= 0 || G <= 0 || !valid_p(p)) return LDIST_EINVAL;
    if (int rc = conv_geometry(B, C, H, W, KH, KW, stride, padding, dilation, q)) return rc;
    if (C % G != 0 || CO % G != 0) return LDIST_EINVAL;
    if ((long long)B * CO * q.HO * q.WO >= (1LL << 31) || (long long)CO * (C / G) * KH * KW >= (1LL << 31))
        return LDIST_ERANGE;
    if (!ldist::norm_conv_supported(q, G, CO)) return LDIST_EUNSUPPORTED;
    return current_device(pr);
}
}  // namespace

int ldist_norm_dist_conv_forward(const float* img, const float* weight, int B, int C, int H, int W, int CO, int G, int KH,
                                 int KW, int stride, int padding, int dilation, float* output, float p,
                                 ldist_stream_t stream) {
    ldist::ConvGeom q{};
    ldist::Problem pr{};
    if (!img || !weight || !output) return LDIST_EINVAL;
    if (int rc = norm_conv_prepare(B, C, H, W, CO, G, KH, KW, stride, padding, dilation, p, q, pr)) return rc;
    return finish(ldist::norm_conv_forward(img, weight, output, p, q, G, CO, pr.num_cu, pr.device, (hipStream_t)stream));
}

int ldist_norm_dist_conv_backward_input(const float* grad_output, const float* img, const float* weight,
                                        const float* output, int B, int C, int H, int W, int CO, int G, int KH, int KW,
                                        int stride, int padding, int dilation, float* grad_img, float p,
                                        ldist_stream_t stream) {
    ldist::ConvGeom q{};
    ldist::Problem pr{};
    if (!grad_output || !img || !weight || !output || !grad_img) return LDIST_EINVAL;
    if (int rc = norm_conv_prepare(B, C, H, W, CO, G, KH, KW, stride, padding, dilation, p, q, pr)) return rc;
    return finish(ldist::norm_conv_backward_input(grad_output, img, weight, output, grad_img, p, q, G, CO, pr.num_cu,
                                                  pr.device, (hipStream_t)stream));
}

int ldist_norm_dist_conv_backward_weight(const float* grad_output, const float* img, const float* weight,
                                         const float* output, int B, int C, int H, int W, int CO, int G, int KH, int KW,
                                         int stride, int padding, int dilation, float* grad_weight, float p,
                                         ldist_stream_t stream) {
    ldist::ConvGeom q{};
    ldist::Problem pr{};
    if (!grad_output || !img || !weight || !output || !grad_weight) return LDIST_EINVAL;
    if (int rc = norm_conv_prepare(B, C, H, W, CO, G, KH, KW, stride, padding, dilation, p, q, pr)) return rc;
    return finish(ldist::norm_conv_backward_weight(grad_output, img, weight, output, grad_weight, p, q, G, CO, pr.num_cu,
                                                   pr.device, (hipStream_t)stream));
}

int ldist_norm_dist_conv_backward(const float* grad_output, const float* img, const float* weight, const float* output,
                                  int B, int C, int H, int W, int CO, int G, int KH, int KW, int stride, int padding,
                                  int dilation, float* grad_img, float* grad_weight, float p, ldist_stream_t stream) {
    ldist::ConvGeom q{};
    ldist::Problem pr{};
    if (!grad_output || !img || !weight || !output || !grad_img || !grad_weight) return LDIST_EINVAL;
    if (int rc = norm_conv_prepare(B, C, H, W, CO, G, KH, KW, stride, padding, dilation, p, q, pr)) return rc;
    if (ldist::norm_conv_backward_fused_image_applicable(q, G, CO, pr.num_cu))
        return finish(ldist::norm_conv_backward_fused_image(grad_output, img, weight, output, grad_img, grad_weight, p, q,
                                                            G, CO, pr.num_cu, pr.device, (hipStream_t)stream));
    if (hipError_t e = ldist::norm_conv_backward_input(grad_output, img, weight, output, grad_img, p, q, G, CO, pr.num_cu,
                                                       pr.device, (hipStream_t)stream);
        e != hipSuccess)
        return finish(e);
    return finish(ldist::norm_conv_backward_weight(grad_output, img, weight, output, grad_weight, p, q, G, CO, pr.num_cu,
                                                   pr.device, (hipStream_t)stream));
}

int ldist_set_conv_staging_override(int mode) {
    if (mode < 0 || mode > 3) return LDIST_EINVAL;
    ldist::g_conv_staging_override = mode;
    return LDIST_OK;
}

int ldist_set_conv_rows_override(int rows) {
    if (rows < 0) return LDIST_EINVAL;
    ldist::g_conv_rows_override = rows;
    return LDIST_OK;
}

int ldist_fold(const float* grad_cols, int B, int C, int H, int W, int KH, int KW, int stride, int padding,
               int dilation, float* grad_img, ldist_stream_t stream) {
    ldist::ConvGeom q{};
    if (!grad_cols || !grad_img) return LDIST_EINVAL;
    if (int rc = conv_geometry(B, C, H, W, KH, KW, stride, padding, dilation, q)) return rc;
    ldist::Problem pr{};
    if (int rc = current_device(pr)) return rc;
    return finish(ldist::fold(grad_cols, grad_img, q, (hipStream_t)stream));
}

int ldist_inf_dist_backward_input_folded(const float* grad_output, const int32_t* pos, int B, int CO, int C, int G,
                                         int H, int W, int KH, int KW, int stride, int padding, int dilation,
                                         float* grad_img, ldist_stream_t stream) {
    ldist::ConvGeom q{};
    if (!grad_output || !pos || !grad_img || CO <= 0 || G <= 0) return LDIST_EINVAL;
    if (int rc = conv_geometry(B, C, H, W, KH, KW, stride, padding, dilation, q)) return rc;
    if (C % G != 0 || CO % G != 0) return LDIST_EINVAL;
    if ((long long)B * CO * q.HO * q.WO >= (1LL << 31)) return LDIST_ERANGE;
    if ((long long)(C / G) * W > 16384) return LDIST_ERANGE;   // one image row of a group must fit the LDS bins
    ldist::Problem pr{};
    if (int rc = current_device(pr)) return rc;
    return finish(ldist::inf_backward_input_folded(grad_output, pos, grad_img, q, G, CO, (hipStream_t)stream));
}

}  // extern "C"
