/*
 * ldist -- L_p / L_inf distance-neuron operators for AMD MI355X (gfx950).
 *
 * C ABI of libldist_hip.so.  Plain pointers and sizes only: every pointer is a
 * DEVICE pointer to float32 / int32 data on the current HIP device, `stream`
 * is a hipStream_t passed as void* (NULL = the default stream).  All calls are
 * asynchronous with respect to the host: they enqueue kernels on `stream` and
 * return.  The library allocates no device memory and never frees or retains
 * the caller's buffers, like the reference launchers (model/norm_dist.py:10-15,
 * 34,37,42,45,63-64 allocate everything in Python).  The only state it keeps
 * between calls is process-wide: the two tuning knobs below, a cache of device
 * properties, and which kernels have had their LDS limit raised on a device.
 *
 * Each of the seven core entry points replaces one `*_cuda` launcher declared
 * in the reference's binding (model/norm_dist.cpp:7-20) and keeps its argument
 * order; `stream` is appended.  As there, CO and CI are totals over all groups.
 *
 * Tensor layout, all contiguous (model/inf_dist_cuda.cu:29-33,65-66):
 *   input   (B, CI, HW)   element ((b*G + g)*K  + k )*HW + hw,   K  = CI/G
 *   weight  (CO, K)       element  (g*NG + n)*K + k,             NG = CO/G
 *   output  (B, CO, HW)   element ((b*G + g)*NG + n )*HW + hw    (also pos, grad_output)
 *
 * Return value: LDIST_OK, or a negative LDIST_E* code.  Nothing is launched
 * when an argument check fails.  No C++ exception crosses this boundary.
 */
#ifndef LDIST_H
#define LDIST_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LDIST_VERSION 100 /* major*10000 + minor*100 + patch */
/* The library is built with hidden visibility; only the entry points below are exported. */
#define LDIST_API __attribute__((visibility("default")))

enum {
    LDIST_OK = 0,
    LDIST_EINVAL = -1,  /* null pointer, non-positive size, CI % G or CO % G non-zero, p <= 1 or NaN */
    LDIST_ERANGE = -2,  /* a tensor has 2^31 or more elements (kernels index with 32 bits) */
    LDIST_ELAUNCH = -3, /* the HIP runtime reported an error at launch (see ldist_last_hip_error) */
    LDIST_EDEVICE = -4, /* the current device is not a gfx950 the library was built for */
    LDIST_EUNSUPPORTED = -5 /* a specialised entry point does not cover this geometry: use the general one */
};

typedef void* ldist_stream_t; /* hipStream_t */

LDIST_API int ldist_version(void);
LDIST_API const char* ldist_strerror(int code);
/* hipError_t of the last failed launch made by the calling thread (0 if none). */
LDIST_API int ldist_last_hip_error(void);

/* Testing and tuning knob, no counterpart in the reference: forces the workgroup
 * tiling of the three forward kernels.  -1 = choose by shape (default), 0 = 128x80
 * tile with two k-groups, 1 = 128x64, 2 = 256x32, 3 = 32x32 with eight k-groups,
 * 4 = 64x80 with two k-groups (two 256-lane workgroups per CU) for the L_inf forward
 * of a fully connected layer with 128-bit loads, the other kernels choosing by shape.
 * 0..4 also keep the L_inf forward of an unfolded-conv layout on the tiled kernels
 * where it would otherwise take the kernel that holds a tile's whole reduction axis
 * in LDS (K up to 320), and 0 / 1 force the register-tiled p-norm backward kernels
 * (128x80 / 128x64 tiles), the one-pass kernel of ldist_norm_dist_backward included,
 * 2 / 3 / 4 keep them off; 5 forces that one-pass kernel on with 128x48 tiles (its third
 * width, which it otherwise takes where the wider ones leave CUs idle) and is like 2
 * for every other kernel.  Process-wide; not thread safe. */
LDIST_API int ldist_set_tile_override(int choice);
/* Tuning knob, no counterpart in the reference: 1 (default) orders the tiles of
 * the forward kernels so that each of the 8 XCDs works on one contiguous run of
 * tiles, 0 keeps the plain order.  Results do not depend on it. */
LDIST_API int ldist_set_xcd_remap(int on);

/* L_inf forward.  Replaces inf_dist_forward_cuda (model/norm_dist.cpp:13-14,
 * model/inf_dist_cuda.cu:173-180).
 *   output[m,n] = max_k |x[m,k] - w[n,k]|
 *   pos[m,n]    = k*, the LOWEST k attaining the maximum, with bit 31 set when
 *                 x[m,k*] - w[n,k*] < 0; 0 when the maximum is 0.
 * A NaN difference never wins.  Values and indices are bit-exact with the
 * reference rule "scan k ascending, update on strict >" (inf_dist_cuda.cu:36-43). */
LDIST_API int ldist_inf_dist_forward(const float* input, const float* weight, int B, int CO, int CI, int G, int HW,
                           float* output, int32_t* pos, ldist_stream_t stream);

/* L_inf forward without pos: output as ldist_inf_dist_forward writes it, bit for bit.  No counterpart in the
 * reference, whose forward always computes pos (model/norm_dist.py:14-15); for forward passes that no gradient
 * follows (evaluation, the value path of a certification pass), which then skip the index bookkeeping and the
 * search for the lowest k.  Covers the fc layout (HW == 1) with more than 16 outputs per group, K a multiple of
 * four and 16-byte aligned tensors; LDIST_EUNSUPPORTED for the rest (nothing is enqueued: call
 * ldist_inf_dist_forward). */
LDIST_API int ldist_inf_dist_forward_values(const float* input, const float* weight, int B, int CO, int CI, int G, int HW,
                                  float* output, ldist_stream_t stream);

/* Interval-bound forward.  Replaces inf_dist_bound_forward_cuda
 * (model/norm_dist.cpp:15-16, model/inf_dist_cuda.cu:181-188).
 *   output_upper = max_k max(|l-w|, |u-w|)
 *   output_lower = max_k min(|l-w|, |u-w|) over the k where not (l-w < 0 < u-w), else 0 */
LDIST_API int ldist_inf_dist_bound_forward(const float* input_lower, const float* input_upper, const float* weight, int B,
                                 int CO, int CI, int G, int HW, float* output_lower, float* output_upper,
                                 ldist_stream_t stream);

/* Values and interval bounds in one pass over the weights: what ldist_inf_dist_forward (without the index)
 * and ldist_inf_dist_bound_forward compute for a point `input` and the box [input_lower, input_upper] around it,
 * bit for bit, followed by the layer's evaluation-mode epilogue.  Replaces the pair of calls certification makes
 * per layer, norm_dist(...) and inf_dist_bound(...) at model/norm_dist.py:134,144-145 (inf_dist_forward_cuda and
 * inf_dist_bound_forward_cuda, model/norm_dist.cpp:13-16), and the shifts after them (:146-155).
 *   mean, bias: (CO) each or NULL; every value v of output channel c leaves as (v - mean[c]) + bias[c], in this
 *   order, the running-mean shift of MeanNorm in evaluation mode and the layer's bias.
 * No index is produced: this path carries no gradient (the reference asserts evaluation mode, :142). */
LDIST_API int ldist_inf_dist_value_bound_forward(const float* input, const float* input_lower, const float* input_upper,
                                       const float* weight, int B, int CO, int CI, int G, int HW, const float* mean,
                                       const float* bias, float* output, float* output_lower, float* output_upper,
                                       ldist_stream_t stream);

/* L_inf backward w.r.t. input.  Replaces inf_dist_backward_input_cuda
 * (model/norm_dist.cpp:17-18, model/inf_dist_cuda.cu:189-196).
 *   grad_input[b, g*K + idx, hw] += (pos >= 0 ? g : -g),  idx = pos & 0x7fffffff
 * grad_input must hold zeros (or the values to accumulate onto) on entry,
 * as the reference requires (model/norm_dist.py:34). */
LDIST_API int ldist_inf_dist_backward_input(const float* grad_output, const int32_t* pos, int B, int CO, int CI, int G, int HW,
                                  float* grad_input, ldist_stream_t stream);

/* L_inf backward w.r.t. weight.  Replaces inf_dist_backward_weight_cuda
 * (model/norm_dist.cpp:19-20, model/inf_dist_cuda.cu:197-204).
 *   grad_weight[g*NG + n, idx] += (pos < 0 ? g : -g), summed over b and hw
 * grad_weight must hold zeros (or the values to accumulate onto) on entry (model/norm_dist.py:37). */
LDIST_API int ldist_inf_dist_backward_weight(const float* grad_output, const int32_t* pos, int B, int CO, int CI, int G, int HW,
                                   float* grad_weight, ldist_stream_t stream);

/* p-norm forward, p > 1.  Replaces norm_dist_forward_cuda
 * (model/norm_dist.cpp:7-8, model/norm_dist_cuda.cu:427-437).
 *   output = m * (1e-10*(1e-10/m)^p + sum_k (|x-w|/m)^p)^(1/p),  m = max(1e-10, max_k |x-w|)
 * i.e. (sum |x-w|^p)^(1/p) evaluated with the reference's max-normalised
 * stabilisation and seeds (norm_dist_cuda.cu:232-233,253-264,289). */
LDIST_API int ldist_norm_dist_forward(const float* input, const float* weight, int B, int CO, int CI, int G, int HW,
                            float* output, float p, ldist_stream_t stream);

/* p-norm backward w.r.t. input.  Replaces norm_dist_backward_input_cuda
 * (model/norm_dist.cpp:9-10, model/norm_dist_cuda.cu:438-448).
 *   grad_input[m,k] = sum_n g[m,n] * (|x-w| / output[m,n])^(p-1) * (x-w > 0 ? 1 : -1)
 * Every element of grad_input is written; it may be uninitialised on entry (model/norm_dist.py:42). */
LDIST_API int ldist_norm_dist_backward_input(const float* grad_output, const float* input, const float* weight,
                                   const float* output, int B, int CO, int CI, int G, int HW, float* grad_input,
                                   float p, ldist_stream_t stream);

/* p-norm backward w.r.t. weight.  Replaces norm_dist_backward_weight_cuda
 * (model/norm_dist.cpp:11-12, model/norm_dist_cuda.cu:449-459).
 *   grad_weight[n,k] += sum_{b,hw} g * (|w-x| / output)^(p-1) * (w-x > 0 ? 1 : -1)
 * grad_weight must hold zeros (or the values to accumulate onto) on entry (model/norm_dist.py:45). */
LDIST_API int ldist_norm_dist_backward_weight(const float* grad_output, const float* input, const float* weight,
                                    const float* output, int B, int CO, int CI, int G, int HW, float* grad_weight,
                                    float p, ldist_stream_t stream);

/* Both p-norm gradients in one call: what ldist_norm_dist_backward_input followed by
 * ldist_norm_dist_backward_weight computes (the reference's norm_dist_backward_input_cuda and
 * norm_dist_backward_weight_cuda, model/norm_dist.cpp:9-12, which its autograd function calls one after the other,
 * model/norm_dist.py:41-46).  No single counterpart in the reference.  Every term
 *   g[m,n] * (|x-w| / output[m,n])^(p-1) * sign(x-w)
 * belongs to both sums.  One kernel evaluates it once and adds it to both for fully connected layers large enough to
 * fill the device at every exponent p > 2 (p = 2 is cheaper as two kernels, p = 3 too unless the tiles fill nine
 * tenths of the device; grad_weight then
 * collects one addend per tile of 128 rows with float atomics, in no fixed order), and for the unfolded-conv layout (HW > 1) with up to
 * about 140 outputs per group (one addend per workgroup); other shapes run the two separate kernels.  grad_input is written whole and may be uninitialised;
 * grad_weight is added to and must hold zeros (or the values to accumulate onto) on entry. */
LDIST_API int ldist_norm_dist_backward(const float* grad_output, const float* input, const float* weight,
                                       const float* output, int B, int CO, int CI, int G, int HW, float* grad_input,
                                       float* grad_weight, float p, ldist_stream_t stream);

/* The two scatter backward passes again, but writing EVERY element of the
 * gradient (zeros where nothing lands) so the caller can pass uninitialised
 * memory and skip its own zero fill.  No counterpart in the reference, which
 * needs torch.zeros_like first (model/norm_dist.py:34,37); results are equal
 * to zero-fill followed by the accumulate entry points above. */
LDIST_API int ldist_inf_dist_backward_input_overwrite(const float* grad_output, const int32_t* pos, int B, int CO, int CI,
                                            int G, int HW, float* grad_input, ldist_stream_t stream);
LDIST_API int ldist_inf_dist_backward_weight_overwrite(const float* grad_output, const int32_t* pos, int B, int CO, int CI,
                                             int G, int HW, float* grad_weight, ldist_stream_t stream);

/* Both of them in one call: what DistF.backward needs when both gradients are wanted (model/norm_dist.py:33-38
 * calls the two native functions one after the other).  For a fully connected layer (HW == 1) the two scatters run
 * as one launch whose workgroups do either, so the short, latency-bound grad_input workgroups run beside the
 * streaming grad_weight ones; other layouts run the two kernels inside the call.  Results are those of the two
 * overwrite entry points. */
LDIST_API int ldist_inf_dist_backward_overwrite(const float* grad_output, const int32_t* pos, int B, int CO, int CI, int G,
                                      int HW, float* grad_input, float* grad_weight, ldist_stream_t stream);

/* Per-channel mean shift of a contiguous (B, C, L) tensor in one kernel:
 *   mean[c] = mean over b and l of x[b,c,l];   y[b,c,l] = x[b,c,l] - mean[c]
 *   running_mean[c] = (1 - momentum) * running_mean[c] + momentum * mean[c]   (when running_mean != NULL)
 * No native counterpart in the reference: this is the training-mode arithmetic of its MeanNorm
 * module (model/norm_dist.py:85-96), which runs as five small torch kernels per layer; the backward
 * pass is the same operation on the gradient (gx = gy - mean(gy)).  mean_out (C floats) and
 * running_mean may be NULL; y must not overlap x. */
LDIST_API int ldist_mean_shift(const float* x, int B, int C, int L, float* y, float* mean_out, float* running_mean,
                     float momentum, ldist_stream_t stream);

/* One AdamW step with row-wise l_p weight decay on a contiguous (rows, cols) parameter, in place
 * and in one kernel.  No native counterpart in the reference: it is the arithmetic of its
 * optimizer (adamw.py:36-85), about sixteen elementwise torch kernels per tensor there.
 * Decay first, on the parameter itself, chosen by p_norm (the p of the owning module):
 *   p_norm <= 0 or NaN  (module without p, :42-43):  w *= 1 - lr*weight_decay
 *   finite p_norm > 0   (:44-50):  a = w^2 + eps, s = a / max_row(a), q = s^(p/2 - 1),
 *                                  w += -lr*weight_decay * (sum_row s*q)^(2/p - 1) * q * w
 *   p_norm = +inf       (:51-55):  only the first element of largest |w| in each row decays
 * then Adam on the decayed value (:73-85) with bias corrections for the 1-based `step`:
 *   m = beta1*m + (1-beta1)*g,  v = beta2*v + (1-beta2)*g*g,
 *   w -= lr/(1-beta1^step) * m / (sqrt(v)/sqrt(1-beta2^step) + eps)
 * grad == NULL: the decay alone (exp_avg, exp_avg_sq are not touched and may be NULL).
 * The hyper-parameters are doubles, as in the reference's Python: 1 - beta2 = 0.001 loses five
 * digits when beta2 is first rounded to float. */
LDIST_API int ldist_adamw_lp_step(float* param, const float* grad, float* exp_avg, float* exp_avg_sq, int rows, int cols,
                        double p_norm, double lr, double beta1, double beta2, double eps, double weight_decay,
                        int step, ldist_stream_t stream);

/* Patch extraction for the convolution-shaped layer, with torch's F.unfold layout, which the
 * reference uses to turn an image into the layer's input (model/norm_dist.py:132,144-145):
 *   cols[b, (c*KH + i)*KW + j, h*WO + w] = img[b, c, h*stride + i*dilation - padding, w*stride + j*dilation - padding]
 * (0 outside the image); HO = (H + 2*padding - dilation*(KH-1) - 1)/stride + 1, WO likewise.
 * img is (B, C, H, W), cols is (B, C*KH*KW, HO*WO).  No native counterpart in the reference. */
LDIST_API int ldist_unfold(const float* img, int B, int C, int H, int W, int KH, int KW, int stride, int padding, int dilation,
                 float* cols, ldist_stream_t stream);

/* L_inf forward of the convolution-shaped layer straight from the image, without the unfolded tensor:
 * what ldist_unfold followed by ldist_inf_dist_forward computes (the reference: F.unfold at
 * model/norm_dist.py:132, then inf_dist_forward_cuda), bit for bit, reading the image once.
 *   img (B, C, H, W), weight (CO, C/G*KH*KW), output and pos (B, CO, HO*WO).
 * Covers 3x3 windows with dilation 1 and stride 1 or 2 (lanes take eight neighbouring positions of a row:
 * output widths that are multiples of 8 waste none), where a group's channels are few enough for their
 * image rows to stay in LDS or a multiple of four (then they are staged), and where the layer is large
 * enough to keep a CU busy;
 * ldist_inf_dist_conv_forward_supported returns 1 for such a geometry, 0 otherwise, and
 * ldist_inf_dist_conv_forward returns LDIST_EUNSUPPORTED for the rest (nothing is enqueued). */
LDIST_API int ldist_inf_dist_conv_forward_supported(int C, int H, int W, int CO, int G, int KH, int KW, int stride, int padding,
                                          int dilation);
LDIST_API int ldist_inf_dist_conv_forward(const float* img, const float* weight, int B, int C, int H, int W, int CO, int G,
                                int KH, int KW, int stride, int padding, int dilation, float* output, int32_t* pos,
                                ldist_stream_t stream);

/* The same without pos, for forward passes that no gradient follows: output as ldist_inf_dist_conv_forward
 * writes it, bit for bit, from a kernel that keeps no per-channel record and searches for no index.  No counterpart
 * in the reference.  Covers what ldist_inf_dist_conv_forward_supported says; LDIST_EUNSUPPORTED otherwise. */
LDIST_API int ldist_inf_dist_conv_forward_values(const float* img, const float* weight, int B, int C, int H, int W, int CO,
                                       int G, int KH, int KW, int stride, int padding, int dilation, float* output,
                                       ldist_stream_t stream);
/* Interval-bound forward of the convolution-shaped layer straight from the lower and upper images: what
 * ldist_unfold of both followed by ldist_inf_dist_bound_forward computes (the reference: F.unfold at
 * model/norm_dist.py:144-145, then inf_dist_bound_forward_cuda), bit for bit, irregular boxes included.
 *   lower_img, upper_img (B, C, H, W), weight (CO, C/G*KH*KW), output_lower and output_upper (B, CO, HO*WO).
 * Covers 3x3 windows with dilation 1 and stride 1 or 2, any number of channels;
 * ldist_inf_dist_bound_conv_forward_supported returns 1 for such a geometry, 0 otherwise, and
 * ldist_inf_dist_bound_conv_forward returns LDIST_EUNSUPPORTED for the rest (nothing is enqueued). */
LDIST_API int ldist_inf_dist_bound_conv_forward_supported(int C, int H, int W, int CO, int G, int KH, int KW, int stride,
                                                          int padding, int dilation);
LDIST_API int ldist_inf_dist_bound_conv_forward(const float* lower_img, const float* upper_img, const float* weight,
                                                int B, int C, int H, int W, int CO, int G, int KH, int KW, int stride,
                                                int padding, int dilation, float* output_lower, float* output_upper,
                                                ldist_stream_t stream);
/* The p-norm layer of convolution shape straight from the image, forward and both gradients, without the
 * unfolded tensor.  They replace F.unfold (model/norm_dist.py:132) followed by norm_dist_forward_cuda,
 * norm_dist_backward_input_cuda and norm_dist_backward_weight_cuda (model/norm_dist.cpp:5-12,
 * model/norm_dist_cuda.cu:228-459) and the fold that autograd runs behind F.unfold:
 *   img (B, C, H, W), weight (CO, C/G*KH*KW), output and grad_output (B, CO, HO*WO), p > 1 finite.
 * Same values as the column entry points on ldist_unfold(img) to float rounding (forward with more than 16 outputs
 * per group and grad_weight: the same arithmetic in the same order; grad_img: a pixel adds up to KH*KW partial sums
 * in no fixed order).
 *   forward:          output is written.
 *   backward_input:   grad_img (B, C, H, W) is written whole; it may be uninitialised on entry.
 *   backward_weight:  grad_weight (CO, C/G*KH*KW) is added to and must hold zeros (or the values to accumulate
 *                     onto) on entry, as with ldist_norm_dist_backward_weight.
 * Covers 3x3 windows of any stride, padding and dilation with more than one output position;
 * ldist_norm_dist_conv_supported returns 1 for such a geometry, 0 otherwise, and the three entry points return
 * LDIST_EUNSUPPORTED for the rest (nothing is enqueued). */
LDIST_API int ldist_norm_dist_conv_supported(int C, int H, int W, int CO, int G, int KH, int KW, int stride, int padding,
                                             int dilation);
LDIST_API int ldist_norm_dist_conv_forward(const float* img, const float* weight, int B, int C, int H, int W, int CO, int G,
                                           int KH, int KW, int stride, int padding, int dilation, float* output, float p,
                                           ldist_stream_t stream);
LDIST_API int ldist_norm_dist_conv_backward_input(const float* grad_output, const float* img, const float* weight,
                                                  const float* output, int B, int C, int H, int W, int CO, int G, int KH,
                                                  int KW, int stride, int padding, int dilation, float* grad_img, float p,
                                                  ldist_stream_t stream);
LDIST_API int ldist_norm_dist_conv_backward_weight(const float* grad_output, const float* img, const float* weight,
                                                   const float* output, int B, int C, int H, int W, int CO, int G, int KH,
                                                   int KW, int stride, int padding, int dilation, float* grad_weight,
                                                   float p, ldist_stream_t stream);
/* Both gradients of the layer above in one call: what ldist_norm_dist_conv_backward_input followed by
 * ldist_norm_dist_conv_backward_weight computes, with the same contracts for grad_img (written whole) and
 * grad_weight (added to).  Where a group's outputs are few enough for its weights to stay in LDS (up to about 140
 * outputs per group) one kernel evaluates every term once and adds it to both sums, and every pixel of grad_img is
 * written by one workgroup (no atomics: grad_img does not depend on scheduling); other layers run the two kernels. */
LDIST_API int ldist_norm_dist_conv_backward(const float* grad_output, const float* img, const float* weight,
                                            const float* output, int B, int C, int H, int W, int CO, int G, int KH, int KW,
                                            int stride, int padding, int dilation, float* grad_img, float* grad_weight,
                                            float p, ldist_stream_t stream);
/* Testing and tuning knob, no counterpart in the reference: output rows per workgroup of
 * ldist_inf_dist_conv_forward; 0 (default) = chosen by shape.  A positive value is clamped to what the
 * geometry allows and also switches off the rule that leaves small or channel-heavy layers, which
 * would keep too few waves on a CU, to the general path.  Process-wide; not thread safe. */
LDIST_API int ldist_set_conv_rows_override(int rows);
/* Testing and tuning knob, no counterpart in the reference: how ldist_inf_dist_conv_forward keeps the
 * image rows in LDS.  0 (default) = by shape; 1 = only the variant that holds all channels of a group;
 * 2 = only the variant that stages four channels at a time (needs C/G % 4 == 0); 3 = neither, so that
 * every geometry is reported unsupported and callers take the column path (A/B comparisons).  A geometry
 * the forced variant cannot take becomes unsupported.  Process-wide; not thread safe. */
LDIST_API int ldist_set_conv_staging_override(int mode);

/* Adjoint of ldist_unfold (what autograd does behind F.unfold): every element of grad_img is written
 * with the sum of the grad_cols entries that were copied from it. */
LDIST_API int ldist_fold(const float* grad_cols, int B, int C, int H, int W, int KH, int KW, int stride, int padding,
               int dilation, float* grad_img, ldist_stream_t stream);

/* ldist_inf_dist_backward_input_overwrite composed with ldist_fold: the gradient of the L_inf layer
 * with respect to the IMAGE, without the (B, C*KH*KW, HO*WO) gradient of the columns in between.
 * grad_output and pos are (B, CO, HO*WO) as produced for the unfolded input; pos & 0x7fffffff is the
 * in-group row (c*KH + i)*KW + j of the columns.  Every element of grad_img (B, C, H, W) is written;
 * contributions whose argmax lies in the padding vanish, as they do in fold.
 * LDIST_ERANGE if (C/G)*W exceeds 16384 floats (use the two separate calls then). */
LDIST_API int ldist_inf_dist_backward_input_folded(const float* grad_output, const int32_t* pos, int B, int CO, int C, int G,
                                         int H, int W, int KH, int KW, int stride, int padding, int dilation,
                                         float* grad_img, ldist_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* LDIST_H */
