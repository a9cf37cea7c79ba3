/*
 * CPU oracle for the L_p / L_inf distance-neuron operators.
 *
 * THIS FILE IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It restates, in plain C,
 * the arithmetic of the reference's seven native entry points so that the HIP
 * kernels can be checked against it.  Only tests/, __graft_entry__.smoke() and
 * the cpu_baseline leg of bench.py may load the library built from it; the
 * product path (the HIP library behind include/ldist.h) never links or calls it.
 *
 * Tensor layout (reference model/inf_dist_cuda.cu:29-33,65-66), all contiguous:
 *   input   (B, CI, HW)   element ((b*G + g)*K  + k )*HW + hw,   K  = CI/G
 *   weight  (CO, K)       element  (g*NG + n)*K + k,             NG = CO/G
 *   output  (B, CO, HW)   element ((b*G + g)*NG + n )*HW + hw
 * CO and CI are totals over all groups (reference model/norm_dist.cpp:26).
 *
 * Every function returns 0, or a negative code for arguments the reference
 * would have mis-indexed on (null pointer, non-positive size, CI % G, CO % G).
 *
 * How each function is pinned (tests/test_oracle_*.py): brute-force closed
 * forms in torch (fp32 for max/abs which are exact, fp64 for power sums),
 * torch.cdist, torch.autograd through the closed form, hand-made known-answer
 * vectors for ties / signs / zeros, and algebraic invariants.  The reference
 * ships no test vectors of its own for this path.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define LDIST_ORACLE_OK 0
#define LDIST_ORACLE_EINVAL (-1)
#define LDIST_ORACLE_ENOMEM (-2)

#define SIGN_FLAG ((int32_t)0x80000000u)

static int check_dims(int B, int CO, int CI, int G, int HW) {
    if (B <= 0 || CO <= 0 || CI <= 0 || G <= 0 || HW <= 0) return LDIST_ORACLE_EINVAL;
    if (CI % G != 0 || CO % G != 0) return LDIST_ORACLE_EINVAL;
    return LDIST_ORACLE_OK;
}

int ldist_oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------------- */
/* L_inf forward: reference model/inf_dist_cuda.cu:10-68.                     */
/*   out = 0, pos = 0 (:14-15); scan k ascending; update only on strict '>'   */
/*   (:39) so ties keep the lowest k and a NaN difference never wins;         */
/*   pos = k, with bit 31 set when x - w < 0 (:41).                           */
/* This is the literal scalar restatement.                                    */
/* ------------------------------------------------------------------------- */
int ldist_oracle_inf_dist_forward_literal(const float* input, const float* weight, int B, int CO, int CI, int G,
                                          int HW, float* output, int32_t* pos) {
    int rc = check_dims(B, CO, CI, G, HW);
    if (rc) return rc;
    if (!input || !weight || !output || !pos) return LDIST_ORACLE_EINVAL;
    const int K = CI / G, NG = CO / G;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; b++) {
        for (int gn = 0; gn < CO; gn++) {
            const int g = gn / NG;
            const float* w = weight + (size_t)gn * K;
            for (int hw = 0; hw < HW; hw++) {
                const float* x = input + ((size_t)(b * G + g) * K) * HW + hw;
                float best = 0.0f;
                int32_t best_pos = 0;
                for (int k = 0; k < K; k++) {
                    float t = x[(size_t)k * HW] - w[k];
                    float a = fabsf(t);
                    if (a > best) {
                        best = a;
                        best_pos = (int32_t)k | (t >= 0 ? 0 : SIGN_FLAG);
                    }
                }
                size_t o = ((size_t)b * CO + gn) * HW + hw;
                output[o] = best;
                pos[o] = best_pos;
            }
        }
    }
    return LDIST_ORACLE_OK;
}

/* Same result as the literal version, arranged so the compiler can vectorise:
 * the value is a plain running maximum (exact, order independent), kept per
 * block of K together with the first block whose maximum strictly exceeds all
 * earlier ones; that block is then scanned for the lowest k that attains the
 * value.  tests/test_oracle_inf.py checks it bit-for-bit against the literal
 * version.  Used for full-size parity runs and as the timed CPU baseline. */
#define FAST_BLOCK 64

__attribute__((target_clones("avx2", "default")))
static float block_absmax(const float* x, const float* w, int n) {
    float lane[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    int k = 0;
    for (; k + 8 <= n; k += 8) {
        for (int j = 0; j < 8; j++) {
            float a = fabsf(x[k + j] - w[k + j]);
            lane[j] = a > lane[j] ? a : lane[j];
        }
    }
    float m = 0.0f;
    for (int j = 0; j < 8; j++) m = lane[j] > m ? lane[j] : m;
    for (; k < n; k++) {
        float a = fabsf(x[k] - w[k]);
        m = a > m ? a : m;
    }
    return m;
}

int ldist_oracle_inf_dist_forward(const float* input, const float* weight, int B, int CO, int CI, int G, int HW,
                                  float* output, int32_t* pos) {
    int rc = check_dims(B, CO, CI, G, HW);
    if (rc) return rc;
    if (!input || !weight || !output || !pos) return LDIST_ORACLE_EINVAL;
    const int K = CI / G, NG = CO / G;
    int fail = 0;
#pragma omp parallel
    {
        /* one gathered x row per thread so the inner loops are unit stride for HW > 1 too */
        float* xrow = (float*)malloc((size_t)K * sizeof(float));
        if (!xrow) {
#pragma omp atomic write
            fail = 1;
        }
#pragma omp for collapse(2) schedule(static)
        for (int bg = 0; bg < B * G; bg++) {
            for (int hw = 0; hw < HW; hw++) {
                if (!xrow) continue;
                const int b = bg / G, g = bg % G;
                const float* xsrc = input + ((size_t)bg * K) * HW + hw;
                for (int k = 0; k < K; k++) xrow[k] = xsrc[(size_t)k * HW];
                for (int n = 0; n < NG; n++) {
                    const float* w = weight + ((size_t)g * NG + n) * K;
                    float best = 0.0f;
                    int best_blk = -1;
                    for (int k0 = 0; k0 < K; k0 += FAST_BLOCK) {
                        int len = K - k0 < FAST_BLOCK ? K - k0 : FAST_BLOCK;
                        float m = block_absmax(xrow + k0, w + k0, len);
                        if (m > best) {
                            best = m;
                            best_blk = k0;
                        }
                    }
                    int32_t p = 0;
                    if (best_blk >= 0) {
                        int end = best_blk + FAST_BLOCK < K ? best_blk + FAST_BLOCK : K;
                        for (int k = best_blk; k < end; k++) {
                            float t = xrow[k] - w[k];
                            if (fabsf(t) == best) {
                                p = (int32_t)k | (t >= 0 ? 0 : SIGN_FLAG);
                                break;
                            }
                        }
                    }
                    size_t o = (((size_t)b * G + g) * NG + n) * HW + hw;
                    output[o] = best;
                    pos[o] = p;
                }
            }
        }
        free(xrow);
    }
    return fail ? LDIST_ORACLE_ENOMEM : LDIST_ORACLE_OK;
}

/* ------------------------------------------------------------------------- */
/* Interval-bound forward: reference model/inf_dist_cuda.cu:73-141.           */
/*   U = max_k max(|l-w|, |u-w|)                       (:108)                 */
/*   L = max_k min(|l-w|, |u-w|), skipping k where l-w < 0 and u-w > 0 (:109) */
/*   both start at 0 (:78); max/min are the NaN-ignoring fmaxf/fminf.         */
/* ------------------------------------------------------------------------- */
int ldist_oracle_inf_dist_bound_forward(const float* input_lower, const float* input_upper, const float* weight,
                                        int B, int CO, int CI, int G, int HW, float* output_lower,
                                        float* output_upper) {
    int rc = check_dims(B, CO, CI, G, HW);
    if (rc) return rc;
    if (!input_lower || !input_upper || !weight || !output_lower || !output_upper) return LDIST_ORACLE_EINVAL;
    const int K = CI / G, NG = CO / G;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; b++) {
        for (int gn = 0; gn < CO; gn++) {
            const int g = gn / NG;
            const float* w = weight + (size_t)gn * K;
            for (int hw = 0; hw < HW; hw++) {
                size_t xo = ((size_t)(b * G + g) * K) * HW + hw;
                const float* xl = input_lower + xo;
                const float* xu = input_upper + xo;
                float lo = 0.0f, up = 0.0f;
                for (int k = 0; k < K; k++) {
                    float tl = xl[(size_t)k * HW] - w[k];
                    float tu = xu[(size_t)k * HW] - w[k];
                    float al = fabsf(tl), au = fabsf(tu);
                    up = fmaxf(up, fmaxf(al, au));
                    if (!(tl < 0 && tu > 0)) lo = fmaxf(lo, fminf(al, au));
                }
                size_t o = ((size_t)b * CO + gn) * HW + hw;
                output_lower[o] = lo;
                output_upper[o] = up;
            }
        }
    }
    return LDIST_ORACLE_OK;
}

/* ------------------------------------------------------------------------- */
/* L_inf backward w.r.t. input: reference model/inf_dist_cuda.cu:143-156.     */
/*   grad_input[b, g*K + idx, hw] += (pos >= 0 ? g : -g), idx = pos & ~bit31  */
/* The reference adds with fp32 atomics in an unspecified order; here each    */
/* destination is summed in double, n ascending, then added to the float      */
/* already in grad_input (which the caller zero-fills, model/norm_dist.py:34).*/
/* ------------------------------------------------------------------------- */
int ldist_oracle_inf_dist_backward_input(const float* grad_output, const int32_t* pos, int B, int CO, int CI, int G,
                                         int HW, float* grad_input) {
    int rc = check_dims(B, CO, CI, G, HW);
    if (rc) return rc;
    if (!grad_output || !pos || !grad_input) return LDIST_ORACLE_EINVAL;
    const int K = CI / G, NG = CO / G;
    int fail = 0;
#pragma omp parallel
    {
        double* acc = (double*)malloc((size_t)K * sizeof(double));
        if (!acc) {
#pragma omp atomic write
            fail = 1;
        }
#pragma omp for collapse(2) schedule(static)
        for (int bg = 0; bg < B * G; bg++) {
            for (int hw = 0; hw < HW; hw++) {
                if (!acc) continue;
                memset(acc, 0, (size_t)K * sizeof(double));
                for (int n = 0; n < NG; n++) {
                    size_t o = ((size_t)bg * NG + n) * HW + hw;
                    int32_t p = pos[o];
                    int idx = (int)(p & 0x7fffffff);
                    if (idx >= K) continue; /* the reference would write out of bounds */
                    float gv = grad_output[o];
                    acc[idx] += (double)(p >= 0 ? gv : -gv);
                }
                float* dst = grad_input + ((size_t)bg * K) * HW + hw;
                for (int k = 0; k < K; k++)
                    if (acc[k] != 0.0) dst[(size_t)k * HW] = (float)((double)dst[(size_t)k * HW] + acc[k]);
            }
        }
        free(acc);
    }
    return fail ? LDIST_ORACLE_ENOMEM : LDIST_ORACLE_OK;
}

/* L_inf backward w.r.t. weight: reference model/inf_dist_cuda.cu:158-171.    */
/*   grad_weight[g*NG + n, idx] += (pos < 0 ? g : -g), summed over b and hw   */
int ldist_oracle_inf_dist_backward_weight(const float* grad_output, const int32_t* pos, int B, int CO, int CI, int G,
                                          int HW, float* grad_weight) {
    int rc = check_dims(B, CO, CI, G, HW);
    if (rc) return rc;
    if (!grad_output || !pos || !grad_weight) return LDIST_ORACLE_EINVAL;
    const int K = CI / G;
    int fail = 0;
#pragma omp parallel
    {
        double* acc = (double*)malloc((size_t)K * sizeof(double));
        if (!acc) {
#pragma omp atomic write
            fail = 1;
        }
#pragma omp for schedule(static)
        for (int gn = 0; gn < CO; gn++) {
            if (!acc) continue;
            memset(acc, 0, (size_t)K * sizeof(double));
            for (int b = 0; b < B; b++) {
                const size_t base = ((size_t)b * CO + gn) * HW;
                for (int hw = 0; hw < HW; hw++) {
                    int32_t p = pos[base + hw];
                    int idx = (int)(p & 0x7fffffff);
                    if (idx >= K) continue;
                    float gv = grad_output[base + hw];
                    acc[idx] += (double)(p < 0 ? gv : -gv);
                }
            }
            float* dst = grad_weight + (size_t)gn * K;
            for (int k = 0; k < K; k++)
                if (acc[k] != 0.0) dst[k] = (float)((double)dst[k] + acc[k]);
        }
        free(acc);
    }
    return fail ? LDIST_ORACLE_ENOMEM : LDIST_ORACLE_OK;
}

/* ------------------------------------------------------------------------- */
/* p-norm forward: reference model/norm_dist_cuda.cu:228-292.                 */
/* The reference keeps a running maximum m (seeded 1e-10, :233) and a running */
/* sum acc of (|x-w|/m)^p (seeded 1e-10, :232); whenever a 16-wide block      */
/* raises m, acc is multiplied by (m_old/m_new)^p (:257-261); the result is   */
/* acc^(1/p) * m (:289).  In exact arithmetic that is                         */
/*   m   = max(1e-10, max_k |x-w|)                                            */
/*   out = m * ( 1e-10*(1e-10/m)^p + sum_k (|x-w|/m)^p )^(1/p)                */
/* which is what this function evaluates, in double, rounding once to float.  */
/* ------------------------------------------------------------------------- */
int ldist_oracle_norm_dist_forward(const float* input, const float* weight, int B, int CO, int CI, int G, int HW,
                                   float* output, float p) {
    int rc = check_dims(B, CO, CI, G, HW);
    if (rc) return rc;
    if (!input || !weight || !output || !(p > 1.0f)) return LDIST_ORACLE_EINVAL;
    const int K = CI / G, NG = CO / G;
    const double pd = (double)p;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; b++) {
        for (int gn = 0; gn < CO; gn++) {
            const int g = gn / NG;
            const float* w = weight + (size_t)gn * K;
            for (int hw = 0; hw < HW; hw++) {
                const float* x = input + ((size_t)(b * G + g) * K) * HW + hw;
                double m = 1e-10;
                for (int k = 0; k < K; k++) {
                    double a = fabs((double)x[(size_t)k * HW] - (double)w[k]);
                    if (a > m) m = a;
                }
                double acc = 1e-10 * pow(1e-10 / m, pd);
                for (int k = 0; k < K; k++) {
                    double a = fabs((double)x[(size_t)k * HW] - (double)w[k]);
                    acc += pow(a / m, pd);
                }
                output[((size_t)b * CO + gn) * HW + hw] = (float)(pow(acc, 1.0 / pd) * m);
            }
        }
    }
    return LDIST_ORACLE_OK;
}

/* The same forward in float, in the reference's own order of operations
 * (16-wide blocks, rescale on a new block maximum, k ascending), with powf in
 * place of the reference's fast __powf.  It shows how far a float evaluation in
 * that order sits from the double result above; it is not the parity target. */
int ldist_oracle_norm_dist_forward_f32(const float* input, const float* weight, int B, int CO, int CI, int G, int HW,
                                       float* output, float p) {
    int rc = check_dims(B, CO, CI, G, HW);
    if (rc) return rc;
    if (!input || !weight || !output || !(p > 1.0f)) return LDIST_ORACLE_EINVAL;
    const int K = CI / G, NG = CO / G;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; b++) {
        for (int gn = 0; gn < CO; gn++) {
            const int g = gn / NG;
            const float* w = weight + (size_t)gn * K;
            for (int hw = 0; hw < HW; hw++) {
                const float* x = input + ((size_t)(b * G + g) * K) * HW + hw;
                float acc = 1e-10f, m = 1e-10f, rm = 1.0f / m;
                for (int k0 = 0; k0 < K; k0 += 16) {
                    int end = k0 + 16 < K ? k0 + 16 : K;
                    float bm = 0.0f;
                    for (int k = k0; k < end; k++) bm = fmaxf(bm, fabsf(x[(size_t)k * HW] - w[k]));
                    if (bm > m) {
                        rm = 1.0f / bm;
                        acc = acc * powf(m * rm, p);
                        m = bm;
                    }
                    for (int k = k0; k < end; k++) acc += powf(fabsf(x[(size_t)k * HW] - w[k]) * rm, p);
                }
                output[((size_t)b * CO + gn) * HW + hw] = powf(acc, 1.0f / p) * m;
            }
        }
    }
    return LDIST_ORACLE_OK;
}

/* ------------------------------------------------------------------------- */
/* p-norm backward w.r.t. input: reference model/norm_dist_cuda.cu:294-361.   */
/*   grad_input[m,k] = sum_n g[m,n] * (|t| * (1/out[m,n]))^(p-1) * s,         */
/*   t = x - w, s = +1 if t > 0 else -1 (:295-296).  Every element is written */
/*   (:359-360).  Evaluated in double from the float inputs.                  */
/* ------------------------------------------------------------------------- */
/*   abs_terms (may be NULL) receives sum_n |g * (|t|/out)^(p-1)|, the scale  */
/*   against which a float evaluation's rounding error is judged.             */
int ldist_oracle_norm_dist_backward_input(const float* grad_output, const float* input, const float* weight,
                                          const float* output, int B, int CO, int CI, int G, int HW,
                                          float* grad_input, float p, float* abs_terms) {
    int rc = check_dims(B, CO, CI, G, HW);
    if (rc) return rc;
    if (!grad_output || !input || !weight || !output || !grad_input || !(p > 1.0f)) return LDIST_ORACLE_EINVAL;
    const int K = CI / G, NG = CO / G;
    const double pm1 = (double)p - 1.0;
#pragma omp parallel for collapse(2) schedule(static)
    for (int bg = 0; bg < B * G; bg++) {
        for (int k = 0; k < K; k++) {
            const int g = bg % G;
            for (int hw = 0; hw < HW; hw++) {
                const double x = (double)input[((size_t)bg * K + k) * HW + hw];
                double acc = 0.0, mag = 0.0;
                for (int n = 0; n < NG; n++) {
                    size_t o = ((size_t)bg * NG + n) * HW + hw;
                    double t = x - (double)weight[((size_t)g * NG + n) * K + k];
                    double ro = 1.0 / (double)output[o];
                    double v = (double)grad_output[o] * pow(fabs(t) * ro, pm1);
                    acc += t > 0 ? v : -v;
                    mag += fabs(v);
                }
                grad_input[((size_t)bg * K + k) * HW + hw] = (float)acc;
                if (abs_terms) abs_terms[((size_t)bg * K + k) * HW + hw] = (float)mag;
            }
        }
    }
    return LDIST_ORACLE_OK;
}

/* p-norm backward w.r.t. weight: reference model/norm_dist_cuda.cu:363-425.  */
/*   grad_weight[n,k] += sum_{b,hw} g * (|t| * (1/out))^(p-1) * s,            */
/*   t = w - x, s = +1 if t > 0 else -1 (:364-365); added onto the caller's   */
/*   zero-filled buffer (:424, model/norm_dist.py:45).                        */
int ldist_oracle_norm_dist_backward_weight(const float* grad_output, const float* input, const float* weight,
                                           const float* output, int B, int CO, int CI, int G, int HW,
                                           float* grad_weight, float p, float* abs_terms) {
    int rc = check_dims(B, CO, CI, G, HW);
    if (rc) return rc;
    if (!grad_output || !input || !weight || !output || !grad_weight || !(p > 1.0f)) return LDIST_ORACLE_EINVAL;
    const int K = CI / G, NG = CO / G;
    const double pm1 = (double)p - 1.0;
#pragma omp parallel for collapse(2) schedule(static)
    for (int gn = 0; gn < CO; gn++) {
        for (int k = 0; k < K; k++) {
            const int g = gn / NG;
            const double w = (double)weight[(size_t)gn * K + k];
            double acc = 0.0, mag = 0.0;
            for (int b = 0; b < B; b++) {
                const size_t obase = ((size_t)b * CO + gn) * HW;
                const size_t xbase = ((size_t)(b * G + g) * K + k) * HW;
                for (int hw = 0; hw < HW; hw++) {
                    double t = w - (double)input[xbase + hw];
                    double ro = 1.0 / (double)output[obase + hw];
                    double v = (double)grad_output[obase + hw] * pow(fabs(t) * ro, pm1);
                    acc += t > 0 ? v : -v;
                    mag += fabs(v);
                }
            }
            float* dst = grad_weight + (size_t)gn * K + k;
            *dst = (float)((double)*dst + acc);
            if (abs_terms) abs_terms[(size_t)gn * K + k] = (float)mag;
        }
    }
    return LDIST_ORACLE_OK;
}

/* Per-channel mean shift of a (B, C, L) tensor: the training-mode arithmetic of the reference's */
/* MeanNorm (model/norm_dist.py:85-96): mean over b and l, y = x - mean, running mean moved by   */
/* momentum.  Sums are taken in double.  mean_out and running_mean may be NULL.                  */
int ldist_oracle_mean_shift(const float* x, int B, int C, int L, float* y, float* mean_out, float* running_mean,
                            float momentum) {
    if (!x || !y || B <= 0 || C <= 0 || L <= 0) return LDIST_ORACLE_EINVAL;
#pragma omp parallel for schedule(static)
    for (int c = 0; c < C; c++) {
        double s = 0.0;
        for (int b = 0; b < B; b++)
            for (int l = 0; l < L; l++) s += (double)x[((size_t)b * C + c) * L + l];
        const double mean = s / ((double)B * (double)L);
        for (int b = 0; b < B; b++)
            for (int l = 0; l < L; l++) {
                const size_t at = ((size_t)b * C + c) * L + l;
                y[at] = (float)((double)x[at] - mean);
            }
        if (mean_out) mean_out[c] = (float)mean;
        if (running_mean) running_mean[c] = (float)((1.0 - (double)momentum) * (double)running_mean[c] + (double)momentum * mean);
    }
    return LDIST_ORACLE_OK;
}

/* One AdamW step with row-wise l_p weight decay on a (rows, cols) parameter: reference           */
/* adamw.py:36-85.  The decay comes first and acts on the parameter itself (:40-56):              */
/*   p_norm <= 0 ("the module has no p", :42-43):  w *= 1 - lr*wd                                  */
/*   finite p_norm (:44-50):  a = w^2 + eps,  s = a / max_row(a),  q = s^(p/2 - 1),                */
/*                            w += -lr*wd * (sum_row s*q)^(2/p - 1) * q * w                         */
/*   p_norm = +inf (:51-55):  only the first element of largest |w| in the row: w -= lr*wd * w     */
/* then Adam on the decayed parameter (:73-85): m = b1*m + (1-b1)*g, v = b2*v + (1-b2)*g*g,        */
/*   w -= lr / (1 - b1^step) * m / (sqrt(v) / sqrt(1 - b2^step) + eps).  `step` counts from 1.     */
/* grad == NULL: the decay alone.  Everything is evaluated in double and rounded once.            */
int ldist_oracle_adamw_lp_step(float* param, const float* grad, float* exp_avg, float* exp_avg_sq, int rows, int cols,
                               double p_norm, double lr, double beta1, double beta2, double eps, double weight_decay,
                               int step) {
    if (!param || rows <= 0 || cols <= 0 || step < 1) return LDIST_ORACLE_EINVAL;
    if (grad && (!exp_avg || !exp_avg_sq)) return LDIST_ORACLE_EINVAL;
    const double lw = lr * weight_decay;
    const double bc1 = 1.0 - pow(beta1, (double)step), bc2 = 1.0 - pow(beta2, (double)step);
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; r++) {
        float* w = param + (size_t)r * cols;
        double* nw = (double*)malloc(sizeof(double) * (size_t)cols);
        if (!nw) continue;
        if (!(p_norm > 0.0)) {
            for (int i = 0; i < cols; i++) nw[i] = (double)w[i] * (1.0 - lw);
        } else if (isinf(p_norm)) {
            int best = 0;
            for (int i = 1; i < cols; i++)
                if (fabsf(w[i]) > fabsf(w[best])) best = i;
            for (int i = 0; i < cols; i++) nw[i] = (double)w[i];
            nw[best] = (double)w[best] - lw * (double)w[best];
        } else {
            const double p = p_norm;
            double mx = 0.0, sum = 0.0;
            for (int i = 0; i < cols; i++) {
                const double a = (double)w[i] * (double)w[i] + eps;
                if (a > mx) mx = a;
            }
            for (int i = 0; i < cols; i++) {
                const double s = ((double)w[i] * (double)w[i] + eps) / mx;
                sum += s * pow(s, p / 2.0 - 1.0);
            }
            const double c = pow(sum, 2.0 / p - 1.0);
            for (int i = 0; i < cols; i++) {
                const double s = ((double)w[i] * (double)w[i] + eps) / mx;
                nw[i] = (double)w[i] - lw * c * pow(s, p / 2.0 - 1.0) * (double)w[i];
            }
        }
        for (int i = 0; i < cols; i++) {
            if (grad) {
                const size_t at = (size_t)r * cols + i;
                const double g = (double)grad[at];
                const double m = beta1 * (double)exp_avg[at] + (1.0 - beta1) * g;
                const double v = beta2 * (double)exp_avg_sq[at] + (1.0 - beta2) * g * g;
                exp_avg[at] = (float)m;
                exp_avg_sq[at] = (float)v;
                nw[i] -= lr / bc1 * m / (sqrt(v) / sqrt(bc2) + eps);
            }
            w[i] = (float)nw[i];
        }
        free(nw);
    }
    return LDIST_ORACLE_OK;
}
