// L_inf distance backward: the gradient of out[m,n] = |x[m,k*] - w[n,k*]| flows to
// exactly one input and one weight element, the argmax k* recorded in pos
// (bit 31 = sign of x - w).  Semantics follow the reference kernels
// model/inf_dist_cuda.cu:143-171:
//   grad_input [b, g*K + idx, hw] += (pos >= 0 ? g : -g)
//   grad_weight[g*NG + n, idx]    += (pos <  0 ? g : -g)
// The reference issues one global atomic per (m,n).  Here every workgroup owns a
// slab of the gradient, gathers its contributions in LDS bins and writes the slab
// out with coalesced stores, so the pass is bounded by streaming grad_output/pos
// in and the gradient out.  In "overwrite" mode the slab is stored whole (zeros
// included), which replaces the caller's zero fill.
// All bins are doubles: on gfx950 an LDS atomic add of a double (ds_add_f64) retires about nine times as many lanes
// per clock as one of a float (ds_add_f32: 0.33 lanes per clock and CU, measured on random addresses; 2.9 for
// doubles, 6 for 32-bit integer adds), and a sum of floats held in a double does not depend on the order of the
// additions (exactly so while the addends' exponents span fewer than 29 binades, to 2^-53 otherwise).  A bin's sum is
// rounded to float once, when the slab is written: the gradients are the correctly rounded sums, the same bits in
// every run, whatever the scheduling.  "Accumulate" entry points add the bin to the caller's value in double and
// round once as well.
#include "kernels.hpp"

#include <algorithm>

namespace ldist {

struct BwdDims {
    int B, G, K, NG, HW;
};

// ---- grad_input ------------------------------------------------------------
// Workgroup = (image b, group g, TH consecutive hw, KC consecutive k).
// bins[kc][th]; element (k, hw) of the slab lives at ((b*G+g)*K + k)*HW + hw.
// bx, by: the workgroup's place in the grid of this scatter (the kernel below passes blockIdx; the kernel that runs
// both scatters of a layer in one launch passes what it dealt to this workgroup).
template <bool OVERWRITE>
__device__ __forceinline__ void backward_input_body(double* bins, int bx, int by, const float* __restrict__ grad_output,
                                                    const int32_t* __restrict__ pos, float* __restrict__ grad_input,
                                                    const BwdDims& d, int th_log2, int KC, int hw_tiles, int vec) {
    const int NT = blockDim.x;
    const int TH = 1 << th_log2;
    const int tile = bx % hw_tiles;
    const int bg = bx / hw_tiles;  // b*G + g
    const int hw0 = tile * TH;
    const int k0 = by * KC;
    const int kc = min(KC, d.K - k0);
    const int nb = kc * TH;
    const size_t obase = (size_t)bg * d.NG * d.HW;
    const size_t xbase = ((size_t)bg * d.K + k0) * d.HW;

    if (vec) {
        // fc layout (TH == 1) with NG, K, kc multiples of 4 and 16-byte aligned tensors: the rows of
        // pos / grad_output and the slab of grad_input are contiguous, so everything moves 128 bits
        // at a time; the loads of a lane's four elements are in flight together.
        double2* b2 = reinterpret_cast<double2*>(bins);
        for (int e = threadIdx.x; e < kc / 2; e += NT) b2[e] = make_double2(0.0, 0.0);
        __syncthreads();
        const int4* p4 = reinterpret_cast<const int4*>(pos + obase);
        const float4* g4 = reinterpret_cast<const float4*>(grad_output + obase);
        for (int e = threadIdx.x; e < d.NG / 4; e += NT) {
            const int4 pv = p4[e];
            const float4 gv = g4[e];
            const int ps[4] = {pv.x, pv.y, pv.z, pv.w};
            const float gs[4] = {gv.x, gv.y, gv.z, gv.w};
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int idx = (ps[q] & 0x7fffffff) - k0;
                if (idx >= 0 && idx < kc) atomicAdd(&bins[idx], (double)(ps[q] >= 0 ? gs[q] : -gs[q]));
            }
        }
        __syncthreads();
        float4* dst = reinterpret_cast<float4*>(grad_input + xbase);
        for (int e = threadIdx.x; e < kc / 4; e += NT) {
            const double2 lo = b2[2 * e], hi = b2[2 * e + 1];
            const float4 v = make_float4((float)lo.x, (float)lo.y, (float)hi.x, (float)hi.y);
            if (OVERWRITE) {
                dst[e] = v;
            } else if (v.x != 0.f || v.y != 0.f || v.z != 0.f || v.w != 0.f) {
                const float4 o = dst[e];
                dst[e] = make_float4((float)((double)o.x + lo.x), (float)((double)o.y + lo.y), (float)((double)o.z + hi.x),
                                     (float)((double)o.w + hi.y));
            }
        }
        return;
    }

    // conv layout with HW % 4 == 0, tiles of at least four positions and 16-byte aligned tensors: four
    // neighbouring positions per lane move with 128-bit loads and stores
    const bool quad = th_log2 >= 2 && (d.HW & 3) == 0 &&
                      ((reinterpret_cast<uintptr_t>(grad_output) | reinterpret_cast<uintptr_t>(pos) |
                        reinterpret_cast<uintptr_t>(grad_input)) & 15u) == 0;
    if (quad) {
        double2* b2 = reinterpret_cast<double2*>(bins);
        for (int e = threadIdx.x; e < nb / 2; e += NT) b2[e] = make_double2(0.0, 0.0);
        __syncthreads();
        const int tq_log2 = th_log2 - 2;                 // quads per tile row
        const int total_q = d.NG << tq_log2;
        for (int e = threadIdx.x; e < total_q; e += NT) {
            const int n = e >> tq_log2, j = (e & ((1 << tq_log2) - 1)) * 4;
            const int hw = hw0 + j;
            if (hw < d.HW) {                              // HW % 4 == 0: the whole quad is inside
                const size_t o = obase + (size_t)n * d.HW + hw;
                const int4 pv = *reinterpret_cast<const int4*>(pos + o);
                const float4 gv = *reinterpret_cast<const float4*>(grad_output + o);
                const int ps[4] = {pv.x, pv.y, pv.z, pv.w};
                const float gs[4] = {gv.x, gv.y, gv.z, gv.w};
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int idx = (ps[q] & 0x7fffffff) - k0;
                    if (idx >= 0 && idx < kc) atomicAdd(&bins[(idx << th_log2) + j + q], (double)(ps[q] >= 0 ? gs[q] : -gs[q]));
                }
            }
        }
        __syncthreads();
        for (int e = threadIdx.x; e < nb / 4; e += NT) {
            const int k = e >> tq_log2, j = (e & ((1 << tq_log2) - 1)) * 4;
            const int hw = hw0 + j;
            if (hw < d.HW) {
                float4* dst = reinterpret_cast<float4*>(grad_input + xbase + (size_t)k * d.HW + hw);
                const double2 lo = b2[2 * e], hi = b2[2 * e + 1];
                const float4 v = make_float4((float)lo.x, (float)lo.y, (float)hi.x, (float)hi.y);
                if (OVERWRITE) {
                    *dst = v;
                } else if (v.x != 0.f || v.y != 0.f || v.z != 0.f || v.w != 0.f) {
                    const float4 o = *dst;
                    *dst = make_float4((float)((double)o.x + lo.x), (float)((double)o.y + lo.y), (float)((double)o.z + hi.x),
                                       (float)((double)o.w + hi.y));
                }
            }
        }
        return;
    }

    for (int e = threadIdx.x; e < nb; e += NT) bins[e] = 0.0;
    __syncthreads();

    const int total = d.NG * TH;
    for (int e = threadIdx.x; e < total; e += NT) {
        const int n = e >> th_log2, j = e & (TH - 1);
        const int hw = hw0 + j;
        if (hw < d.HW) {
            const size_t o = obase + (size_t)n * d.HW + hw;
            const int p = pos[o];
            const int idx = (p & 0x7fffffff) - k0;
            if (idx >= 0 && idx < kc) {
                const float gv = grad_output[o];
                atomicAdd(&bins[(idx << th_log2) + j], (double)(p >= 0 ? gv : -gv));
            }
        }
    }
    __syncthreads();

    for (int e = threadIdx.x; e < nb; e += NT) {
        const int k = e >> th_log2, j = e & (TH - 1);
        const int hw = hw0 + j;
        if (hw < d.HW) {
            float* dst = grad_input + xbase + (size_t)k * d.HW + hw;
            const double v = bins[e];
            if (OVERWRITE) *dst = (float)v;
            else if (v != 0.0) *dst = (float)((double)*dst + v);
        }
    }
}

template <bool OVERWRITE>
__global__ void __launch_bounds__(1024)
inf_backward_input_kernel(const float* __restrict__ grad_output, const int32_t* __restrict__ pos,
                          float* __restrict__ grad_input, BwdDims d, int th_log2, int KC, int hw_tiles, int vec) {
    extern __shared__ __align__(16) double bins[];
    backward_input_body<OVERWRITE>(bins, blockIdx.x, blockIdx.y, grad_output, pos, grad_input, d, th_log2, KC, hw_tiles, vec);
}

// ---- grad_weight -----------------------------------------------------------
// Workgroup = (group g, NB consecutive outputs n, KC consecutive k -- all of K when a row of bins fits in 64 KB and
// the rows alone fill the device).  For one image the NB rows of grad_output/pos are one contiguous run of NB*HW
// elements.  bins[nb][kc].  A workgroup scans every image and is the only writer of its slab: a layer with few rows
// (a grouped conv layer: 128 rows of 131 072 contributions each) is spread over the device by giving a row to
// several workgroups with a k range each (they read the same lines, side by side in one L2), never by splitting the
// images, whose partial sums could only be joined with float atomics in an order that changes from run to run.
template <bool OVERWRITE>
__device__ __forceinline__ void backward_weight_body(double* bins, int bx, int by, const float* __restrict__ grad_output,
                                                     const int32_t* __restrict__ pos, float* __restrict__ grad_weight,
                                                     const BwdDims& d, int NB, int KC, int n_blocks) {
    const int NT = blockDim.x;
    // Neighbouring blocks of outputs read neighbouring few-byte pieces of the same memory lines (in the fc layout a
    // block's grad_output / pos entries of one image are NB * 4 bytes).  Workgroups go to the eight XCDs in turn, each
    // with its own L2, so XCD x takes the x-th eighth of the blocks: neighbours then share the lines in one L2
    // instead of fetching them eight times.  Where that matters (many blocks) the launcher rounds n_blocks up to a
    // multiple of eight; otherwise the blocks keep their order.
    const int id = bx % n_blocks;
    const int g = bx / n_blocks;
    const int nblk = (n_blocks & 7) == 0 ? (id % 8) * (n_blocks / 8) + id / 8 : id;
    const int n0 = nblk * NB;
    if (n0 >= d.NG) return;
    const int nb = min(NB, d.NG - n0);
    const int k0 = by * KC;
    const int kc = min(KC, d.K - k0);
    const int b0 = 0, b1 = d.B;
    // kc is a multiple of 4 whenever vec is set, so rows of bins and of grad_weight stay 16-byte aligned
    const bool vec = (kc & 3) == 0 && (d.K & 3) == 0 && (reinterpret_cast<uintptr_t>(grad_weight) & 15u) == 0;
    if (vec) {   // 16 bytes of bins per store
        float4* b4 = reinterpret_cast<float4*>(bins);
        for (int e = threadIdx.x; e < nb * kc / 2; e += NT) b4[e] = make_float4(0.f, 0.f, 0.f, 0.f);
    } else {
        for (int e = threadIdx.x; e < nb * kc; e += NT) bins[e] = 0.0;
    }
    __syncthreads();

    const int run = nb * d.HW;  // contiguous elements per image
    const size_t img_stride = (size_t)d.G * d.NG * d.HW;
    const size_t first = ((size_t)g * d.NG + n0) * d.HW;
    if (d.HW == 1) {
        // several images per pass: element i -> (image i / nb, output i % nb)
        // index and gradient of four elements are fetched together: one after the other (the gradient only once the
        // index says it is wanted) a wave waited out two memory latencies per element
        const int total = (b1 - b0) * nb;
        for (int i0 = threadIdx.x; i0 < total; i0 += 4 * NT) {
            int p[4], nn[4];
            float gv[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int i = i0 + NT * u < total ? i0 + NT * u : i0;   // past the end: the first one again, not added
                const int bb = i / nb;
                nn[u] = i - bb * nb;
                const size_t o = (size_t)(b0 + bb) * img_stride + first + nn[u];
                p[u] = pos[o];
                gv[u] = grad_output[o];
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int idx = (p[u] & 0x7fffffff) - k0;
                if ((u == 0 || i0 + NT * u < total) && idx >= 0 && idx < kc)
                    atomicAdd(&bins[nn[u] * kc + idx], (double)(p[u] < 0 ? gv[u] : -gv[u]));
            }
        }
    } else {
        auto add = [&](int p, float gv, int nn) {
            const int idx = (p & 0x7fffffff) - k0;
            if (idx >= 0 && idx < kc) atomicAdd(&bins[nn * kc + idx], (double)(p < 0 ? gv : -gv));
        };
        // HW % 4 == 0 and aligned tensors: four positions per lane with 128-bit loads and four such groups in
        // flight (one position per trip, the index first and the gradient after it, left a wave waiting out two
        // memory latencies per 256 bytes).  Images and positions form one index space, so that every lane of a
        // large workgroup has work even where an image's run is short.
        const bool vec_in = (d.HW & 3) == 0 && ((reinterpret_cast<uintptr_t>(grad_output) | reinterpret_cast<uintptr_t>(pos)) & 15u) == 0;
        if (vec_in) {
            const int quads = run / 4, hwq = d.HW / 4;
            const long total = (long)(b1 - b0) * quads;
            constexpr int U = 4;
            for (long i0 = threadIdx.x; i0 < total; i0 += (long)U * NT) {
                int4 pv[U];
                float4 gv[U];
                int nn[U];
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const long i = i0 + (long)u * NT < total ? i0 + (long)u * NT : i0;   // past the end: the first again, not added
                    const int bb = (int)(i / quads), q = (int)(i - (long)bb * quads);
                    const size_t o = (size_t)(b0 + bb) * img_stride + first + (size_t)q * 4;
                    pv[u] = *reinterpret_cast<const int4*>(pos + o);
                    gv[u] = *reinterpret_cast<const float4*>(grad_output + o);
                    nn[u] = q / hwq;
                }
#pragma unroll
                for (int u = 0; u < U; u++) {
                    if (u == 0 || i0 + (long)u * NT < total) {
                        add(pv[u].x, gv[u].x, nn[u]); add(pv[u].y, gv[u].y, nn[u]);
                        add(pv[u].z, gv[u].z, nn[u]); add(pv[u].w, gv[u].w, nn[u]);
                    }
                }
            }
        } else {
            const long total = (long)(b1 - b0) * run;
            for (long i = threadIdx.x; i < total; i += NT) {
                const int bb = (int)(i / run), e = (int)(i - (long)bb * run);
                const size_t o = (size_t)(b0 + bb) * img_stride + first + e;
                add(pos[o], grad_output[o], e / d.HW);
            }
        }
    }
    __syncthreads();

    if (vec && OVERWRITE) {
        const int kc4 = kc / 4;
        for (int e = threadIdx.x; e < nb * kc4; e += NT) {
            const int nn = e / kc4, k4 = e - nn * kc4;
            float* dst = grad_weight + ((size_t)g * d.NG + n0 + nn) * d.K + k0 + k4 * 4;
            const double2* b = reinterpret_cast<const double2*>(bins) + 2 * e;   // nn * kc + 4 * k4, kc a multiple of four
            const double2 lo = b[0], hi = b[1];
            *reinterpret_cast<float4*>(dst) = make_float4((float)lo.x, (float)lo.y, (float)hi.x, (float)hi.y);
        }
        return;
    }
    for (int e = threadIdx.x; e < nb * kc; e += NT) {
        const int nn = e / kc, k = e - nn * kc;
        float* dst = grad_weight + ((size_t)g * d.NG + n0 + nn) * d.K + k0 + k;
        const double v = bins[e];
        if (OVERWRITE) {
            *dst = (float)v;
        } else if (v != 0.0) {
            *dst = (float)((double)*dst + v);
        }
    }
}

template <bool OVERWRITE>
__global__ void __launch_bounds__(1024)
inf_backward_weight_kernel(const float* __restrict__ grad_output, const int32_t* __restrict__ pos,
                           float* __restrict__ grad_weight, BwdDims d, int NB, int KC, int n_blocks) {
    extern __shared__ __align__(16) unsigned char bin_bytes[];
    backward_weight_body<OVERWRITE>(reinterpret_cast<double*>(bin_bytes), blockIdx.x, blockIdx.y, grad_output, pos, grad_weight,
                                    d, NB, KC, n_blocks);
}

// ---- grad_weight of a fully connected layer: bins of one row ---------------------------------
// The kernel above keeps bins for all rows of its block; for K = 5120 one row of doubles is 40 KB, so a block of rows
// would leave a CU with one workgroup, which waits in turn for its reads and (before it can leave) for its stores.
// Here a workgroup still reads a block of NBR rows at once (NBR * 4 bytes of every image's row), keeps the values in
// registers and then takes the rows one after the other through bins of a single row: add, write the row and put the
// zeros back.  Four workgroups then wait side by side on a CU.
constexpr int kRowBinsPre = 8;   // values per lane: 2048 per block
template <bool OVERWRITE>
__device__ __forceinline__ void backward_weight_rowbins(double* bins, int bx, const float* __restrict__ grad_output,
                                                        const int32_t* __restrict__ pos, float* __restrict__ grad_weight,
                                                        const BwdDims& d, int NBR, int n_blocks) {
    constexpr int NT = 256;
    const int K = d.K, tid = threadIdx.x;
    const int idb = bx % n_blocks, g = bx / n_blocks;
    const int nblk = (n_blocks & 7) == 0 ? (idb % 8) * (n_blocks / 8) + idb / 8 : idb;   // see backward_weight_body
    const int n0 = nblk * NBR;
    if (n0 >= d.NG) return;
    const int nb = min(NBR, d.NG - n0);
    const int total = d.B * nb;                    // <= kRowBinsPre * NT: the launcher's condition
    const size_t img_stride = (size_t)d.G * d.NG, first = (size_t)g * d.NG + n0;
    int p[kRowBinsPre], nn[kRowBinsPre];
    float gv[kRowBinsPre];
#pragma unroll
    for (int u = 0; u < kRowBinsPre; u++) {
        const int i = tid + NT * u;
        const int ii = i < total ? i : 0;          // past the end: element 0 again, never added
        const int bb = ii / nb;
        nn[u] = i < total ? ii - bb * nb : -1;
        const size_t o = (size_t)bb * img_stride + first + (ii - bb * nb);
        p[u] = pos[o];
        gv[u] = grad_output[o];
    }
    const bool vec = (K & 3) == 0 && (reinterpret_cast<uintptr_t>(grad_weight) & 15u) == 0;
    if ((K & 1) == 0) {
        for (int e = tid; e < K / 2; e += NT) reinterpret_cast<double2*>(bins)[e] = make_double2(0.0, 0.0);
    } else {
        for (int e = tid; e < K; e += NT) bins[e] = 0.0;
    }
    __syncthreads();
    for (int r = 0; r < nb; r++) {
#pragma unroll
        for (int u = 0; u < kRowBinsPre; u++) {
            const int idx = p[u] & 0x7fffffff;
            if (nn[u] == r && idx < K) atomicAdd(&bins[idx], (double)(p[u] < 0 ? gv[u] : -gv[u]));
        }
        __syncthreads();
        float* row = grad_weight + (first + r) * K;
        if (vec) {
            for (int e = tid; e < K / 4; e += NT) {
                double2* b2 = reinterpret_cast<double2*>(bins) + 2 * e;
                const double2 lo = b2[0], hi = b2[1];
                float4* dst = reinterpret_cast<float4*>(row) + e;
                if (OVERWRITE) {
                    *dst = make_float4((float)lo.x, (float)lo.y, (float)hi.x, (float)hi.y);
                } else if (lo.x != 0.0 || lo.y != 0.0 || hi.x != 0.0 || hi.y != 0.0) {
                    const float4 o = *dst;
                    *dst = make_float4((float)((double)o.x + lo.x), (float)((double)o.y + lo.y), (float)((double)o.z + hi.x),
                                       (float)((double)o.w + hi.y));
                }
                b2[0] = make_double2(0.0, 0.0);
                b2[1] = make_double2(0.0, 0.0);
            }
        } else {
            for (int e = tid; e < K; e += NT) {
                const double v = bins[e];
                if (OVERWRITE) row[e] = (float)v;
                else if (v != 0.0) row[e] = (float)((double)row[e] + v);
                bins[e] = 0.0;
            }
        }
        __syncthreads();
    }
}

template <bool OVERWRITE>
__global__ void __launch_bounds__(256)
inf_backward_weight_rowbins_kernel(const float* __restrict__ grad_output, const int32_t* __restrict__ pos,
                                   float* __restrict__ grad_weight, BwdDims d, int NBR, int n_blocks) {
    extern __shared__ __align__(16) unsigned char bin_bytes[];
    backward_weight_rowbins<OVERWRITE>(reinterpret_cast<double*>(bin_bytes), blockIdx.x, grad_output, pos, grad_weight, d, NBR,
                                       n_blocks);
}

// ---- both scatters of a fully connected layer in one launch ------------------
// grad_input (a workgroup per image and group: few bytes, mostly waiting for memory) and grad_weight (a workgroup per
// block of output rows: bound by the stores of its slab) are independent.  As two launches one runs after the other;
// on two streams they overlap but pay for the joins (measured: slower).  Here the workgroups of one grid do either:
// the grad_weight workgroups come first and the grad_input workgroups last, where they run beside the tail of the
// stores (512 x 5120 x 5120, bins for whole blocks: 36.5 us against 41.5 us for the two launches; grad_input first: 39.5 us; one grad_input
// workgroup after every three of grad_weight: 46 us).  Both write their slabs whole ("overwrite"); one k range each.
struct BothPlan {
    int wgs_x, wgs_w;                 // workgroups per scatter
    int th_log2, kc_x, hw_tiles, vec; // grad_input's launch parameters
    int nb, kc_w, n_blocks;           // grad_weight's
    int rowbins;                      // grad_weight through bins of one row (backward_weight_rowbins)
};

__global__ void __launch_bounds__(256)
inf_backward_both_kernel(const float* __restrict__ grad_output, const int32_t* __restrict__ pos,
                         float* __restrict__ grad_input, float* __restrict__ grad_weight, BwdDims d, BothPlan pl) {
    extern __shared__ __align__(16) unsigned char bin_bytes[];
    const int i = blockIdx.x;
    if (i >= pl.wgs_w) {
        backward_input_body<true>(reinterpret_cast<double*>(bin_bytes), i - pl.wgs_w, 0, grad_output, pos, grad_input, d, pl.th_log2,
                                  pl.kc_x, pl.hw_tiles, pl.vec);
        return;
    }
    if (pl.rowbins)
        backward_weight_rowbins<true>(reinterpret_cast<double*>(bin_bytes), i, grad_output, pos, grad_weight, d, pl.nb, pl.n_blocks);
    else
        backward_weight_body<true>(reinterpret_cast<double*>(bin_bytes), i, 0, grad_output, pos, grad_weight, d, pl.nb, pl.kc_w,
                                   pl.n_blocks);
}

static constexpr int kBinBytes = 64 * 1024;                           // LDS bins per workgroup
static constexpr int kInputBins = kBinBytes / (int)sizeof(double);

hipError_t inf_backward_input(const float* grad_output, const int32_t* pos, float* grad_input, const Problem& pr,
                              bool overwrite, hipStream_t stream) {
    const BwdDims d{pr.B, pr.G, pr.K, pr.NG, pr.HW};
    // widest hw tile (power of two, at most 64) whose bins still cover all K channels in one pass
    int th_log2 = 0;
    while ((2 << th_log2) <= pr.HW && (2 << th_log2) <= 64 && (size_t)(2 << th_log2) * pr.K <= kInputBins) th_log2++;
    const int TH = 1 << th_log2;
    const int KC = min(pr.K, kInputBins / TH);
    const int hw_tiles = (pr.HW + TH - 1) / TH;
    const dim3 grid((unsigned)pr.B * pr.G * hw_tiles, (unsigned)((pr.K + KC - 1) / KC));
    const size_t lds = (size_t)KC * TH * sizeof(double);
    // fc layout, everything a multiple of four floats and 16-byte aligned: 128-bit path
    const int vec = pr.HW == 1 && pr.NG % 4 == 0 && pr.K % 4 == 0 && KC % 4 == 0 && aligned16(grad_output) &&
                    aligned16(pos) && aligned16(grad_input);
    // few workgroups (one per image and group in the fc layout): more lanes each keep more loads in flight
    const long wgs = (long)grid.x * grid.y;
    const long work = pr.HW == 1 ? pr.NG : (long)pr.NG * TH;        // elements scanned per workgroup
    int threads = 256;
    if (wgs < 8L * pr.num_cu && work >= 4096) threads = 512;
    if (wgs < 4L * pr.num_cu && work >= 16384) threads = 1024;
    if (overwrite)
        hipLaunchKernelGGL(inf_backward_input_kernel<true>, grid, dim3(threads), lds, stream, grad_output, pos,
                           grad_input, d, th_log2, KC, hw_tiles, vec);
    else
        hipLaunchKernelGGL(inf_backward_input_kernel<false>, grid, dim3(threads), lds, stream, grad_output, pos,
                           grad_input, d, th_log2, KC, hw_tiles, vec);
    return hipGetLastError();
}

// Launch shape of inf_backward_weight_kernel.
struct WeightPlan {
    int NB, KC, n_blocks, real_blocks, k_ranges, threads;
};

static WeightPlan plan_backward_weight(const Problem& pr) {
    WeightPlan wp{};
    const int slots = kInputBins;
    // One pass over all K channels per workgroup when a row of bins fits and the rows fill the device: every k range
    // re-reads the row's grad_output / pos.
    wp.KC = min(pr.K, slots);
    wp.NB = max(1, min(min(pr.NG, 8), slots / wp.KC));
    // fewer rows per block while the blocks do not fill the device
    while (wp.NB > 1 && (long)pr.G * ((pr.NG + wp.NB - 1) / wp.NB) < 2L * pr.num_cu) wp.NB = (wp.NB + 1) / 2;
    wp.real_blocks = (pr.NG + wp.NB - 1) / wp.NB;
    const long rows = (long)pr.G * wp.real_blocks;
    const long scanned = (long)pr.B * pr.HW * wp.NB;               // contributions a workgroup looks at
    if (rows < pr.num_cu && scanned >= 16384) {
        // still too few: k ranges of at least 16 channels (multiples of four), up to one workgroup per CU
        const int want = (int)min((long)((pr.num_cu + rows - 1) / rows), (long)max(1, wp.KC / 16));
        const int kc = ((wp.KC + want - 1) / want + 3) / 4 * 4;
        wp.KC = max(4, min(wp.KC, kc));
    }
    wp.k_ranges = (pr.K + wp.KC - 1) / wp.KC;
    // many blocks: a multiple of eight, for the kernel's XCD-aware block order (the extra workgroups leave at once)
    wp.n_blocks = wp.real_blocks >= 64 ? (wp.real_blocks + 7) / 8 * 8 : wp.real_blocks;
    // few workgroups with long scans: more lanes each keep more loads in flight
    const long wgs = rows * wp.k_ranges;
    wp.threads = 256;
    if (wgs < 8L * pr.num_cu && scanned >= 8192) wp.threads = 512;
    if (wgs < 4L * pr.num_cu && scanned >= 32768) wp.threads = 1024;
    return wp;
}

// Rows per block for the kernel with bins of one row (0: the layer does not take it): fully connected layout, a
// block's values fit the lanes' registers, one k range, and enough blocks to keep four workgroups on every CU.
static int rowbins_rows(const Problem& pr) {
    if (pr.HW != 1 || pr.K > kInputBins) return 0;
    const int nbr = min(pr.NG, min(4, (kRowBinsPre * 256) / max(pr.B, 1)));
    if (nbr < 2 || (long)pr.G * ((pr.NG + nbr - 1) / nbr) < 4L * pr.num_cu) return 0;
    return nbr;
}

hipError_t inf_backward_weight(const float* grad_output, const int32_t* pos, float* grad_weight, const Problem& pr,
                               bool overwrite, hipStream_t stream) {
    const BwdDims d{pr.B, pr.G, pr.K, pr.NG, pr.HW};
    if (const int nbr = rowbins_rows(pr)) {   // bins of one row, see backward_weight_rowbins
        const int blocks_r = (pr.NG + nbr - 1) / nbr;
        const int nblocks_r = blocks_r >= 64 ? (blocks_r + 7) / 8 * 8 : blocks_r;
        const dim3 grid((unsigned)(pr.G * nblocks_r));
        const size_t lds = (size_t)pr.K * sizeof(double);
        if (overwrite)
            hipLaunchKernelGGL(inf_backward_weight_rowbins_kernel<true>, grid, dim3(256), lds, stream, grad_output, pos,
                               grad_weight, d, nbr, nblocks_r);
        else
            hipLaunchKernelGGL(inf_backward_weight_rowbins_kernel<false>, grid, dim3(256), lds, stream, grad_output, pos,
                               grad_weight, d, nbr, nblocks_r);
        return hipGetLastError();
    }
    const WeightPlan wp = plan_backward_weight(pr);
    const dim3 grid((unsigned)(pr.G * wp.n_blocks), (unsigned)wp.k_ranges);
    const size_t lds = (size_t)wp.NB * wp.KC * sizeof(double);
    if (overwrite)
        hipLaunchKernelGGL(inf_backward_weight_kernel<true>, grid, dim3(wp.threads), lds, stream, grad_output, pos, grad_weight, d,
                           wp.NB, wp.KC, wp.n_blocks);
    else
        hipLaunchKernelGGL(inf_backward_weight_kernel<false>, grid, dim3(wp.threads), lds, stream, grad_output, pos, grad_weight, d,
                           wp.NB, wp.KC, wp.n_blocks);
    return hipGetLastError();
}

// Both scatters of a layer, each writing its gradient whole.  One launch (inf_backward_both_kernel) for the fully
// connected layout when each scatter is a single k range and grad_weight needs no split over the images; otherwise
// the two launches of the separate entry points.
hipError_t inf_backward_both(const float* grad_output, const int32_t* pos, float* grad_input, float* grad_weight,
                             const Problem& pr, hipStream_t stream) {
    const int nbr = rowbins_rows(pr);
    const bool rowbins = nbr > 0;
    const WeightPlan wp = plan_backward_weight(pr);
    const int nb = rowbins ? nbr : wp.NB;
    const int real_blocks = (pr.NG + nb - 1) / nb;
    const int n_blocks = real_blocks >= 64 ? (real_blocks + 7) / 8 * 8 : real_blocks;
    const long wgs_x = (long)pr.B * pr.G, wgs_w = (long)pr.G * n_blocks;
    // one launch of 256-lane workgroups: grad_weight as one k range per block of rows, enough blocks to fill the device
    const bool one_launch = pr.HW == 1 && pr.K <= kInputBins && (rowbins || (wp.k_ranges == 1 && wp.threads == 256)) &&
                            (long)pr.G * real_blocks >= 2L * pr.num_cu && wgs_x + wgs_w < (1L << 31);
    if (!one_launch) {
        if (hipError_t e = inf_backward_input(grad_output, pos, grad_input, pr, true, stream); e != hipSuccess) return e;
        return inf_backward_weight(grad_output, pos, grad_weight, pr, true, stream);
    }
    const BwdDims d{pr.B, pr.G, pr.K, pr.NG, pr.HW};
    BothPlan pl{};
    pl.wgs_x = (int)wgs_x;
    pl.wgs_w = (int)wgs_w;
    pl.th_log2 = 0;
    pl.kc_x = pr.K;
    pl.hw_tiles = 1;
    pl.vec = pr.NG % 4 == 0 && pr.K % 4 == 0 && aligned16(grad_output) && aligned16(pos) && aligned16(grad_input);
    pl.nb = nb;
    pl.kc_w = pr.K;
    pl.n_blocks = n_blocks;
    pl.rowbins = rowbins;
    const size_t lds = (size_t)(rowbins ? 1 : nb) * pr.K * sizeof(double);
    hipLaunchKernelGGL(inf_backward_both_kernel, dim3((unsigned)(wgs_x + wgs_w)), dim3(256), lds, stream, grad_output, pos,
                       grad_input, grad_weight, d, pl);
    return hipGetLastError();
}

}  // namespace ldist
