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
// The bins of grad_input (and of grad_weight in the conv layout) are doubles: on gfx950 an LDS atomic add of a
// double (ds_add_f64) retires about nine times as many lanes per clock as one of a float (ds_add_f32: 0.33 lanes
// per clock and CU, measured on random addresses; 2.9 for doubles, 6 for 32-bit integer adds), and the binning was
// what those kernels waited for.  A bin's sum is rounded to float once, when the slab is written: exact where an
// element receives one contribution, otherwise at least as close to the true sum as any order of float additions.
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
                float4 o = dst[e];
                o.x += v.x; o.y += v.y; o.z += v.z; o.w += v.w;
                dst[e] = o;
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
                    float4 o = *dst;
                    o.x += v.x; o.y += v.y; o.z += v.z; o.w += v.w;
                    *dst = o;
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
            const float v = (float)bins[e];
            if (OVERWRITE) *dst = v;
            else if (v != 0.f) *dst += v;
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
// Workgroup = (group g, NB consecutive outputs n, KC consecutive k -- all of K when
// a row of bins fits in 64 KB -- and a slice of the images b).  For one image the NB rows of grad_output/pos are one
// contiguous run of NB*HW elements.  bins[nb][kc].
// When the images are split over several workgroups (SPLIT) the bins are added
// to grad_weight with global atomics, otherwise the workgroup is the only
// writer of its slab.
// BIN: float bins in the fc layout (a row of bins receives at most one contribution per image, and what the kernel
// waits for are its strided reads of grad_output / pos columns: twice the rows per workgroup count for more than
// faster atomics), double bins otherwise (B * HW contributions per row: 131 072 in a 3x3 conv layer of 32 x 32
// images at batch 128, where the float atomics took three times as long as everything else).
template <bool OVERWRITE, bool SPLIT, class BIN>
__device__ __forceinline__ void backward_weight_body(BIN* bins, int bx, int by, int bz, const float* __restrict__ grad_output,
                                                     const int32_t* __restrict__ pos, float* __restrict__ grad_weight,
                                                     const BwdDims& d, int NB, int KC, int n_blocks, int b_per_wg) {
    constexpr int NT = 256;
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
    const int b0 = bz * b_per_wg;
    const int b1 = min(d.B, b0 + b_per_wg);
    // kc is a multiple of 4 whenever vec is set, so rows of bins and of grad_weight stay 16-byte aligned
    const bool vec = (kc & 3) == 0 && (d.K & 3) == 0 && (reinterpret_cast<uintptr_t>(grad_weight) & 15u) == 0;
    if (vec) {   // 16 bytes of bins per store
        float4* b4 = reinterpret_cast<float4*>(bins);
        for (int e = threadIdx.x; e < nb * kc * (int)sizeof(BIN) / 16; e += NT) b4[e] = make_float4(0.f, 0.f, 0.f, 0.f);
    } else {
        for (int e = threadIdx.x; e < nb * kc; e += NT) bins[e] = (BIN)0;
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
                if ((u == 0 || i0 + NT * u < total) && idx >= 0 && idx < kc) {
                    // A float add in LDS retires a third of a lane per clock and CU, an exchange some six lanes.  A
                    // row of bins takes one contribution per image, so most bins take none or one: the value goes in
                    // by exchange, and what it displaced (another image's contribution to the same bin: some five in
                    // a hundred) is added back with the slow instruction.  Whatever the interleaving, every
                    // displaced value is added exactly once.
                    BIN* bin = &bins[nn[u] * kc + idx];
                    const BIN v = (BIN)(p[u] < 0 ? gv[u] : -gv[u]);
                    if constexpr (sizeof(BIN) == sizeof(float)) {
                        const float displaced = atomicExch(reinterpret_cast<float*>(bin), (float)v);
                        if (displaced != 0.f) atomicAdd(reinterpret_cast<float*>(bin), displaced);
                    } else {
                        atomicAdd(bin, v);
                    }
                }
            }
        }
    } else {
        auto add = [&](int p, float gv, int nn) {
            const int idx = (p & 0x7fffffff) - k0;
            if (idx >= 0 && idx < kc) atomicAdd(&bins[nn * kc + idx], (BIN)(p < 0 ? gv : -gv));
        };
        // HW % 4 == 0 and aligned tensors: four positions per lane with 128-bit loads and two such groups in
        // flight (one position per trip, the index first and the gradient after it, left a wave waiting out two
        // memory latencies per 256 bytes)
        const bool vec_in = (d.HW & 3) == 0 && ((reinterpret_cast<uintptr_t>(grad_output) | reinterpret_cast<uintptr_t>(pos)) & 15u) == 0;
        for (int b = b0; b < b1; b++) {
            const size_t base = (size_t)b * img_stride + first;
            if (vec_in) {
                const int4* pq = reinterpret_cast<const int4*>(pos + base);
                const float4* gq = reinterpret_cast<const float4*>(grad_output + base);
                const int quads = run / 4, hwq = d.HW / 4;
                for (int q0 = threadIdx.x; q0 < quads; q0 += 2 * NT) {
                    const int q1 = q0 + NT < quads ? q0 + NT : q0;
                    const int4 pa = pq[q0], pb = pq[q1];
                    const float4 ga = gq[q0], gb = gq[q1];
                    const int na = q0 / hwq;
                    add(pa.x, ga.x, na); add(pa.y, ga.y, na); add(pa.z, ga.z, na); add(pa.w, ga.w, na);
                    if (q1 != q0) {
                        const int nb_ = q1 / hwq;
                        add(pb.x, gb.x, nb_); add(pb.y, gb.y, nb_); add(pb.z, gb.z, nb_); add(pb.w, gb.w, nb_);
                    }
                }
            } else {
                for (int e = threadIdx.x; e < run; e += NT) add(pos[base + e], grad_output[base + e], e / d.HW);
            }
        }
    }
    __syncthreads();

    if (vec && OVERWRITE && !SPLIT) {
        const int kc4 = kc / 4;
        for (int e = threadIdx.x; e < nb * kc4; e += NT) {
            const int nn = e / kc4, k4 = e - nn * kc4;
            float* dst = grad_weight + ((size_t)g * d.NG + n0 + nn) * d.K + k0 + k4 * 4;
            const BIN* b = bins + 4 * e;   // nn * kc + 4 * k4, kc a multiple of four
            *reinterpret_cast<float4*>(dst) = make_float4((float)b[0], (float)b[1], (float)b[2], (float)b[3]);
        }
        return;
    }
    for (int e = threadIdx.x; e < nb * kc; e += NT) {
        const int nn = e / kc, k = e - nn * kc;
        float* dst = grad_weight + ((size_t)g * d.NG + n0 + nn) * d.K + k0 + k;
        const float v = (float)bins[e];
        if (SPLIT) {
            if (v != 0.f) atomicAdd(dst, v);
        } else if (OVERWRITE) {
            *dst = v;
        } else if (v != 0.f) {
            *dst += v;
        }
    }
}

template <bool OVERWRITE, bool SPLIT, class BIN>
__global__ void __launch_bounds__(256)
inf_backward_weight_kernel(const float* __restrict__ grad_output, const int32_t* __restrict__ pos,
                           float* __restrict__ grad_weight, BwdDims d, int NB, int KC, int n_blocks, int b_per_wg) {
    extern __shared__ __align__(16) unsigned char bin_bytes[];
    backward_weight_body<OVERWRITE, SPLIT, BIN>(reinterpret_cast<BIN*>(bin_bytes), blockIdx.x, blockIdx.y, blockIdx.z,
                                                grad_output, pos, grad_weight, d, NB, KC, n_blocks, b_per_wg);
}

// ---- grad_weight of a fully connected layer, written whole: bins of one row ----------------
// The kernel above keeps bins for all rows of its block, 60 KB for three rows of K = 5120, so two workgroups share a
// CU, and each of them waits in turn for its reads and (before it can leave) for its stores.  Here a workgroup still
// reads a block of NBR rows at once (NBR * 4 bytes of every image's row), keeps the values in registers and then
// takes the rows one after the other through bins of a single row: add, store the row and put the zeros back.  The
// bins are a third of the size, so three times the workgroups wait side by side.
constexpr int kRowBinsPre = 8;   // values per lane: 2048 per block
__device__ __forceinline__ void backward_weight_rowbins(float* bins, int bx, const float* __restrict__ grad_output,
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
    for (int e = tid; e < K; e += NT) bins[e] = 0.f;
    __syncthreads();
    const bool vec = (K & 3) == 0 && (reinterpret_cast<uintptr_t>(grad_weight) & 15u) == 0;
    for (int r = 0; r < nb; r++) {
#pragma unroll
        for (int u = 0; u < kRowBinsPre; u++) {
            const int idx = p[u] & 0x7fffffff;
            if (nn[u] == r && idx < K) {           // by exchange, displaced values added back: see backward_weight_body
                const float displaced = atomicExch(&bins[idx], p[u] < 0 ? gv[u] : -gv[u]);
                if (displaced != 0.f) atomicAdd(&bins[idx], displaced);
            }
        }
        __syncthreads();
        float* row = grad_weight + (first + r) * K;
        if (vec) {
            for (int e = tid; e < K / 4; e += NT) {
                float4* b4 = reinterpret_cast<float4*>(bins) + e;
                reinterpret_cast<float4*>(row)[e] = *b4;
                *b4 = make_float4(0.f, 0.f, 0.f, 0.f);
            }
        } else {
            for (int e = tid; e < K; e += NT) { row[e] = bins[e]; bins[e] = 0.f; }
        }
        __syncthreads();
    }
}

__global__ void __launch_bounds__(256)
inf_backward_weight_rowbins_kernel(const float* __restrict__ grad_output, const int32_t* __restrict__ pos,
                                   float* __restrict__ grad_weight, BwdDims d, int NBR, int n_blocks) {
    extern __shared__ __align__(16) unsigned char bin_bytes[];
    backward_weight_rowbins(reinterpret_cast<float*>(bin_bytes), blockIdx.x, grad_output, pos, grad_weight, d, NBR, n_blocks);
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
        backward_weight_rowbins(reinterpret_cast<float*>(bin_bytes), i, grad_output, pos, grad_weight, d, pl.nb, pl.n_blocks);
    else
        backward_weight_body<true, false, float>(reinterpret_cast<float*>(bin_bytes), i, 0, 0, grad_output, pos, grad_weight,
                                                 d, pl.nb, pl.kc_w, pl.n_blocks, d.B);
}

__global__ void __launch_bounds__(256) fill_zero_kernel(float* __restrict__ p, size_t n) {
    const size_t stride = (size_t)gridDim.x * 256 * 4;
    for (size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4; i < n; i += stride) {
        if (i + 4 <= n && (reinterpret_cast<uintptr_t>(p + i) & 15u) == 0) {
            *reinterpret_cast<float4*>(p + i) = make_float4(0.f, 0.f, 0.f, 0.f);
        } else {
            for (size_t j = i; j < n && j < i + 4; j++) p[j] = 0.f;
        }
    }
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

template <bool OVERWRITE, bool SPLIT, class BIN>
static void launch_backward_weight(dim3 grid, size_t lds, hipStream_t stream, const float* grad_output, const int32_t* pos,
                                   float* grad_weight, const BwdDims& d, int NB, int KC, int n_blocks, int b_per_wg) {
    hipLaunchKernelGGL((inf_backward_weight_kernel<OVERWRITE, SPLIT, BIN>), grid, dim3(256), lds, stream, grad_output, pos,
                       grad_weight, d, NB, KC, n_blocks, b_per_wg);
}

hipError_t inf_backward_weight(const float* grad_output, const int32_t* pos, float* grad_weight, const Problem& pr,
                               bool overwrite, hipStream_t stream) {
    const BwdDims d{pr.B, pr.G, pr.K, pr.NG, pr.HW};
    const bool wide = pr.HW > 1;   // double bins, see the kernel
    const int slots = kBinBytes / (wide ? (int)sizeof(double) : (int)sizeof(float));
    // One pass over all K channels per workgroup when a row of bins fits: re-reading the strided
    // grad_output/pos columns for every channel range costs more than the smaller row block.
    const int KC = min(pr.K, slots);
    const int NB = max(1, min(min(pr.NG, 8), slots / KC));
    const int real_blocks = (pr.NG + NB - 1) / NB;
    // many blocks: a multiple of eight, for the kernel's XCD-aware block order (the extra workgroups leave at once)
    const int n_blocks = real_blocks >= 64 ? (real_blocks + 7) / 8 * 8 : real_blocks;
    const int k_ranges = (pr.K + KC - 1) / KC;
    const long slabs = (long)pr.G * real_blocks * k_ranges;
    // split the images over workgroups only when the slabs alone cannot fill the device
    int splits = 1;
    if (slabs < 2L * pr.num_cu) {
        const long rows = (long)pr.B * pr.HW;
        const long by_work = max(1L, rows * NB / 16384);  // keep at least 16K contributions per workgroup
        splits = (int)min((long)pr.B, min(by_work, (4L * pr.num_cu + slabs - 1) / slabs));
        if (splits > 65535) splits = 65535;
    }
    const int b_per_wg = (pr.B + splits - 1) / splits;
    splits = (pr.B + b_per_wg - 1) / b_per_wg;
    const dim3 grid((unsigned)(pr.G * n_blocks), (unsigned)k_ranges, (unsigned)splits);
    const size_t lds = (size_t)NB * KC * (wide ? sizeof(double) : sizeof(float));
#define LDIST_BWD_W(OVER, SPLIT)                                                                                        \
    do {                                                                                                                \
        if (wide) launch_backward_weight<OVER, SPLIT, double>(grid, lds, stream, grad_output, pos, grad_weight, d, NB, KC, \
                                                              n_blocks, b_per_wg);                                      \
        else launch_backward_weight<OVER, SPLIT, float>(grid, lds, stream, grad_output, pos, grad_weight, d, NB, KC,     \
                                                        n_blocks, b_per_wg);                                            \
    } while (0)
    {   // bins of one row, see inf_backward_weight_rowbins_kernel
        const int nbr = min(pr.NG, min(4, (kRowBinsPre * 256) / max(pr.B, 1)));
        const int blocks_r = nbr > 0 ? (pr.NG + nbr - 1) / nbr : 0;
        if (!wide && overwrite && nbr >= 2 && k_ranges == 1 && (long)pr.G * blocks_r >= 4L * pr.num_cu) {
            const int nblocks_r = blocks_r >= 64 ? (blocks_r + 7) / 8 * 8 : blocks_r;
            hipLaunchKernelGGL(inf_backward_weight_rowbins_kernel, dim3((unsigned)(pr.G * nblocks_r)), dim3(256),
                               (size_t)pr.K * sizeof(float), stream, grad_output, pos, grad_weight, d, nbr, nblocks_r);
            return hipGetLastError();
        }
    }
    if (splits > 1) {
        if (overwrite) {
            const size_t n = (size_t)pr.G * pr.NG * pr.K;
            const unsigned blocks = (unsigned)min((size_t)4096, (n + 1023) / 1024);
            hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks), dim3(256), 0, stream, grad_weight, n);
        }
        LDIST_BWD_W(false, true);
    } else if (overwrite) {
        LDIST_BWD_W(true, false);
    } else {
        LDIST_BWD_W(false, false);
    }
#undef LDIST_BWD_W
    return hipGetLastError();
}

// Both scatters of a layer, each writing its gradient whole.  One launch (inf_backward_both_kernel) for the fully
// connected layout when each scatter is a single k range and grad_weight needs no split over the images; otherwise
// the two launches of the separate entry points.
hipError_t inf_backward_both(const float* grad_output, const int32_t* pos, float* grad_input, float* grad_weight,
                             const Problem& pr, hipStream_t stream) {
    const int slots_w = kBinBytes / (int)sizeof(float);
    const int nbr = min(pr.NG, min(4, (kRowBinsPre * 256) / max(pr.B, 1)));
    const bool rowbins = nbr >= 2 && (long)pr.G * ((pr.NG + nbr - 1) / nbr) >= 4L * pr.num_cu;
    const int nb = rowbins ? nbr : max(1, min(min(pr.NG, 8), slots_w / max(pr.K, 1)));
    const int real_blocks = (pr.NG + nb - 1) / nb;
    const int n_blocks = real_blocks >= 64 ? (real_blocks + 7) / 8 * 8 : real_blocks;
    const long wgs_x = (long)pr.B * pr.G, wgs_w = (long)pr.G * n_blocks;
    const bool one_launch = pr.HW == 1 && pr.K <= kInputBins && pr.K <= slots_w &&
                            (long)pr.G * real_blocks >= 2L * pr.num_cu &&   // inf_backward_weight would not split the images
                            wgs_x + wgs_w < (1L << 31);
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
    const size_t lds = std::max((size_t)pr.K * sizeof(double), (size_t)(rowbins ? 1 : nb) * pr.K * sizeof(float));
    hipLaunchKernelGGL(inf_backward_both_kernel, dim3((unsigned)(wgs_x + wgs_w)), dim3(256), lds, stream, grad_output, pos,
                       grad_input, grad_weight, d, pl);
    return hipGetLastError();
}

}  // namespace ldist
