// Both p-norm gradients of a fully connected layer in one pass over the terms (reference
// model/norm_dist_cuda.cu:294-425 computes the gradients in two kernels that each evaluate every term):
//   t[m,n,k]          = g[m,n] * (|x[m,k] - w[n,k]| / out[m,n])^(p-1) * sign(x - w)
//   grad_input [m,k]  = sum_n t[m,n,k]          grad_weight[n,k] += -sum_m t[m,n,k]
// For a general p the term is a logarithm and an exponential (v_log_f32, v_exp_f32: a quarter of the rate of
// the other instructions), and that is what bounds either gradient; sharing the term between the two sums takes
// 4.2 ms on 512 x 5120 -> 5120 at p = 20.5 where the two separate kernels take 3.6 + 3.1 ms.
//
// The kernel has the shape of the register-tiled grad_input kernel: a workgroup owns 128 rows m x BN inputs k and
// walks the outputs n; a lane keeps an 8 x TN patch of x and of the grad_input sums (BN x TN = 80 x 5, 64 x 4 or
// 48 x 3: the host takes the width whose tiles fill the device best).  For grad_weight the lane
// also adds, per output n, its eight rows' terms of each of its TN columns (one more fused multiply-add per term),
// the sixteen lanes that share those columns (one DPP row: the lane index runs along m first here) add their
// partial sums over each half of the row with three row shifts, the halves' last lanes park the two totals of the
// tile's 128 rows in two LDS tiles [stage's outputs][BN], and once per stage the whole workgroup adds the tiles'
// sum onto grad_weight with float atomics
// (64 consecutive columns per instruction).  grad_weight therefore collects one addend per tile of 128 rows, in no
// fixed order, and must be zero-filled (or hold the values to accumulate onto) by the caller, as with the separate
// call.  IE = 0: any p > 2; the power is taken of the normalised difference (x - w) / out, which never leaves the
// float range.
//
// IE = p - 1 for the multiply-only exponents (1, 2, 3, 7).  There the two register-tiled kernels of
// norm_backward_tiled.hip each spend a subtraction and the multiplications of the power on every term before their
// one fused multiply-add; here the term is shared and each sum costs its fused multiply-add only (p = 8: 7.9 vector
// instructions per term for both sums, counted in the loop, instead of 7.1 + 6.5), and x, w, g and out are staged
// once.  As in those kernels the power is taken of the raw difference with F = g / out^(p-1) staged in place of g,
// and a stage that holds an output outside [2^-12, 2^12] is reduced the careful way from g and 1/out.  The loop does
// not fetch the next row's operands ahead: with a second fragment in flight the kernel spills, and what it spills it
// reloads behind the stage's global loads, so that every wait for a reloaded value waits for those as well (measured:
// no faster than this form).  What keeps it from the rate its instruction count promises (1.6 ms at p = 8) is the
// time its waves do not issue arithmetic: 20 % of it at waits (each row's LDS fetch, the stage's loads), as much again
// at the stage's barriers, the conversion and the flush, which nothing overlaps with one workgroup per CU.
#include "fwd_engine.hpp"
#include "pow.hpp"
#include "wave_reduce.hpp"

namespace ldist {

template <class GEO, int IE>
__global__ void __launch_bounds__(GEO::NT, 2)
norm_backward_fused_kernel(const float* __restrict__ grad_output, const float* __restrict__ input,
                           const float* __restrict__ weight, const float* __restrict__ output,
                           float* __restrict__ grad_input, float* __restrict__ grad_weight, float e, Dims d) {
    constexpr int BM = GEO::BM, BN = GEO::BN, TM = GEO::TM, TN = GEO::TN, KS = GEO::KS, KK = GEO::KK;
    constexpr int NGRP = GEO::NGRP, NT = GEO::NT, XS = GEO::XS, WS = GEO::WS;
    constexpr int STAGE = 2 * XS + WS;     // [F or g][1/out][w]
    static_assert(GEO::TY == 16, "the lanes that share a column fill one DPP row");
    using RowLoad = RowsK<BM, GEO::SM, NT, KK, 4>;   // outputs are contiguous in g and out
    using ColLoad = RowsT<BN, GEO::SN, NT, KK, 4>;
    static_assert((KS - 1) * TM * TN * NGRP <= STAGE, "merge area fits in the panels");
    extern __shared__ __align__(16) float lds[];

    int tm, tk, g;
    tile_of_block(d, tm, tk, g);
    const int m0 = tm * BM, k0 = tk * BN;
    const int tid = threadIdx.x;
    const int grp = tid / NGRP, t = tid % NGRP;
    const int ty = t % GEO::TY, tx = t / GEO::TY;    // m first: the 16 lanes of a column group are neighbours
    const int K = d.K, NG = d.NG;

    // sign(u) * |u|^(p-1).  IE == 0: as u * |u|^(p-2) (the host sends exponents p <= 2 to the separate kernels);
    // u == 0 gives 0
    const float em1 = in_vgpr(e - 1.0f);
    const float em2 = em1;   // p - 2: the exponent of |x - w| beside the factor (x - w) itself
    auto spower = [&](float u) {   // by reference: the integer-exponent instantiations do not use em1
        if constexpr (IE == 0) return spow_by_mul(u, em1);
        else if constexpr (IE == 1) return u;
        else if constexpr (IE == 2) return u * __builtin_fabsf(u);
        else return pow_int<IE>(u);
    };

    // the lane's patch of x, and where its columns' sums go in grad_weight (row n = 0 of group g)
    float q[TM][TN], acc[TM][TN];
    int wcol[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int k = k0 + GEO::col(tx, j);
        wcol[j] = k < K ? k : -1;
    }
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int m = m0 + GEO::row(ty, i);
#pragma unroll
        for (int j = 0; j < TN; j++) {
            acc[i][j] = 0.f;
            q[i][j] = (m < d.M && wcol[j] >= 0) ? input[((size_t)m * d.G + g) * K + wcol[j]] : 0.f;
        }
    }
    float* const gw_group = grad_weight + (size_t)g * NG * K;
    // The lane's column sums of output n (already summed over its rows) are summed over each half of the 16 lanes
    // that share the columns (three DPP row shifts; lanes 7 and 15 of the row hold the halves' totals) and parked in
    // two LDS tiles [stage's outputs][BN columns], one per half; the sign: d/dw of |x - w| is minus d/dx.  The fourth
    // shift, which would join the halves, costs more than the second tile: a DPP instruction takes 4.4 clocks, the
    // twenty-five of a step (five sums) were a quarter of the p = 8 launch, and without the last level 2.51 -> 2.28 ms
    // on 512 x 5120 -> 5120.  (LDS float atomics from the four quarter totals instead: 3.13 ms.)  The tiles go
    // onto grad_weight once per stage (flush_weight_tile): straight from here an atomic instruction had four active
    // lanes (the last lane of each row of sixteen), and the float atomics of a 5120-wide layer, 105 M in 26 M
    // instructions, took 1.7 ms of the launch's 4.2.
    float* const Gs = lds + 2 * XS + GEO::WS;   // 2 x [KK][BN], all zero between stages
    auto add_weight_row = [&](int n_local, const float (&s)[TN]) {
        float tot[TN];
#pragma unroll
        for (int j = 0; j < TN; j++) tot[j] = dpp_lanes_total<8>(s[j]);
        if ((ty & 7) == 7) {
            float* half = Gs + (ty >> 3) * (KK * BN);
#pragma unroll
            for (int j = 0; j < TN; j++) half[n_local * BN + GEO::col(tx, j)] = -tot[j];
        }
    };
    // All lanes of the workgroup: 64 consecutive columns of one output per wave instruction; two parked zeros (nothing
    // added: padding, or a row the large-exponent path passed over) cost no atomic.  Leaves the tiles zero.
    auto flush_weight_tile = [&](int n_first) {
        for (int i = tid; i < KK * BN; i += GEO::NT) {
            const float a = Gs[i], b = Gs[i + KK * BN];
            if (a != 0.f || b != 0.f) {
                Gs[i] = 0.f;
                Gs[i + KK * BN] = 0.f;
                const int nl = i / BN, c = i - nl * BN;
                if (n_first + nl < NG && k0 + c < K) atomicAdd(gw_group + (size_t)(n_first + nl) * K + k0 + c, a + b);
            }
        }
    };

    // ---- staging: g and out (rows m, reduction n) and the weights of the stage's outputs ----
    RowLoad gk, ok_;
    ColLoad wl;
    const float* gbase = grad_output + ((size_t)m0 * d.G + g) * NG;
    const float* obase = output + ((size_t)m0 * d.G + g) * NG;
    const float* wbase = weight + (size_t)g * NG * K;
    // Buffer loads whose byte offsets are worked out again from the lane's number at every stage (a handful of
    // instructions per vector) instead of being kept: kept across the k loop, the eleven offsets (or, before them,
    // eleven 64-bit addresses) were spilled, and a spilled value that the loop needs is reloaded behind the stage's
    // loads, so that the loop's wait for it also waits for them -- the whole workgroup then stands still until the
    // next stage's panels have arrived.  An offset of all ones lies outside the descriptors' 2 GB range and reads as
    // zeros, which stands for every predicate: rows past the matrix (they must not add to grad_weight), outputs past
    // NG in the last stage, columns past K, lanes without a vector in a round.
    const __amdgpu_buffer_rsrc_t g_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(gbase), 0, (int)0x80000000u, 0x00020000);
    const __amdgpu_buffer_rsrc_t o_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(obase), 0, (int)0x80000000u, 0x00020000);
    typedef float F4 __attribute__((ext_vector_type(4)));
    auto load = [&](int n_first) {
        int lane = tid;
        asm volatile("" : "+v"(lane));   // opaque: keeps the offsets below from being computed once and carried along
        {   // g and out: rows m of the tile, 16 vectors of four outputs per row
            static_assert(RowLoad::PER_ROW == 16 && NT % RowLoad::PER_ROW == 0, "a lane keeps its outputs over the rounds");
            const int row0 = lane / RowLoad::PER_ROW, nq = (lane % RowLoad::PER_ROW) * 4;
            const unsigned ldb = 4u * (unsigned)(d.G * NG);
            const bool n_ok = n_first + nq < NG;                      // NG % 4 == 0: a vector is inside or outside
            const int rows_valid = d.M - m0;
#pragma unroll
            for (int i = 0; i < RowLoad::N; i++) {
                const int row = row0 + i * (NT / RowLoad::PER_ROW);
                const unsigned o = (n_ok && row < rows_valid && row < BM) ? (unsigned)row * ldb + 4u * nq : ~0u;
                const F4 gv = __builtin_bit_cast(F4, __builtin_amdgcn_raw_buffer_load_b128(g_rsrc, o, n_first * 4, 0));
                const F4 ov = __builtin_bit_cast(F4, __builtin_amdgcn_raw_buffer_load_b128(o_rsrc, o, n_first * 4, 0));
                gk.v[i][0] = gv.x; gk.v[i][1] = gv.y; gk.v[i][2] = gv.z; gk.v[i][3] = gv.w;
                ok_.v[i][0] = ov.x; ok_.v[i][1] = ov.y; ok_.v[i][2] = ov.z; ok_.v[i][3] = ov.w;
            }
        }
        {   // weights: the stage's outputs n_first .. n_first + KK - 1, BN / 4 vectors of four columns per output
            const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<float*>(wbase + (size_t)n_first * K + k0), 0, (int)0x80000000u, 0x00020000);
#pragma unroll
            for (int i = 0; i < ColLoad::N; i++) {
                const int id = lane + i * NT;
                const int rr = id / ColLoad::PER_ROW, cq = id - rr * ColLoad::PER_ROW;
                const bool ok = (ColLoad::TOTAL % NT == 0 || id < ColLoad::TOTAL) && n_first + rr < NG && k0 + cq * 4 < K;
                const unsigned o = ok ? 4u * ((unsigned)rr * (unsigned)K + (unsigned)cq * 4u) : ~0u;
                const F4 t = __builtin_bit_cast(F4, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, o, 0, 0));
                wl.v[i][0] = t.x; wl.v[i][1] = t.y; wl.v[i][2] = t.z; wl.v[i][3] = t.w;
            }
        }
    };
    // every (row, output) pair has its own largest term among its K differences, and a row of the test holds
    // 16 pairs x 4 TN columns per wave: with a short K most rows hold one and the tests only cost
    const bool sparse = e >= 63.0f && K >= 1024;
    const float cut = __builtin_exp2f(-36.0f / e);
    // General exponent without the tests: the term g * u * |u|^(p-2), u = (x - w) / out, can be taken as
    //   g * (x - w) * exp2((p - 2) * log2|x - w| + log2(out^-(p-1))),
    // the second summand staged per (row, output) in place of 1/out: the division of every difference by its output
    // becomes part of the exponent's fused multiply-add (five plain instructions per term beside the logarithm and
    // the exponential instead of six; 4.19 -> 3.87 ms on 512 x 5120 -> 5120).  The exponent is then a difference of
    // two numbers of the size of (p - 1) * |log2 out| for the terms that count (|x - w| near out), and what the
    // hardware logarithm of either is off by, one unit in the last place of |log2 out|, becomes a relative error of
    // the term (p - 1) times as large.  A gradient whose terms cancel is held to 1e-6 * p / 8 of the sum of their
    // magnitudes, which the two errors together stay inside only while |log2 out| < 1 (2 * (p - 1) * 2^-24 * ln 2
    // = 8e-8 * (p - 1)); outputs in [1/16, 16] measured 1.07 times the tolerance on a 3x3 conv layer of one channel per
    // group at p = 47.  So the form is voted per stage, as the factored form of the multiply-only exponents is: a
    // stage whose outputs all lie in [1/2, 2] takes it, any other stage divides first.
    // What "near 1" means is settled once per workgroup: `unit` is the power of two nearest to the geometric mean of
    // the largest and the smallest output of the first stage, the lane's patch of x and every stage's weights are taken in that unit
    // (exact: powers of two), and so are the outputs, so that data of any overall magnitude takes the logarithmic
    // form; a layer whose outputs differ by more than the window does not.
    const bool logscale = IE == 0 && !sparse;
    float unit_inv = 1.0f;   // 1 / unit
    // Turns the parked out values into what the panel holds: 1/out, and 0 where nothing was loaded (padding loads g
    // and out as 0; a real 0 output gives inf like the reference), so that padding multiplies by 0, not by infinity.
    // IE > 0, factored: g becomes g / out^IE.
    auto convert = [&](bool factored) {
#pragma unroll
        for (int i = 0; i < RowLoad::N; i++)
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const bool present = ok_.v[i][c] != 0.f || gk.v[i][c] != 0.f;
                const float ri = present ? __builtin_amdgcn_rcpf(ok_.v[i][c] * unit_inv) : 0.f;   // unit_inv: 1 unless logscale
                if constexpr (IE > 0) {
                    ok_.v[i][c] = ri;
                    if (factored) gk.v[i][c] *= pow_int<IE>(ri);
                } else if (!factored) {
                    ok_.v[i][c] = ri;
                } else {
                    // general exponent, a stage in the logarithmic form: the panel holds log2 of out^-(p-1), which
                    // the term's exponent starts from; minus infinity where nothing was loaded, so that the power is 0.
                    // The logarithm is taken of the output itself (no reciprocal in between), and what the product
                    // -(p-1) * log2 out loses when it is rounded to a float goes into g as a factor.
                    const float lo = __builtin_amdgcn_logf(present ? ok_.v[i][c] * unit_inv : 1.0f);   // nothing loaded: g stays 0
                    const float hi = -e * lo;
                    gk.v[i][c] *= __builtin_amdgcn_exp2f(__builtin_fmaf(-e, lo, -hi));
                    ok_.v[i][c] = present ? hi : -__builtin_inff();
                }
            }
    };
    // logscale: the stage's weights in units of `unit`, like the lane's patch of x
    auto scale_weights = [&]() {
        if (logscale) {
#pragma unroll
            for (int i = 0; i < ColLoad::N; i++)
#pragma unroll
                for (int c = 0; c < 4; c++) wl.v[i][c] *= unit_inv;
        }
    };
    // Whether this lane parked an output outside the range of the short form (before the conversion): IE > 0, the
    // range in which out^-IE and the raw differences' powers are safe floats; IE == 0, that of the logarithmic form
    auto out_of_range = [&]() {
        bool unsafe = false;
        const float lo = IE > 0 ? 0x1p-12f : 0.5f, hi = IE > 0 ? 0x1p12f : 2.0f;
#pragma unroll
        for (int i = 0; i < RowLoad::N; i++)
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const float ov = ok_.v[i][c] * unit_inv;
                if (ok_.v[i][c] != 0.f || gk.v[i][c] != 0.f) unsafe |= !(ov >= lo && ov <= hi);
            }
        return unsafe;
    };
    auto store = [&]() {
        gk.store(lds, tid);
        ok_.store(lds + XS, tid);
        if constexpr (TN == 3) {
            // three columns per lane at a pitch of four in the panel, so that the sweep's 128-bit reads stay as they
            // are: column c of the tile lives at word (c / 3) * 4 + c % 3 of its panel row
            float* panel = lds + 2 * XS;
#pragma unroll
            for (int i = 0; i < ColLoad::N; i++) {
                const int id = tid + i * NT;
                if (ColLoad::TOTAL % NT != 0 && id >= ColLoad::TOTAL) continue;
                const int rr = id / ColLoad::PER_ROW, cq = id - rr * ColLoad::PER_ROW;
#pragma unroll
                for (int c4 = 0; c4 < 4; c4++) {
                    const int c = cq * 4 + c4, third = c / 3;
                    panel[rr * GEO::SN + ((third * 4 + (c - third * 3)) ^ swz(rr))] = wl.v[i][c4];
                }
            }
        } else {
            wl.store(lds + 2 * XS, tid);
        }
    };

    const int nstage = (NG + KK - 1) / KK;
    for (int i = tid; i < 2 * KK * BN; i += GEO::NT) Gs[i] = 0.f;
    load(0);
    if (logscale) {
        float top = 0.f, nbot = -__builtin_inff();   // the largest and minus the smallest output this lane loaded
#pragma unroll
        for (int i = 0; i < RowLoad::N; i++)
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const float ov = ok_.v[i][c];
                if (ov > 0.f && ov < __builtin_inff()) {   // padding is 0; a NaN is not taken either
                    top = __builtin_fmaxf(top, ov);
                    nbot = __builtin_fmaxf(nbot, -ov);
                }
            }
        top = wave_max(top);
        nbot = wave_max(nbot);
        constexpr int NW = GEO::NT / 64;
        float* tops = Gs;   // zero again before the loop below uses it
        __syncthreads();    // the zero fill above is complete
        if ((tid & 63) == 63) { tops[tid >> 6] = top; tops[NW + (tid >> 6)] = nbot; }
        __syncthreads();
#pragma unroll
        for (int w = 0; w < NW; w++) {
            top = __builtin_fmaxf(w == 0 ? tops[0] : top, tops[w]);
            nbot = __builtin_fmaxf(w == 0 ? tops[NW] : nbot, tops[NW + w]);
        }
        __syncthreads();
        if ((tid & 63) == 63) { tops[tid >> 6] = 0.f; tops[NW + (tid >> 6)] = 0.f; }
        // the power of two nearest (as a ratio) to the geometric mean of the two, so that the window of the vote
        // reaches as far below the smallest as above the largest; kept well inside the float range; 2^-exponent by
        // its bits
        const float mid = __builtin_sqrtf(top) * __builtin_sqrtf(-nbot) * 1.41421356f;
        const int ex = min(100, max(-100, (int)((__float_as_uint(mid) >> 23) & 0xff) - 127));
        unit_inv = top > 0.f ? __uint_as_float((unsigned)(127 - ex) << 23) : 1.0f;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) q[i][j] *= unit_inv;
    }
    bool factored = false;   // the stage in LDS takes the short form (IE > 0: factored; IE == 0: logarithmic)
    if (IE > 0 || logscale) factored = !__syncthreads_or(out_of_range());
    convert(factored);
    scale_weights();
    store();
    __syncthreads();
    for (int s = 0; s < nstage; s++) {
        if (s + 1 < nstage) load((s + 1) * KK);
        const float* fp = lds + grp * kChunk * GEO::SM;
        const float* wp = lds + 2 * XS + grp * kChunk * GEO::SN;
        // No operand prefetch: a second fragment in flight does not fit next to the patch, the sums and the weight
        // row's partial sums (it spills, and measured 15 % slower); the LDS latency of a row hides behind the forty
        // logarithms and exponentials of the other wave on the SIMD.
        if constexpr (IE > 0) {
            if (factored) {
                sweep_chunk_plain<GEO, 1>(fp, wp, tx, ty, [&](const Frag<GEO, 1, 1>& f, int kk) {
                    float sum[TN];
#pragma unroll
                    for (int j = 0; j < TN; j++) sum[j] = 0.f;
#pragma unroll
                    for (int i = 0; i < TM; i++)
#pragma unroll
                        for (int j = 0; j < TN; j++) {
                            const float sp = spower(q[i][j] - f.w[0][j]);
                            acc[i][j] = __builtin_fmaf(f.x[0][0][i], sp, acc[i][j]);
                            sum[j] = __builtin_fmaf(f.x[0][0][i], sp, sum[j]);
                        }
                    add_weight_row(grp * kChunk + kk, sum);
                });
            } else {
                sweep_chunk_plain<GEO, 2>(fp, wp, tx, ty, [&](const Frag<GEO, 2, 1>& f, int kk) {
                    float sum[TN];
#pragma unroll
                    for (int j = 0; j < TN; j++) sum[j] = 0.f;
#pragma unroll
                    for (int i = 0; i < TM; i++)
#pragma unroll
                        for (int j = 0; j < TN; j++) {
                            const float sp = spower((q[i][j] - f.w[0][j]) * f.x[1][0][i]);
                            acc[i][j] = __builtin_fmaf(f.x[0][0][i], sp, acc[i][j]);
                            sum[j] = __builtin_fmaf(f.x[0][0][i], sp, sum[j]);
                        }
                    add_weight_row(grp * kChunk + kk, sum);
                });
            }
        } else if (sparse) {
            // Large exponents: |u|^(p-1) <= 2^-36 for |u| <= cut, less than the rounding of one term of unit size, and
            // nearly every normalised difference is that small, while the logarithm and the exponential are most of
            // a term's cost.  One row of the lane's patch at a time (TN terms that share g and 1/out): when no lane
            // of the wave has |x - w| / out above the cut, the wave passes over the row for both sums; a step whose
            // rows are all passed over adds nothing to grad_weight either.  All tests of a step come before the
            // first branch, so the branches wait for scalar registers only.
            sweep_chunk_plain<GEO, 2>(fp, wp, tx, ty, [&](const Frag<GEO, 2, 1>& f, int kk) {
                unsigned long long hot[TM], any = 0;
#pragma unroll
                for (int i = 0; i < TM; i++) {
                    float top = 0.f;
#pragma unroll
                    for (int j = 0; j < TN; j++) top = __builtin_fmaxf(top, __builtin_fabsf(q[i][j] - f.w[0][j]));
                    hot[i] = __builtin_amdgcn_ballot_w64(top * f.x[1][0][i] > cut);
                    any |= hot[i];
                }
                if (any == 0) return;
                float sum[TN];
#pragma unroll
                for (int j = 0; j < TN; j++) sum[j] = 0.f;
#pragma unroll
                for (int i = 0; i < TM; i++) {
                    if (hot[i] == 0) continue;
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        const float sp = spower((q[i][j] - f.w[0][j]) * f.x[1][0][i]);
                        acc[i][j] = __builtin_fmaf(f.x[0][0][i], sp, acc[i][j]);
                        sum[j] = __builtin_fmaf(f.x[0][0][i], sp, sum[j]);
                    }
                }
                add_weight_row(grp * kChunk + kk, sum);
            });
        } else if (factored) {
            sweep_chunk_plain<GEO, 2>(fp, wp, tx, ty, [&](const Frag<GEO, 2, 1>& f, int kk) {
                float sum[TN];
#pragma unroll
                for (int j = 0; j < TN; j++) sum[j] = 0.f;
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        const float df = q[i][j] - f.w[0][j];
                        const float sp = df * __builtin_amdgcn_exp2f(__builtin_fmaf(__builtin_amdgcn_logf(__builtin_fabsf(df)), em2, f.x[1][0][i]));
                        acc[i][j] = __builtin_fmaf(f.x[0][0][i], sp, acc[i][j]);   // two fused multiply-adds, not a
                        sum[j] = __builtin_fmaf(f.x[0][0][i], sp, sum[j]);         // shared product and two additions
                    }
                add_weight_row(grp * kChunk + kk, sum);
            });
        } else {
            sweep_chunk_plain<GEO, 2>(fp, wp, tx, ty, [&](const Frag<GEO, 2, 1>& f, int kk) {
                float sum[TN];
#pragma unroll
                for (int j = 0; j < TN; j++) sum[j] = 0.f;
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        const float sp = spower((q[i][j] - f.w[0][j]) * f.x[1][0][i]);
                        acc[i][j] = __builtin_fmaf(f.x[0][0][i], sp, acc[i][j]);
                        sum[j] = __builtin_fmaf(f.x[0][0][i], sp, sum[j]);
                    }
                add_weight_row(grp * kChunk + kk, sum);
            });
        }
        // everyone is done reading the panels and the stage's grad_weight tile is complete; the vote on the next
        // stage's outputs rides on the same barrier
        if (IE > 0 || logscale) factored = !__syncthreads_or(s + 1 < nstage ? out_of_range() : false);
        else __syncthreads();
        flush_weight_tile(s * KK);
        if (s + 1 < nstage) {
            convert(factored);
            scale_weights();
            store();
        }
        __syncthreads();
    }

    // ---- the k-groups add their grad_input sums through LDS, the first one writes the tile ----
    float* part = lds;
#pragma unroll 1
    for (int turn = KS - 1; turn >= 1; turn--) {
        if (grp == turn) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) part[(i * TN + j) * NGRP + t] = acc[i][j];
        }
        __syncthreads();
        if (grp == 0) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) acc[i][j] += part[(i * TN + j) * NGRP + t];
        }
        __syncthreads();
    }
    if (grp == 0) {
        Dims od = d;
        od.NG = K;   // the result has the input's shape: K columns per group
        store_patch<GEO, false>(grad_input, acc, od, m0, k0, g, tx, ty, d.ovec != 0);
    }
}

template <class GEO, int IE>
static hipError_t launch_fused(const Problem& pr, hipStream_t stream, const float* grad_output, const float* input,
                               const float* weight, const float* output, float* grad_input, float* grad_weight, float p) {
    Dims d = make_dims(pr);
    d.ovec = 1;   // the result has the input's shape: K % 4 == 0, aligned
    d.tiles_m = (d.M + GEO::BM - 1) / GEO::BM;
    d.tiles_n = (d.K + GEO::BN - 1) / GEO::BN;
    const unsigned grid = (unsigned)d.tiles_m * d.tiles_n * d.G;
    constexpr size_t lds = (size_t)(2 * GEO::XS + GEO::WS + 2 * GEO::KK * GEO::BN) * sizeof(float);   // panels, the two grad_weight tiles
    auto kern = norm_backward_fused_kernel<GEO, IE>;
    static LdsRecord lds_allowed = {};
    if (hipError_t e = allow_lds(kern, lds, pr.device, lds_allowed); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(GEO::NT), lds, stream, grad_output, input, weight, output, grad_input,
                       grad_weight, p - 1.0f, d);
    return hipGetLastError();
}

// Exponents p - 1 for which the one-pass kernel has a multiply-only instantiation.
static int fused_int_power(float p) {
    const int ie = small_int_power(p - 1.0f);
    return (ie == 1 || ie == 2 || ie == 3 || ie == 7) ? ie : 0;
}

// Whether the one-pass kernel takes the problem: the fc layout, every panel loadable with 128-bit loads, and a shape
// that fills the device with 128-row tiles (the rest stays with the two separate kernels).
bool norm_backward_fused_applicable(const Problem& pr, float p, const void* grad_output, const void* input,
                                    const void* weight, const void* output, const void* grad_input,
                                    const void* grad_weight) {
    if (fused_int_power(p) == 0 && !(p > 2.0f)) return false;   // the general kernel takes sign(u) |u|^(p-1) as u |u|^(p-2)
    if (pr.HW != 1 || pr.K % 4 != 0 || pr.NG % 4 != 0) return false;
    // a lane addresses its vectors by 32-bit byte offsets from its tile's first row: 128 rows of G * NG elements of g
    // and out, 64 rows of K weights
    if (4LL * 130 * pr.G * pr.NG >= (1LL << 31) || 4LL * 66 * pr.K >= (1LL << 31)) return false;
    if (!(aligned16(grad_output) && aligned16(input) && aligned16(weight) && aligned16(output) && aligned16(grad_input) &&
          aligned16(grad_weight)))
        return false;
    if (g_tile_override == 0 || g_tile_override == 1 || g_tile_override == 5) return true;   // tests and tuning: forced on (128 x 80, 128 x 64, 128 x 48)
    if (g_tile_override >= 2) return false;                          // forced off
    // p = 2: a term is one instruction and sharing it saves less than the row sums of grad_weight cost (512 x 5120 ->
    // 5120: 1.44 against 1.42 ms).  p = 3: 1.65 against 1.83 ms where the tiles fill the device (10240 inputs: 3.30
    // against 3.71 ms), a tie at 192 tiles of 256 (3072 inputs), a loss at 128.  p = 4: 1.88 against 2.22 ms, p = 8:
    // 2.27 against 3.06 ms.
    const int ie = fused_int_power(p);
    if (ie == 1) return false;
    const long M = (long)pr.B * pr.HW;
    const long t48 = ((M + 127) / 128) * ((pr.K + 47) / 48) * pr.G;   // the narrowest tiles: the most workgroups
    return t48 * 10 >= (ie == 2 ? 9L : 7L) * pr.num_cu && pr.NG >= 256;
}

template <class GEO>
static hipError_t launch_fused_for(const Problem& pr, hipStream_t stream, const float* grad_output, const float* input,
                                   const float* weight, const float* output, float* grad_input, float* grad_weight,
                                   float p) {
    switch (fused_int_power(p)) {
        case 1: return launch_fused<GEO, 1>(pr, stream, grad_output, input, weight, output, grad_input, grad_weight, p);
        case 2: return launch_fused<GEO, 2>(pr, stream, grad_output, input, weight, output, grad_input, grad_weight, p);
        case 3: return launch_fused<GEO, 3>(pr, stream, grad_output, input, weight, output, grad_input, grad_weight, p);
        case 7: return launch_fused<GEO, 7>(pr, stream, grad_output, input, weight, output, grad_input, grad_weight, p);
        default: return launch_fused<GEO, 0>(pr, stream, grad_output, input, weight, output, grad_input, grad_weight, p);
    }
}

hipError_t norm_backward_fused(const float* grad_output, const float* input, const float* weight, const float* output,
                               float* grad_input, float* grad_weight, float p, const Problem& pr, hipStream_t stream) {
    const long rows = (long)pr.B * pr.HW;
    // Rounds of workgroups (one per CU) times columns per tile, the narrower tiles charged for what a term costs more
    // in them (more LDS words and cross-lane steps per term).  3072 inputs at batch 512: 156 tiles of 80 columns, 192
    // of 64 or 256 of 48 -- only the last fill the 256 CUs.
    const long rt = (rows + 127) / 128;
    const long t80 = rt * ((pr.K + 79) / 80) * pr.G, t64 = rt * ((pr.K + 63) / 64) * pr.G, t48 = rt * ((pr.K + 47) / 48) * pr.G;
    const double c80 = (double)((t80 + pr.num_cu - 1) / pr.num_cu) * 80, c64 = (double)((t64 + pr.num_cu - 1) / pr.num_cu) * 64 * 1.1,
                 c48 = (double)((t48 + pr.num_cu - 1) / pr.num_cu) * 48 * 1.2;
    if (g_tile_override == 0 || (g_tile_override != 1 && g_tile_override != 5 && c80 <= c64 && c80 <= c48))
        return launch_fused_for<Geo<128, 80, 8, 5, 2>>(pr, stream, grad_output, input, weight, output, grad_input, grad_weight, p);
    if (g_tile_override == 1 || (g_tile_override != 5 && c64 <= c48))
        return launch_fused_for<Geo<128, 64, 8, 4, 2>>(pr, stream, grad_output, input, weight, output, grad_input, grad_weight, p);
    return launch_fused_for<Geo<128, 48, 8, 3, 2>>(pr, stream, grad_output, input, weight, output, grad_input, grad_weight, p);
}

}  // namespace ldist
