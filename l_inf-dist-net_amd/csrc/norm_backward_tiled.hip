// p-norm distance backward with respect to the input for p = 2, 3, 4, 8 on the register-tiled engine of the
// forward kernels (reference model/norm_dist_cuda.cu:294-361):
//   grad_input[m,k] = sum_n g[m,n] * (|x[m,k] - w[n,k]| / out[m,n])^(p-1) * sign(x - w).
// A workgroup owns a BM x BN tile of the (row m, input k) plane of one group and walks the outputs n in stages
// of KS*32.  A lane keeps its TM x TN patch of x and of the sums in registers; per n it reads the TM row values
// F[m,n] = g[m,n] / out[m,n]^(p-1) and the TN weights w[n,k] with 128-bit LDS loads, so every value fetched from
// LDS is reused TN (TM) times, and a term costs the subtraction, the multiplications of the power and one fused
// multiply-add:  sum += F * (x - w)^(p-1)  (odd exponents keep the sign by themselves, even ones take one factor
// as |x - w|).  Taking the power of the raw difference needs (x-w)^(p-1) and out^-(p-1) inside the float range:
// every stage checks the outputs it loads, and a stage that holds one outside [2^-12, 2^12] is reduced the
// careful way, g * ((x - w) / out)^(p-1), from the g and 1/out panels (a lean rolled loop, seldom taken).
#include "fwd_engine.hpp"
#include "pow.hpp"

namespace ldist {

// IE = p - 1 (1, 2, 3 or 7).  d.K is the number of inputs per group (the tile's columns), d.NG the outputs per
// group (the reduction), d.tiles_n counts column tiles.
template <class GEO, bool CONV, int IE>
__global__ void __launch_bounds__(GEO::NT, 2)
norm_backward_input_tiled_kernel(const float* __restrict__ grad_output, const float* __restrict__ input,
                                 const float* __restrict__ weight, const float* __restrict__ output,
                                 float* __restrict__ grad_input, Dims d) {
    constexpr int BM = GEO::BM, BN = GEO::BN, TM = GEO::TM, TN = GEO::TN, KS = GEO::KS, KK = GEO::KK;
    constexpr int NGRP = GEO::NGRP, NT = GEO::NT, XS = GEO::XS, WS = GEO::WS;
    constexpr int STAGE = 2 * XS + WS;     // [F or g][1/out][w]
    using RowLoadK = RowsK<BM, GEO::SM, NT, KK, 4>;   // fc: outputs are contiguous in g and out
    using RowLoadM = RowsM<BM, GEO::SM, NT, KK, 4>;   // conv: rows are
    using ColLoad = RowsT<BN, GEO::SN, NT, KK, 4>;
    static_assert((KS - 1) * TM * TN * NGRP <= STAGE, "merge area fits in the panels");
    extern __shared__ __align__(16) float lds[];

    int tm, tk, g;
    tile_of_block(d, tm, tk, g);
    const int m0 = tm * BM, k0 = tk * BN;
    const int tid = threadIdx.x;
    const int grp = tid / NGRP, t = tid % NGRP;
    const int tx = t % GEO::TX, ty = t / GEO::TX;
    const int K = d.K, NG = d.NG;

    auto spower = [](float u) {   // sign(u) * |u|^IE
        if constexpr (IE == 1) return u;
        else if constexpr (IE == 2) return u * __builtin_fabsf(u);
        else return pow_int<IE>(u);
    };

    // the lane's patch of x
    float q[TM][TN], acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int m = m0 + GEO::row(ty, i);
        const RowAddr<CONV> ra(Dims{d.B, d.G, K, K, d.HW, d.M, 0, 0, 0, 0, 0}, m < d.M ? m : 0, g);
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int k = k0 + GEO::col(tx, j);
            acc[i][j] = 0.f;
            q[i][j] = (m < d.M && k < K) ? input[ra.x + (size_t)k * ra.xk] : 0.f;
        }
    }

    // ---- staging: g and out (same layout: rows m, reduction n) and the weights of the stage's outputs ----
    RowLoadK gk, ok_;
    RowLoadM gm, om;
    ColLoad wl;
    int off_m[RowLoadM::N];
    const float* gbase = CONV ? grad_output : grad_output + ((size_t)m0 * d.G + g) * NG;
    const float* obase = CONV ? output : output + ((size_t)m0 * d.G + g) * NG;
    const float* wbase = weight + (size_t)g * NG * K;
    if constexpr (CONV) RowLoadM::offsets(off_m, m0, d.M, d.HW, d.G, g, NG, tid);
    auto load = [&](int n_first) {
        wl.load(wbase, K, n_first, NG, k0, K, tid);
        if constexpr (CONV) {
            gm.load(grad_output, off_m, d.HW, n_first, NG, tid);
            om.load(output, off_m, d.HW, n_first, NG, tid);
        } else {
            gk.load(gbase, d.G * NG, d.M - m0, n_first, NG, tid);
            ok_.load(obase, d.G * NG, d.M - m0, n_first, NG, tid);
        }
    };
    // Turns the parked g / out values into what the panels hold: 1/out (0 where nothing was loaded, so that the
    // careful form multiplies by 0 instead of by an infinity), and g or g / out^IE.  Returns whether an output
    // outside the range of the factored form was seen (before the conversion).
    auto convert = [&](bool factored_known, bool factored) {
        bool unsafe = false;
        auto one = [&](float& gv, float& ov) {
            const bool present = ov != 0.f || gv != 0.f;    // padding loads both as 0; a real 0 output gives inf like the reference
            if (!factored_known) {
                if (present) unsafe |= !(ov >= 0x1p-12f && ov <= 0x1p12f);
                return;
            }
            const float ri = present ? __builtin_amdgcn_rcpf(ov) : 0.f;
            ov = ri;
            if (factored) gv = gv * pow_int<IE>(ri);
        };
        if constexpr (CONV) {
#pragma unroll
            for (int i = 0; i < RowLoadM::N; i++)
#pragma unroll
                for (int e = 0; e < 4; e++) one(gm.v[i][e], om.v[i][e]);
        } else {
#pragma unroll
            for (int i = 0; i < RowLoadK::N; i++)
#pragma unroll
                for (int e = 0; e < 4; e++) one(gk.v[i][e], ok_.v[i][e]);
        }
        return unsafe;
    };
    auto store = [&]() {
        if constexpr (CONV) { gm.store(lds, tid); om.store(lds + XS, tid); }
        else { gk.store(lds, tid); ok_.store(lds + XS, tid); }
        wl.store(lds + 2 * XS, tid);
    };

    const int nstage = (NG + KK - 1) / KK;
    load(0);
    bool factored = !__syncthreads_or(convert(false, false));
    convert(true, factored);
    store();
    __syncthreads();
    for (int s = 0; s < nstage; s++) {
        if (s + 1 < nstage) load((s + 1) * KK);
        const float* fp = lds + grp * kChunk * GEO::SM;
        const float* wp = lds + 2 * XS + grp * kChunk * GEO::SN;
        if (factored) {
            sweep_chunk<GEO, 1, 2>(fp, wp, tx, ty, [&](const Frag<GEO, 1, 2>& f, int) {
#pragma unroll
                for (int e = 0; e < 2; e++)
#pragma unroll
                    for (int i = 0; i < TM; i++)
#pragma unroll
                        for (int j = 0; j < TN; j++) acc[i][j] += f.x[0][e][i] * spower(q[i][j] - f.w[e][j]);
            });
        } else {
            sweep_chunk_plain<GEO, 2>(fp, wp, tx, ty, [&](const Frag<GEO, 2, 1>& f, int) {
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) acc[i][j] += f.x[0][0][i] * spower((q[i][j] - f.w[0][j]) * f.x[1][0][i]);
            });
        }
        // everyone is done reading the panels; the vote on the next stage's outputs rides on the same barrier
        const bool next_unsafe = __syncthreads_or(s + 1 < nstage ? convert(false, false) : false);
        if (s + 1 < nstage) {
            factored = !next_unsafe;
            convert(true, factored);
            store();
        }
        __syncthreads();
    }

    // ---- the k-groups add their sums through LDS, the first one writes the tile ----
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
        store_patch<GEO, CONV>(grad_input, acc, od, m0, k0, g, tx, ty, d.ovec != 0);
    }
}

// grad_weight in the fc layout (reference model/norm_dist_cuda.cu:363-425), same scheme with the roles exchanged:
//   grad_weight[n,k] += sum_m g[m,n] * (|w[n,k] - x[m,k]| / out[m,n])^(p-1) * sign(w - x).
// Tile rows are the outputs n, columns the inputs k, the reduction walks the batch rows m; the lane's patch holds
// w, the row panel F[m,n] (n contiguous in g and out: no transpose), the column panel x[m,k].  Every element of
// the gradient belongs to one workgroup, which adds its sum onto the buffer (the caller zero-fills it, as the
// reference asks).
template <class GEO, int IE>
__global__ void __launch_bounds__(GEO::NT, 2)
norm_backward_weight_tiled_kernel(const float* __restrict__ grad_output, const float* __restrict__ input,
                                  const float* __restrict__ weight, const float* __restrict__ output,
                                  float* __restrict__ grad_weight, Dims d) {
    constexpr int BM = GEO::BM, BN = GEO::BN, TM = GEO::TM, TN = GEO::TN, KS = GEO::KS, KK = GEO::KK;
    constexpr int NGRP = GEO::NGRP, NT = GEO::NT, XS = GEO::XS, WS = GEO::WS;
    constexpr int STAGE = 2 * XS + WS;     // [F or g][1/out][x]
    using RowLoad = RowsM<BM, GEO::SM, NT, KK, 4>;
    using ColLoad = RowsT<BN, GEO::SN, NT, KK, 4>;
    static_assert((KS - 1) * TM * TN * NGRP <= STAGE, "merge area fits in the panels");
    extern __shared__ __align__(16) float lds[];

    int tn, tk, g;
    tile_of_block(d, tn, tk, g);            // d.tiles_m counts tiles of outputs, d.tiles_n tiles of inputs
    const int n0 = tn * BM, k0 = tk * BN;
    const int tid = threadIdx.x;
    const int grp = tid / NGRP, t = tid % NGRP;
    const int tx = t % GEO::TX, ty = t / GEO::TX;
    const int K = d.K, NG = d.NG, M = d.M;

    auto spower = [](float u) {   // sign(u) * |u|^IE
        if constexpr (IE == 1) return u;
        else if constexpr (IE == 2) return u * __builtin_fabsf(u);
        else return pow_int<IE>(u);
    };

    float q[TM][TN], acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int n = n0 + GEO::row(ty, i);
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int k = k0 + GEO::col(tx, j);
            acc[i][j] = 0.f;
            q[i][j] = (n < NG && k < K) ? weight[((size_t)g * NG + n) * K + k] : 0.f;
        }
    }

    RowLoad gl, ol;
    ColLoad xl;
    int off_n[RowLoad::N];
#pragma unroll
    for (int i = 0; i < RowLoad::N; i++) {
        const int n = n0 + ((tid + i * NT) % RowLoad::PER_K) * 4;
        off_n[i] = n < NG ? g * NG + n : -1;   // NG % 4 == 0: a group of four outputs is whole or absent
    }
    const float* xbase = input + (size_t)g * K;
    auto load = [&](int m_first) {
        xl.load(xbase, d.G * K, m_first, M, k0, K, tid);
        gl.load(grad_output, off_n, d.G * NG, m_first, M, tid);
        ol.load(output, off_n, d.G * NG, m_first, M, tid);
    };
    auto convert = [&](bool factored_known, bool factored) {   // as in the grad_input kernel
        bool unsafe = false;
#pragma unroll
        for (int i = 0; i < RowLoad::N; i++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                float& gv = gl.v[i][e];
                float& ov = ol.v[i][e];
                const bool present = ov != 0.f || gv != 0.f;
                if (!factored_known) {
                    if (present) unsafe |= !(ov >= 0x1p-12f && ov <= 0x1p12f);
                    continue;
                }
                const float ri = present ? __builtin_amdgcn_rcpf(ov) : 0.f;
                ov = ri;
                if (factored) gv = gv * pow_int<IE>(ri);
            }
        return unsafe;
    };
    auto store = [&]() {
        gl.store(lds, tid);
        ol.store(lds + XS, tid);
        xl.store(lds + 2 * XS, tid);
    };

    const int nstage = (M + KK - 1) / KK;
    load(0);
    bool factored = !__syncthreads_or(convert(false, false));
    convert(true, factored);
    store();
    __syncthreads();
    for (int s = 0; s < nstage; s++) {
        if (s + 1 < nstage) load((s + 1) * KK);
        const float* fp = lds + grp * kChunk * GEO::SM;
        const float* xp = lds + 2 * XS + grp * kChunk * GEO::SN;
        if (factored) {
            sweep_chunk<GEO, 1, 2>(fp, xp, tx, ty, [&](const Frag<GEO, 1, 2>& f, int) {
#pragma unroll
                for (int e = 0; e < 2; e++)
#pragma unroll
                    for (int i = 0; i < TM; i++)
#pragma unroll
                        for (int j = 0; j < TN; j++) acc[i][j] += f.x[0][e][i] * spower(q[i][j] - f.w[e][j]);
            });
        } else {
            sweep_chunk_plain<GEO, 2>(fp, xp, tx, ty, [&](const Frag<GEO, 2, 1>& f, int) {
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) acc[i][j] += f.x[0][0][i] * spower((q[i][j] - f.w[0][j]) * f.x[1][0][i]);
            });
        }
        const bool next_unsafe = __syncthreads_or(s + 1 < nstage ? convert(false, false) : false);
        if (s + 1 < nstage) {
            factored = !next_unsafe;
            convert(true, factored);
            store();
        }
        __syncthreads();
    }

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
#pragma unroll
        for (int i = 0; i < TM; i++) {
            const int n = n0 + GEO::row(ty, i);
            if (n >= NG) continue;
            float* row = grad_weight + ((size_t)g * NG + n) * K;
#pragma unroll
            for (int r = 0; r < TN / 4; r++) {      // the lane's columns come in groups of four: K % 4 == 0, 16-byte aligned
                const int k = k0 + GEO::col(tx, 4 * r);
                if (k < K) {
                    float4 v = *reinterpret_cast<float4*>(row + k);
                    v.x += acc[i][4 * r]; v.y += acc[i][4 * r + 1]; v.z += acc[i][4 * r + 2]; v.w += acc[i][4 * r + 3];
                    *reinterpret_cast<float4*>(row + k) = v;
                }
            }
#pragma unroll
            for (int j = TN / 4 * 4; j < TN; j++) {
                const int k = k0 + GEO::col(tx, j);
                if (k < K) row[k] += acc[i][j];
            }
        }
    }
}

template <class GEO, bool CONV, int IE>
static hipError_t launch_nbi(const Problem& pr, bool ovec, hipStream_t stream, const float* grad_output, const float* input,
                             const float* weight, const float* output, float* grad_input) {
    Dims d = make_dims(pr);
    d.ovec = ovec;
    d.tiles_m = (d.M + GEO::BM - 1) / GEO::BM;
    d.tiles_n = (d.K + GEO::BN - 1) / GEO::BN;
    const unsigned grid = (unsigned)d.tiles_m * d.tiles_n * d.G;
    constexpr size_t lds = (size_t)(2 * GEO::XS + GEO::WS) * sizeof(float);
    if (!CONV) d.m_block = choose_m_block(d.tiles_m, 2 * GEO::BM, GEO::BN, resident_per_xcd(GEO::NT, lds, pr.num_cu));
    auto kern = norm_backward_input_tiled_kernel<GEO, CONV, IE>;
    static LdsRecord lds_allowed = {};
    if (hipError_t e = allow_lds(kern, lds, pr.device, lds_allowed); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(GEO::NT), lds, stream, grad_output, input, weight, output, grad_input, d);
    return hipGetLastError();
}

template <class GEO, int IE>
static hipError_t launch_nbw(const Problem& pr, hipStream_t stream, const float* grad_output, const float* input,
                             const float* weight, const float* output, float* grad_weight) {
    Dims d = make_dims(pr);
    d.tiles_m = (d.NG + GEO::BM - 1) / GEO::BM;
    d.tiles_n = (d.K + GEO::BN - 1) / GEO::BN;
    const unsigned grid = (unsigned)d.tiles_m * d.tiles_n * d.G;
    constexpr size_t lds = (size_t)(2 * GEO::XS + GEO::WS) * sizeof(float);
    // A tile of outputs streams two panels over all rows (grad_output, output), a tile of inputs one: walked with
    // all output tiles before the next input tile, the workgroups that share an L2 read their own two panels each
    // (40 output tiles of 0.5 MB on a 5120-wide layer); in blocks they share both kinds of panel.
    d.m_block = choose_m_block(d.tiles_m, 2 * GEO::BM, GEO::BN, resident_per_xcd(GEO::NT, lds, pr.num_cu));
    auto kern = norm_backward_weight_tiled_kernel<GEO, IE>;
    static LdsRecord lds_allowed = {};
    if (hipError_t e = allow_lds(kern, lds, pr.device, lds_allowed); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(GEO::NT), lds, stream, grad_output, input, weight, output, grad_weight, d);
    return hipGetLastError();
}

static bool tiled_common(const Problem& pr, float p, const void* a, const void* b, const void* c, const void* e, const void* f) {
    const int ie = small_int_power(p - 1.0f);
    if (!(ie == 1 || ie == 2 || ie == 3 || ie == 7)) return false;
    if (pr.K % 4 != 0 || (pr.HW == 1 ? pr.NG % 4 != 0 : pr.HW % 4 != 0)) return false;
    return aligned16(a) && aligned16(b) && aligned16(c) && aligned16(e) && aligned16(f);
}

// tiles of 128 rows x 80 or 64 columns: the shape that leaves the fewest idle columns per round of workgroups
static bool wide_tiles(long rows, long cols, int G, int num_cu) {
    const long t80 = ((rows + 127) / 128) * ((cols + 79) / 80) * G, t64 = ((rows + 127) / 128) * ((cols + 63) / 64) * G;
    const double c80 = (double)((t80 + num_cu - 1) / num_cu) * 80, c64 = (double)((t64 + num_cu - 1) / num_cu) * 64 * 1.1;
    return g_tile_override == 0 || (g_tile_override != 1 && c80 <= c64);
}

// Whether the tiled kernel takes the problem: a multiply-only exponent, every panel loadable with 128-bit loads,
// and enough tiles to keep the device busy (small problems stay on the 64 x 64 kernel, which makes more workgroups).
bool norm_backward_input_tiled_applicable(const Problem& pr, float p, const void* grad_output, const void* input,
                                          const void* weight, const void* output, const void* grad_input) {
    if (!tiled_common(pr, p, grad_output, input, weight, output, grad_input)) return false;
    if (g_tile_override == 0 || g_tile_override == 1) return true;   // tests and tuning: forced on (128 x 80, 128 x 64)
    if (g_tile_override >= 2) return false;                          // forced off
    const long M = (long)pr.B * pr.HW;
    const long t80 = ((M + 127) / 128) * ((pr.K + 79) / 80) * pr.G, t64 = ((M + 127) / 128) * ((pr.K + 63) / 64) * pr.G;
    return (t80 > t64 ? t80 : t64) * 10 >= 7L * pr.num_cu && pr.NG >= 256;
}

// grad_weight: the fc layout only (in the conv layout the reduction walks positions and images).
bool norm_backward_weight_tiled_applicable(const Problem& pr, float p, const void* grad_output, const void* input,
                                           const void* weight, const void* output, const void* grad_weight) {
    if (pr.HW != 1 || !tiled_common(pr, p, grad_output, input, weight, output, grad_weight)) return false;
    if (g_tile_override == 0 || g_tile_override == 1) return true;
    if (g_tile_override >= 2) return false;
    const long t64 = (((long)pr.NG + 127) / 128) * ((pr.K + 63) / 64) * pr.G;
    return t64 >= pr.num_cu && pr.B >= 256;   // fewer tiles: the 64 x 64 kernel shares the rows out over workgroups
}

#define LDIST_TILED_SWITCH(CALL)  \
    switch (ie) {                 \
        case 1: CALL(1);          \
        case 2: CALL(2);          \
        case 3: CALL(3);          \
        case 7: CALL(7);          \
        default: return hipErrorInvalidValue;   /* the applicable() test said no */ \
    }

hipError_t norm_backward_input_tiled(const float* grad_output, const float* input, const float* weight,
                                     const float* output, float* grad_input, float p, const Problem& pr,
                                     hipStream_t stream) {
    const int ie = small_int_power(p - 1.0f);
    const bool conv = pr.HW != 1;
    const bool ovec = true;   // the result has the input's shape: K % 4 == 0 (fc), HW % 4 == 0 (conv), aligned
    const bool wide = wide_tiles((long)pr.B * pr.HW, pr.K, pr.G, pr.num_cu);
#define LDIST_NBI(IE)                                                                                                     \
    if (wide)                                                                                                             \
        return conv ? launch_nbi<Geo<128, 80, 8, 5, 2>, true, IE>(pr, ovec, stream, grad_output, input, weight, output, grad_input)   \
                    : launch_nbi<Geo<128, 80, 8, 5, 2>, false, IE>(pr, ovec, stream, grad_output, input, weight, output, grad_input); \
    return conv ? launch_nbi<Geo<128, 64, 8, 4, 2>, true, IE>(pr, ovec, stream, grad_output, input, weight, output, grad_input)       \
                : launch_nbi<Geo<128, 64, 8, 4, 2>, false, IE>(pr, ovec, stream, grad_output, input, weight, output, grad_input)
    LDIST_TILED_SWITCH(LDIST_NBI)
#undef LDIST_NBI
}

hipError_t norm_backward_weight_tiled(const float* grad_output, const float* input, const float* weight,
                                      const float* output, float* grad_weight, float p, const Problem& pr,
                                      hipStream_t stream) {
    const int ie = small_int_power(p - 1.0f);
    const bool wide = wide_tiles(pr.NG, pr.K, pr.G, pr.num_cu);
#define LDIST_NBW(IE)                                                                                                  \
    if (wide) return launch_nbw<Geo<128, 80, 8, 5, 2>, IE>(pr, stream, grad_output, input, weight, output, grad_weight); \
    return launch_nbw<Geo<128, 64, 8, 4, 2>, IE>(pr, stream, grad_output, input, weight, output, grad_weight)
    LDIST_TILED_SWITCH(LDIST_NBW)
#undef LDIST_NBW
}

}  // namespace ldist
